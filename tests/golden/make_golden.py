"""Writes tests/golden/*.npz: inputs and the outputs the REFERENCE's own host code gives for them.

Run in the build container only (it needs oracle/_ref/libbfaintb_ref.so, which is compiled from the
reference's headers where they lie under /root/reference; see oracle/Makefile target `ref`):

    make -C oracle ref && python tests/golden/make_golden.py

The fixtures hold data only.  Inputs come from numpy's PCG64 generator with the seeds below, so
they can be regenerated anywhere; the expected outputs come from the reference's gemm_rrr
(host_ref.hpp:3-25), type_convert / bf16_convert_rtn (datatype.hpp:31-55, 80-121),
mem_transfer<int8_t,float> (mem_transfer.hpp:23-32) and valid_vector (validation.hpp:7-46).
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))
fp = C.POINTER(C.c_float)
u16p = C.POINTER(C.c_uint16)
u8p = C.POINTER(C.c_uint8)


def ref_gemm(a, b, s):
    r = oracle.ref()
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    s = np.ascontiguousarray(s, np.float32)
    m, k = a.shape
    _, n = b.shape
    c = np.zeros((m, n), np.float32)
    r.ref_gemm_rrr(c.ctypes.data_as(fp), a.ctypes.data_as(fp), b.ctypes.data_as(fp), s.ctypes.data_as(fp), m, n, k, k, n, n)
    return c


def ref_rne(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.zeros(x.shape, np.uint16)
    oracle.ref().ref_f32_to_bf16_rne_n(out.ctypes.data_as(u16p), x.ctypes.data_as(fp), x.size)
    return out


def ref_rtz(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.zeros(x.shape, np.uint16)
    oracle.ref().ref_f32_to_bf16_rtz_n(out.ctypes.data_as(u16p), x.ctypes.data_as(fp), x.size)
    return out


def widen(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def main():
    r = oracle.ref()
    assert r is not None, "build oracle/_ref first (make -C oracle ref)"

    # ---- C1: M=64 K=256 N=128, A ~ N(0,1), q uniform [-128,127], scale uniform [0.001,0.01], seed 0
    rng = np.random.Generator(np.random.PCG64(0))
    m, k, n = 64, 256, 128
    a_f32 = rng.standard_normal((m, k), dtype=np.float32)
    q = rng.integers(-128, 128, size=(k, n), dtype=np.int64).astype(np.int8)
    s_f32 = rng.uniform(0.001, 0.01, size=n).astype(np.float32)
    a_bf = ref_rne(a_f32)                      # activations as the device sees them
    s_bf = ref_rne(s_f32)
    b_bytes = np.zeros((k, n), np.uint8)       # reference wire format via its own mem_transfer
    qf = np.ascontiguousarray(q.astype(np.float32))
    r.ref_mem_transfer_int8(b_bytes.ctypes.data_as(u8p), qf.ctypes.data_as(fp), qf.size)
    w_f32 = q.astype(np.float32) * widen(s_bf)[None, :]          # exact in fp32
    w_bf = ref_rne(w_f32)
    c_rrr = ref_gemm(widen(a_bf), q.astype(np.float32), widen(s_bf))          # unrounded weights (host_ref as called by main)
    c_oracle = ref_gemm(widen(a_bf), widen(w_bf), np.ones(n, np.float32))     # bf16 weights, unit scales
    np.savez_compressed(os.path.join(OUT, "c1_seed0.npz"), a_f32=a_f32, q=q, s_f32=s_f32, a_bf=a_bf, s_bf=s_bf,
                        b_bytes=b_bytes, w_bf=w_bf, c_rrr=c_rrr, c_oracle=c_oracle)

    # ---- the reference's own regime: everything in {-2,-1,0,1} (random_gen.hpp:24,37,50), its default shape
    rng = np.random.Generator(np.random.PCG64(1))
    m, n, k = 32, 128, 512
    a = rng.integers(-2, 2, size=(m, k)).astype(np.float32)
    b = rng.integers(-2, 2, size=(k, n)).astype(np.float32)
    s = rng.integers(-2, 2, size=n).astype(np.float32)
    c = ref_gemm(a, b, s)
    a_dev = np.zeros((m, k), np.uint16)
    r.ref_mem_transfer_bf16(a_dev.ctypes.data_as(u16p), a.ctypes.data_as(fp), a.size)
    b_dev = np.zeros((k, n), np.uint8)
    r.ref_mem_transfer_int8(b_dev.ctypes.data_as(u8p), b.ctypes.data_as(fp), b.size)
    c_bf = ref_rtz(c)  # truncation, as the reference device epilogue does; exact here (small integers)
    ok_exact = int(r.ref_valid_vector_bf16(c.ctypes.data_as(fp), c_bf.ctypes.data_as(u16p), c.size, 1e-3))
    np.savez_compressed(os.path.join(OUT, "int_regime_seed1.npz"), a=a, b=b, s=s, c=c, a_dev=a_dev, b_dev=b_dev,
                        c_bf_trunc=c_bf, valid_exact=np.int32(ok_exact))

    # ---- converter known answers straight from the reference's routines
    special = np.array([0x00000000, 0x80000000, 0x3F800000, 0x3F7FFFFF, 0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF,
                        0x7F7FFFFF, 0x7F800000, 0xFF800000, 0x7F800001, 0x7FC00000, 0x7F80FFFF, 0x00000001, 0x00008000,
                        0x00018000, 0x007FFFFF, 0x00800000, 0xC2F6E979, 0x477FE000, 0x477FFFFF], np.uint32)
    rng = np.random.Generator(np.random.PCG64(2))
    rnd = rng.integers(0, 2**32, size=4096, dtype=np.uint64).astype(np.uint32)
    bits = np.concatenate([special, rnd])
    f = bits.view(np.float32)
    rne = ref_rne(f)
    rtz = ref_rtz(f)
    all16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    back_f = np.zeros(65536, np.float32)
    r.ref_bf16_to_f32_n(back_f.ctypes.data_as(fp), all16.ctypes.data_as(u16p), 65536)
    back = back_f.view(np.uint32)
    codes = np.arange(-128, 128).astype(np.float32)
    code_bytes = np.zeros(256, np.uint8)
    r.ref_mem_transfer_int8(code_bytes.ctypes.data_as(u8p), codes.ctypes.data_as(fp), 256)
    np.savez_compressed(os.path.join(OUT, "converters.npz"), f32_bits=bits, rne=rne, rtz=rtz, bf16_to_f32_bits=back,
                        int8_values=codes, int8_bytes=code_bytes)

    # ---- valid_vector verdicts on hand-built cases
    cases = []
    base = np.array([1.0, 2.0, -3.0, 4.0, 100.0, 0.5], np.float32)
    def verdict(ref_v, pred_bits):
        ref_v = np.ascontiguousarray(ref_v, np.float32)
        pred_bits = np.ascontiguousarray(pred_bits, np.uint16)
        return int(r.ref_valid_vector_bf16(ref_v.ctypes.data_as(fp), pred_bits.ctypes.data_as(u16p), ref_v.size, 1e-3))
    p_exact = ref_rtz(base)
    cases.append((base, p_exact))
    off = base.copy(); off[3] = 4.0 * 1.0078125  # one bf16 step above 4: 0.78 % off
    cases.append((base, ref_rtz(off)))
    z = np.array([0.0, 1.0, 2.0], np.float32)
    cases.append((z, ref_rtz(z)))                                        # zero ref, zero pred
    cases.append((z, ref_rtz(np.array([0.125, 1.0, 2.0], np.float32))))  # zero ref, non-zero pred
    neg = np.array([-4.0, -8.0, 1600.0], np.float32)
    cases.append((neg, ref_rtz(np.array([-4.03125, -8.0, 1600.0], np.float32))))  # negative ref off by 0.78 %: |r-p|/r is negative, so the per-element test lets it pass
    refs = np.zeros((len(cases), 6), np.float32); preds = np.zeros((len(cases), 6), np.uint16); lens = np.zeros(len(cases), np.int32); verd = np.zeros(len(cases), np.int32)
    for i, (rv, pv) in enumerate(cases):
        lens[i] = rv.size; refs[i, :rv.size] = rv; preds[i, :pv.size] = pv; verd[i] = verdict(rv, pv)
    np.savez_compressed(os.path.join(OUT, "valid_vector_cases.npz"), refs=refs, preds=preds, lens=lens, verdicts=verd)
    print("golden fixtures written to", OUT, "verdicts", verd.tolist(), "int-regime valid", ok_exact)


if __name__ == "__main__":
    main()
