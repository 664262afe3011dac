"""Pins the oracle's gemm_rrr restatement and validation logic (CPU only)."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import Problem, ulp_violations, widen

fp = C.POINTER(C.c_float)


def test_golden_c1_from_reference(golden_dir):
    g = np.load(f"{golden_dir}/c1_seed0.npz")
    a = widen(g["a_bf"])
    # the reference's gemm_rrr on (bf16 A, integer q, bf16 scale): what its main() would check against
    c = oracle.gemm_rrr(a, g["q"].astype(np.float32), widen(g["s_bf"]))
    assert np.array_equal(c.view(np.uint32), g["c_rrr"].view(np.uint32))
    assert np.array_equal(oracle.gemm_rrr(a, g["q"].astype(np.float32), widen(g["s_bf"]), fast=True).view(np.uint32),
                          g["c_rrr"].view(np.uint32))
    # the GEMM oracle proper: bf16 dequantised weights, unit scales
    w = oracle.dequant(g["b_bytes"], g["s_bf"], 256, 128, 8, 0)
    assert np.array_equal(w, g["w_bf"])
    assert np.array_equal(oracle.gemm_bf16(g["a_bf"], w).view(np.uint32), g["c_oracle"].view(np.uint32))
    assert np.array_equal(oracle.gemm_bf16_rows(g["a_bf"], w, threads=3).view(np.uint32), g["c_oracle"].view(np.uint32))
    # inputs in the fixture are what the documented generator gives (PCG64 seed 0), so it can be regenerated
    rng = np.random.Generator(np.random.PCG64(0))
    a_f32 = rng.standard_normal((64, 256), dtype=np.float32)
    assert np.array_equal(a_f32, g["a_f32"]) and np.array_equal(oracle.f32_to_bf16_rne(a_f32), g["a_bf"])
    assert np.array_equal(oracle.mem_transfer_int8(g["q"].astype(np.float32)), g["b_bytes"])


def test_golden_int_regime_from_reference(golden_dir):
    g = np.load(f"{golden_dir}/int_regime_seed1.npz")
    c = oracle.gemm_rrr(g["a"], g["b"], g["s"])
    assert np.array_equal(c.view(np.uint32), g["c"].view(np.uint32))
    assert np.array_equal(oracle.f32_to_bf16_rtz(g["a"]), g["a_dev"])
    assert np.array_equal(oracle.mem_transfer_int8(g["b"]), g["b_dev"])
    ok, pp, nr = oracle.valid_vector(g["c"], g["c_bf_trunc"])
    assert ok == bool(g["valid_exact"]) and pp == 0


@pytest.mark.skipif(not oracle.have_ref(), reason="reference wrapper not built (needs /root/reference)")
@pytest.mark.parametrize("m,n,k,lda,ldb,ldc", [(3, 5, 7, 7, 5, 5), (8, 16, 64, 70, 20, 18), (64, 128, 256, 256, 128, 128)])
def test_gemm_rrr_bit_for_bit_against_compiled_reference(m, n, k, lda, ldb, ldc):
    rng = np.random.Generator(np.random.PCG64(m * 1000 + n))
    a = rng.standard_normal((m, lda)).astype(np.float32)
    b = rng.integers(-128, 128, size=(k, ldb)).astype(np.float32)
    s = rng.uniform(0.001, 0.01, size=n).astype(np.float32)
    c_ref = np.full((m, ldc), np.float32(-7), np.float32)
    c_mine = c_ref.copy()
    c_fast = c_ref.copy()
    args = lambda c: (c.ctypes.data_as(fp), a.ctypes.data_as(fp), b.ctypes.data_as(fp), s.ctypes.data_as(fp), m, n, k, lda, ldb, ldc)
    oracle.ref().ref_gemm_rrr(*args(c_ref))
    oracle.lib.orc_gemm_rrr(*args(c_mine))
    oracle.lib.orc_gemm_rrr_fast(*args(c_fast))
    assert np.array_equal(c_ref.view(np.uint32), c_mine.view(np.uint32))
    assert np.array_equal(c_ref.view(np.uint32), c_fast.view(np.uint32))
    assert (c_ref[:, n:] == -7).all()  # padding beyond n is untouched


def test_gemm_rrr_closed_forms():
    k, n, m = 96, 8, 4
    s = np.array([0.5, 1, 2, 4, -1, 0.25, 8, 0], np.float32)
    # all ones: C = K * scale[n]
    c = oracle.gemm_rrr(np.ones((m, k), np.float32), np.ones((k, n), np.float32), s)
    assert np.array_equal(c, np.tile(k * s, (m, 1)))
    # identity A picks rows of B, scaled per column
    b = np.arange(k * n, dtype=np.float32).reshape(k, n) - 300
    c = oracle.gemm_rrr(np.eye(m, k, dtype=np.float32), b, s)
    assert np.array_equal(c, b[:m] * s[None, :])
    # a transposed-operand slip would fail here: single non-zero at A[1,5], B[5,3]
    a = np.zeros((m, k), np.float32); a[1, 5] = 3
    b = np.zeros((k, n), np.float32); b[5, 3] = 7
    c = oracle.gemm_rrr(a, b, s)
    want = np.zeros((m, n), np.float32); want[1, 3] = 3 * (7 * s[3])
    assert np.array_equal(c, want)


def test_gemm_rrr_is_sequential_fp32():
    # numpy float32 scalar loop: the exact operation order of host_ref.hpp:19-21
    rng = np.random.Generator(np.random.PCG64(21))
    m, n, k = 2, 3, 257
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.integers(-128, 128, size=(k, n)).astype(np.float32)
    s = rng.uniform(0.001, 0.01, size=n).astype(np.float32)
    want = np.zeros((m, n), np.float32)
    for i in range(m):
        for j in range(n):
            acc = np.float32(0)
            for kk in range(k):
                acc = np.float32(acc + np.float32(a[i, kk] * np.float32(b[kk, j] * s[j])))
            want[i, j] = acc
    got = oracle.gemm_rrr(a, b, s)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and it is close to (but, being fp32, generally not equal to) the fp64 value
    c64 = a.astype(np.float64) @ (b.astype(np.float64) * s.astype(np.float64))
    assert np.allclose(got, c64, rtol=1e-5, atol=1e-5)


def test_small_int_regime_is_order_independent():
    # in the reference's regime every partial sum is an exactly representable integer: any summation
    # order gives the same bits, so the oracle equals the fp64 result exactly
    p = Problem(8, 32, 512, regime="small_int", seed=4)
    c = p.c_ref()
    c64 = widen(p.a_bf).astype(np.float64) @ widen(p.w_bf).astype(np.float64)
    assert np.array_equal(c.astype(np.float64), c64)


def test_gemm_bf16_equals_gemm_rrr_with_unit_scales():
    p = Problem(5, 48, 192, seed=9)
    c1 = oracle.gemm_bf16(p.a_bf, p.w_bf)
    c2 = oracle.gemm_rrr(widen(p.a_bf), widen(p.w_bf), np.ones(48, np.float32))
    assert np.array_equal(c1.view(np.uint32), c2.view(np.uint32))
    c64 = oracle.gemm_bf16_f64(p.a_bf, p.w_bf)
    assert np.allclose(c1, c64, rtol=1e-4, atol=1e-4)


def test_valid_vector_cases_from_reference(golden_dir):
    g = np.load(f"{golden_dir}/valid_vector_cases.npz")
    for refs, preds, ln, verdict in zip(g["refs"], g["preds"], g["lens"], g["verdicts"]):
        ok, _, _ = oracle.valid_vector(refs[:ln], preds[:ln])
        assert ok == bool(verdict)
    assert g["verdicts"].tolist() == [1, 0, 1, 0, 1]


def test_valid_vector_hand_cases():
    r = np.array([1.0, 2.0, 4.0, 8.0], np.float32)
    assert oracle.valid_vector(r, oracle.f32_to_bf16_rtz(r))[0]
    off = r.copy(); off[1] = 2.015625  # 0.78 % off
    ok, pp, _ = oracle.valid_vector(r, oracle.f32_to_bf16_rtz(off))
    assert not ok and pp == 1
    z = np.zeros(3, np.float32)
    ok, pp, nr = oracle.valid_vector(z, oracle.f32_to_bf16_rtz(z))
    assert pp == 0 and not ok  # all-zero reference: nrms is 0/0 = NaN, and NaN < 1e-3 is false (a quirk of the criterion)


def test_check_ulp():
    ref = np.array([1.0, 1.0, 1.0, -256.0, 1e-4, 1e-4, 0.0], np.float32)
    #                exact  +2ulp    +3ulp     -2ulp        rel 0.5 %     rel 5 %   zero
    pred = np.array([1.0, 1.015625, 1.0234375, -260.0, 1.005e-4, 1.05e-4, 0.0], np.float32)
    bits = oracle.f32_to_bf16_rne(pred)
    for i, want_bad in enumerate([0, 0, 1, 0, 0, 1, 0]):
        bad, worst, _ = oracle.check_ulp(ref[i:i + 1], bits[i:i + 1])
        assert bad == want_bad, (i, worst)
    bad, worst, idx = oracle.check_ulp(ref, bits)
    assert bad == 2


def test_numpy_and_c_acceptance_checks_agree():
    rng = np.random.Generator(np.random.PCG64(8))
    ref = (rng.standard_normal(20000) * np.exp(rng.uniform(-12, 4, 20000))).astype(np.float32)
    noisy = ref * (1 + rng.standard_normal(20000).astype(np.float32) * 0.006)
    bits = oracle.f32_to_bf16_rne(noisy)
    bad_np, _ = ulp_violations(ref, bits)
    bad_c, _, _ = oracle.check_ulp(ref, bits)
    assert 100 < bad_c < 19000 and bad_c == len(bad_np)
