"""Pins the oracle's number-format and wire-format functions (CPU only).

Each check is chosen so that a plausible slip — wrong shift, missing tie rule, sign of the +128 —
fails it: reference-produced fixtures, the reference's own compiled routines where built,
exhaustive identities, and torch.bfloat16 as an independent RNE implementation.
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import widen

L = oracle.lib


def test_bf16_round_trip_exhaustive(golden_dir):
    g = np.load(f"{golden_dir}/converters.npz")
    all16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = oracle.bf16_to_f32(all16)
    # widening is a 16-bit shift: compare bit patterns with what the reference's converter produced
    assert np.array_equal(f.view(np.uint32), g["bf16_to_f32_bits"])
    assert np.array_equal(f.view(np.uint32), all16.astype(np.uint32) << 16)
    # truncation inverts widening for every bf16 value, NaNs included (bit-level)
    assert np.array_equal(oracle.f32_to_bf16_rtz(f), all16)
    # RNE leaves exactly representable values alone (NaN payloads aside)
    notnan = ~np.isnan(f)
    assert np.array_equal(oracle.f32_to_bf16_rne(f)[notnan], all16[notnan])


def test_known_answers():
    ka_rtz = {0x3F800000: 0x3F80, 0x3F7FFFFF: 0x3F7F, 0xBF7FFFFF: 0xBF7F}
    ka_rne = {0x3F808000: 0x3F80,  # tie, kept mantissa even -> stays
              0x3F818000: 0x3F82,  # tie, kept mantissa odd -> up
              0x3F808001: 0x3F81,  # just above the tie
              0x3F807FFF: 0x3F80,  # just below
              0x3F7FFFFF: 0x3F80,  # carry into the exponent
              0x7F7FFFFF: 0x7F80,  # rounds up to Inf
              0x7F800000: 0x7F80, 0xFF800000: 0xFF80,
              0x7F800001: 0x7F81,  # signalling NaN keeps a payload bit
              0x00008000: 0x0000, 0x00018000: 0x0002}
    for bits, want in ka_rtz.items():
        assert L.orc_f32_to_bf16_rtz(C.c_float(np.uint32(bits).view(np.float32))) == want
    for bits, want in ka_rne.items():
        assert oracle.f32_to_bf16_rne(np.array([bits], np.uint32).view(np.float32))[0] == want, hex(bits)


def test_converters_match_reference_fixture(golden_dir):
    g = np.load(f"{golden_dir}/converters.npz")
    f = g["f32_bits"].view(np.float32)
    assert np.array_equal(oracle.f32_to_bf16_rne(f), g["rne"])
    assert np.array_equal(oracle.f32_to_bf16_rtz(f), g["rtz"])
    assert np.array_equal(oracle.mem_transfer_int8(g["int8_values"]), g["int8_bytes"])


def test_rne_matches_torch_bfloat16():
    import torch
    rng = np.random.Generator(np.random.PCG64(7))
    bits = rng.integers(0, 2**32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    keep = ~np.isnan(f)
    f = f[keep]
    t = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_rne(f), t)


@pytest.mark.skipif(not oracle.have_ref(), reason="reference wrapper not built (needs /root/reference)")
def test_converters_match_compiled_reference():
    r = oracle.ref()
    rng = np.random.Generator(np.random.PCG64(11))
    bits = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    u16p, fp = C.POINTER(C.c_uint16), C.POINTER(C.c_float)
    for mine, theirs in ((oracle.f32_to_bf16_rne, r.ref_f32_to_bf16_rne_n), (oracle.f32_to_bf16_rtz, r.ref_f32_to_bf16_rtz_n)):
        out = np.zeros(f.size, np.uint16)
        theirs(out.ctypes.data_as(u16p), f.ctypes.data_as(fp), f.size)
        assert np.array_equal(mine(f), out)
    x = rng.standard_normal(4096).astype(np.float32) * 100
    out = np.zeros(4096, np.uint16)
    r.ref_mem_transfer_bf16(out.ctypes.data_as(C.POINTER(C.c_uint16)), x.ctypes.data_as(C.POINTER(C.c_float)), x.size)
    assert np.array_equal(out, oracle.f32_to_bf16_rtz(x))
    assert r.ref_row_major_name() == b"RowMajor" and r.ref_column_major_name() == b"ColumnMajor"


def test_excess128_closed_form():
    q = np.arange(-128, 128)
    got = oracle.mem_transfer_int8(q.astype(np.float32))
    assert np.array_equal(got, ((q + 128) & 0xFF).astype(np.uint8))
    assert got[0] == 0x00 and got[128] == 0x80 and got[255] == 0xFF
    # fractional inputs truncate toward zero before the offset (static_cast<int8_t>)
    assert oracle.mem_transfer_int8(np.array([1.9, -1.9, 0.5], np.float32)).tolist() == [129, 127, 128]


def test_magic_number_decode_is_exact():
    for u in range(256):
        assert L.orc_magic_dequant_int8(u) == float(u - 128)


def test_int4_packing_brute_force():
    rng = np.random.Generator(np.random.PCG64(3))
    q = rng.integers(-8, 8, size=(6, 32)).astype(np.int8)
    packed = oracle.pack_int4(q)
    assert packed.shape == (6, 16)
    for i in range(6):
        for j in range(32):
            byte = int(packed[i, j // 2])
            code = (byte >> 4) if j % 2 else (byte & 0xF)
            assert code - 8 == q[i, j]
    # the extremes land where the format says
    assert oracle.pack_int4(np.array([[-8, 7]], np.int8))[0, 0] == 0xF0


@pytest.mark.parametrize("bits,group", [(8, 0), (8, 32), (4, 0), (4, 128)])
def test_dequant_against_numpy(bits, group):
    rng = np.random.Generator(np.random.PCG64(5))
    k, n = 256, 64
    lo, hi = (-128, 128) if bits == 8 else (-8, 8)
    q = rng.integers(lo, hi, size=(k, n)).astype(np.int8)
    groups = k // group if group else 1
    s_bf = oracle.f32_to_bf16_rne(rng.uniform(0.001, 0.02, size=(groups, n)).astype(np.float32))
    b = oracle.mem_transfer_int8(q.astype(np.float32)) if bits == 8 else oracle.pack_int4(q)
    w = oracle.dequant(b, s_bf, k, n, bits, group)
    # independent statement: float64 product (exact), rounded once to bf16 by torch
    import torch
    srow = widen(s_bf).astype(np.float64)
    gidx = (np.arange(k) // group) if group else np.zeros(k, int)
    prod = q.astype(np.float64) * srow[gidx]
    assert np.array_equal(prod.astype(np.float32).astype(np.float64), prod), "int x bf16 must be exact in fp32"
    want = torch.from_numpy(prod.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(w, want)
    # truncating variant differs from RNE somewhere and never exceeds it in magnitude
    w_rtz = oracle.dequant(b, s_bf, k, n, bits, group, rtz=True)
    assert np.array_equal(w_rtz, (prod.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
    assert (w_rtz != w).any()


def test_dequant_with_the_reference_kernels_arithmetic():
    # fp32 scales, product rounded to fp32 by the multiply, then the high 16 bits (bf16gemm_kernel_gfx90a.s:29-35):
    # independent statement in numpy float32 arithmetic, exhaustive over the 256 codes for scales with full mantissas
    rng = np.random.Generator(np.random.PCG64(6))
    k, n = 256, 48
    q = np.tile(np.arange(-128, 128, dtype=np.int64)[:, None], (1, n)).astype(np.int8)
    s = rng.uniform(-0.02, 0.02, size=n).astype(np.float32)
    s[:4] = np.array([1.0, -1.0, 0.0, 3.0000002], np.float32)
    b = oracle.mem_transfer_int8(q.astype(np.float32))
    w = oracle.dequant(b, s, k, n, 8, 0, rtz=True)
    prod = q.astype(np.float32) * s[None, :]                 # one IEEE fp32 multiply per weight
    assert np.array_equal(w, (prod.view(np.uint32) >> 16).astype(np.uint16))
    assert np.array_equal(w[:, 0], oracle.f32_to_bf16_rtz(q[:, 0].astype(np.float32)))   # unit scale: the code itself
    # truncation never grows a magnitude, and it differs from both other contracts on this data
    assert np.all(np.abs(widen(w)) <= np.abs(prod))
    assert (w != oracle.dequant(b, s, k, n, 8, 0, rtz=False)).any()
    assert (w != oracle.dequant(b, oracle.f32_to_bf16_rne(s.reshape(1, n)), k, n, 8, 0, rtz=True)).any()


def test_int_times_bf16_scale_is_exact_exhaustive():
    # every 8-bit integer times every positive normal bf16 significand pattern: the fp32 product equals the exact one
    q = np.arange(-128, 128, dtype=np.float64)[:, None]
    sig = widen(np.arange(0x3F80, 0x4000, dtype=np.uint32).astype(np.uint16)).astype(np.float64)[None, :]
    exact = q * sig
    assert np.array_equal(exact.astype(np.float32).astype(np.float64), exact)


def test_prepacked_order_positions_and_inverse():
    # the packed operand order has no counterpart in the reference: pin the restatement by positions worked out by
    # hand from the documented byte map, and by its inverse
    rng = np.random.default_rng(5)
    k, n = 192, 48
    b = rng.integers(0, 256, size=(k, n), dtype=np.uint8)
    pk = oracle.pack_mfma16(b, k, n, 8)
    assert pk.size == k * n
    # row 37 = chunk 0, K-block 1, kg 0, r 5; column 5 = block 0, nl 5: lane 5 -> byte 5*16 + 8*1 + 5
    assert pk[93] == b[37, 5]
    # row 150 = chunk 2 (128..191), h 0, kg 2 (rows 16..23 of the K-block), r 6; column 40 = block 2, nl 8:
    # chunk index (2 * 3 + 2) = 8, lane 16*2 + 8 = 40 -> 8*1024 + 40*16 + 0*8 + 6
    assert pk[8 * 1024 + 40 * 16 + 6] == b[150, 40]
    assert np.array_equal(oracle.unpack_mfma16(pk, k, n, 8), b)

    k, n = 256, 32
    q = rng.integers(-8, 8, size=(k, n), dtype=np.int8)
    b4 = oracle.pack_int4(q)
    pk4 = oracle.pack_mfma16(b4, k, n, 4)
    assert pk4.size == k * n // 2
    code = lambda r, c: int(q[r, c]) + 8
    # row 100 = chunk 0, h 3, kg 0, r 4; column 21 = block 1, nl 5: chunk index 1*2+0 = 2, lane 5
    # -> byte 2*1024 + 5*16 + 4*3 + 4/2, low nibble (r even); the high nibble is row 101
    assert pk4[2 * 1024 + 5 * 16 + 14] == (code(100, 21) | (code(101, 21) << 4))
    # row 255 = chunk 1, h 3, kg 3, r 7; column 0: chunk index 1, lane 48 -> byte 1024 + 48*16 + 12 + 3, high nibble
    assert pk4[1024 + 48 * 16 + 15] >> 4 == code(255, 0)
    assert np.array_equal(oracle.unpack_mfma16(pk4, k, n, 4), b4)


def test_colmajor_codes_positions():
    # column-major device bytes (no counterpart in the reference): positions worked out by hand from the stated format
    q = np.zeros((8, 4), np.int8)
    q[3, 2], q[4, 2], q[5, 2], q[0, 1] = -128, 127, -1, 5
    b = oracle.colmajor_codes(q, 8)
    assert b.shape == (4, 8) and b[2, 3] == 0 and b[2, 4] == 255 and b[2, 5] == 127 and b[1, 0] == 133 and b[0, 0] == 128
    q4 = np.zeros((8, 4), np.int8)
    q4[4, 3], q4[5, 3], q4[0, 0], q4[7, 1] = -8, 7, 3, -1
    b4 = oracle.colmajor_codes(q4, 4)
    assert b4.shape == (4, 4)
    assert b4[3, 2] == 0xF0            # rows 4 (code 0, low nibble) and 5 (code 15, high nibble) of column 3
    assert b4[0, 0] == (8 << 4 | 11)   # row 0: 3 + 8 = 11 low; row 1: zero -> 8 high
    assert b4[1, 3] == (7 << 4 | 8)    # row 7 of column 1: -1 + 8 = 7 in the high nibble of byte 3
    # and it is the transpose of the row-major form, code by code
    rng = np.random.default_rng(9)
    q = rng.integers(-8, 8, size=(64, 32), dtype=np.int8)
    rm, cm = oracle.pack_int4(q), oracle.colmajor_codes(q, 4)
    for (r, c) in [(0, 0), (13, 7), (63, 31), (20, 30), (41, 1)]:
        row_code = (rm[r, c // 2] >> (4 * (c % 2))) & 15
        col_code = (cm[c, r // 2] >> (4 * (r % 2))) & 15
        assert row_code == col_code == q[r, c] + 8
