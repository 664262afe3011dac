"""TEST INFRASTRUCTURE ONLY: numpy-facing loader for the CPU oracle.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this package; the shipped
library and driver never do.  `liboracle.so` is the C restatement in ``bfaintb_oracle.c``;
``_ref/libbfaintb_ref.so`` (optional) is the reference's own host code compiled from its headers.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libbfaintb_ref.so")

_sz = C.c_size_t
_fp = C.POINTER(C.c_float)
_u16p = C.POINTER(C.c_uint16)
_u8p = C.POINTER(C.c_uint8)


def build(with_ref=True):
    """Compile the oracle (and, where the reference sources exist, the reference wrapper)."""
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    if with_ref and os.path.isdir("/root/reference/bfAintBGemm"):
        subprocess.run(["make", "-C", _HERE, "-B", "ref"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build(with_ref=False)
    lib = C.CDLL(_LIB_PATH)
    lib.orc_bf16_to_f32.restype = C.c_float
    lib.orc_bf16_to_f32.argtypes = [C.c_uint16]
    lib.orc_f32_to_bf16_rtz.restype = C.c_uint16
    lib.orc_f32_to_bf16_rtz.argtypes = [C.c_float]
    lib.orc_f32_to_bf16_rne.restype = C.c_uint16
    lib.orc_f32_to_bf16_rne.argtypes = [C.c_float]
    lib.orc_int8_to_excess128.restype = C.c_uint8
    lib.orc_int8_to_excess128.argtypes = [C.c_float]
    lib.orc_magic_dequant_int8.restype = C.c_float
    lib.orc_magic_dequant_int8.argtypes = [C.c_uint8]
    lib.orc_bf16_to_f32_n.argtypes = [_fp, _u16p, _sz]
    lib.orc_mem_transfer_bf16.argtypes = [_u16p, _fp, _sz]
    lib.orc_f32_to_bf16_rne_n.argtypes = [_u16p, _fp, _sz]
    lib.orc_mem_transfer_int8.argtypes = [_u8p, _fp, _sz]
    lib.orc_pack_int4.argtypes = [_u8p, C.POINTER(C.c_int8), _sz, _sz, _sz, _sz]
    lib.orc_dequant.argtypes = [_u16p, _u8p, C.c_void_p, _sz, _sz, _sz, _sz, _sz, C.c_int, _sz, C.c_int, C.c_int]
    for name in ("orc_gemm_rrr", "orc_gemm_rrr_fast"):
        getattr(lib, name).argtypes = [_fp, _fp, _fp, _fp, _sz, _sz, _sz, _sz, _sz, _sz]
    lib.orc_gemm_bf16.argtypes = [_fp, _u16p, _u16p, _sz, _sz, _sz, _sz, _sz, _sz]
    lib.orc_gemm_bf16_f64.argtypes = [C.POINTER(C.c_double), _u16p, _u16p, _sz, _sz, _sz, _sz, _sz, _sz]
    lib.orc_valid_vector.restype = C.c_int
    lib.orc_valid_vector.argtypes = [_fp, _u16p, C.c_int, C.c_float, C.POINTER(C.c_int), _fp]
    lib.orc_check_ulp.restype = C.c_long
    lib.orc_check_ulp.argtypes = [_fp, _u16p, _sz, C.c_double, C.c_double, C.c_double, C.POINTER(C.c_double),
                                  C.POINTER(_sz)]
    return lib


lib = _load()


def have_ref():
    return os.path.exists(_REF_PATH)


_ref = None


def ref():
    """The reference's own host routines (compiled from its headers); None if not built."""
    global _ref
    if _ref is None and have_ref():
        r = C.CDLL(_REF_PATH)
        r.ref_gemm_rrr.argtypes = [_fp, _fp, _fp, _fp, _sz, _sz, _sz, _sz, _sz, _sz]
        r.ref_f32_to_bf16_rtz.restype = C.c_uint16
        r.ref_f32_to_bf16_rtz.argtypes = [C.c_float]
        r.ref_f32_to_bf16_rne.restype = C.c_uint16
        r.ref_f32_to_bf16_rne.argtypes = [C.c_float]
        r.ref_bf16_to_f32.restype = C.c_float
        r.ref_bf16_to_f32.argtypes = [C.c_uint16]
        r.ref_f32_to_bf16_rtz_n.argtypes = [_u16p, _fp, _sz]
        r.ref_f32_to_bf16_rne_n.argtypes = [_u16p, _fp, _sz]
        r.ref_bf16_to_f32_n.argtypes = [_fp, _u16p, _sz]
        r.ref_mem_transfer_bf16.argtypes = [_u16p, _fp, _sz]
        r.ref_mem_transfer_int8.argtypes = [_u8p, _fp, _sz]
        r.ref_valid_vector_bf16.restype = C.c_int
        r.ref_valid_vector_bf16.argtypes = [_fp, _u16p, C.c_int, C.c_float]
        r.ref_row_major_name.restype = C.c_char_p
        r.ref_column_major_name.restype = C.c_char_p
        _ref = r
    return _ref


def _p(a, t):
    return a.ctypes.data_as(t)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# ---- array-level helpers ----------------------------------------------------------------------

def bf16_to_f32(x):
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib.orc_bf16_to_f32_n(_p(out, _fp), _p(x, _u16p), x.size)
    return out


def f32_to_bf16_rtz(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.orc_mem_transfer_bf16(_p(out, _u16p), _p(x, _fp), x.size)
    return out


def f32_to_bf16_rne(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.orc_f32_to_bf16_rne_n(_p(out, _u16p), _p(x, _fp), x.size)
    return out


def mem_transfer_int8(x):
    """float matrix of integer values -> excess-128 bytes."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib.orc_mem_transfer_int8(_p(out, _u8p), _p(x, _fp), x.size)
    return out


def pack_int4(q):
    """int8 matrix [k, n] with values in [-8, 7] -> packed excess-8 bytes [k, n/2]."""
    q = _c(q, np.int8)
    k, n = q.shape
    assert n % 2 == 0
    out = np.empty((k, n // 2), np.uint8)
    lib.orc_pack_int4(_p(out, _u8p), _p(q, C.POINTER(C.c_int8)), k, n, n, n // 2)
    return out


def colmajor_codes(q, bits=8):
    """Integer weights q [k, n] -> the column-major device bytes [n, k*bits/8]: one row per column, k contiguous;
    8-bit excess-128, 4-bit excess-8 with row 2j in the low and row 2j+1 in the high nibble of byte j.  (No counterpart in
    the reference, which declares the ColumnMajor tag, gemm_tensor_layout.hpp:16-19, and never stores B that way; pinned by
    hand-computed positions in tests/test_oracle_formats.py.)"""
    q = np.asarray(q).astype(np.int64).T  # [n, k]
    if bits == 8:
        return np.ascontiguousarray((q + 128).astype(np.uint8))
    u = (q + 8).astype(np.uint8)
    return np.ascontiguousarray(u[:, 0::2] | (u[:, 1::2] << 4))


def pack_mfma16(b, k, n, bits=8):
    """Row-major packed codes b (uint8 [k, n] for 8-bit, [k, n/2] for 4-bit, the wire formats above) -> the library's
    pre-packed operand order, as a flat uint8 array of k * n * bits / 8 bytes.

    No counterpart in the reference (it keeps B row-major, bfAintBGemm.cc:101-103); this restates the byte map that
    awesome_fusion_amd/csrc/bfaintb_packed.hip documents, with array reshapes instead of the kernel's index
    arithmetic: column blocks of 16, K-chunks of R rows (64 for 8-bit, 128 for 4-bit), and inside a chunk, for lane
    16*kg + nl, the codes of column nl, rows 32*h + 8*kg + r in the order (h, r).  Pinned in the tests by
    hand-computed positions and by its inverse."""
    b = _c(b, np.uint8)
    if bits == 8:
        assert b.shape == (k, n) and k % 64 == 0 and n % 16 == 0
        v = b.reshape(k // 64, 2, 4, 8, n // 16, 16)          # [kc, h, kg, r, nb, nl]
        return np.ascontiguousarray(v.transpose(4, 0, 2, 5, 1, 3)).reshape(-1)   # [nb, kc, kg, nl, h, r]
    assert bits == 4 and b.shape == (k, n // 2) and k % 128 == 0 and n % 16 == 0
    codes = np.empty((k, n), np.uint8)
    codes[:, 0::2] = b & 15
    codes[:, 1::2] = b >> 4
    v = codes.reshape(k // 128, 4, 4, 8, n // 16, 16).transpose(4, 0, 2, 5, 1, 3)   # [nb, kc, kg, nl, h, r]
    v = np.ascontiguousarray(v)
    return (v[..., 0::2] | (v[..., 1::2] << 4)).astype(np.uint8).reshape(-1)      # row r even in the low nibble


def unpack_mfma16(packed, k, n, bits=8):
    """Inverse of pack_mfma16."""
    packed = _c(packed, np.uint8)
    if bits == 8:
        v = packed.reshape(n // 16, k // 64, 4, 16, 2, 8)      # [nb, kc, kg, nl, h, r]
        return np.ascontiguousarray(v.transpose(1, 4, 2, 5, 0, 3)).reshape(k, n)
    v = packed.reshape(n // 16, k // 128, 4, 16, 4, 4)
    codes = np.empty(v.shape[:-1] + (8,), np.uint8)
    codes[..., 0::2] = v & 15
    codes[..., 1::2] = v >> 4
    codes = np.ascontiguousarray(codes.transpose(1, 4, 2, 5, 0, 3)).reshape(k, n)
    return (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)


def dequant(b, scale, k, n, bits=8, group_size=0, rtz=False):
    """Dequantized weights as bf16 bit patterns [k, n].  scale: uint16 (bf16 bits) or float32,
    shape [groups, n] (or [n])."""
    b = _c(b, np.uint8)
    scale = np.ascontiguousarray(scale)
    is_f32 = scale.dtype == np.float32
    assert is_f32 or scale.dtype == np.uint16
    scale2 = scale.reshape(-1, n)
    groups = (k // group_size) if group_size else 1
    assert scale2.shape[0] == groups, (scale2.shape, groups)
    w = np.empty((k, n), np.uint16)
    lib.orc_dequant(_p(w, _u16p), _p(b, _u8p), scale2.ctypes.data_as(C.c_void_p), k, n, n, n, n, bits,
                    group_size, int(is_f32), int(rtz))
    return w


def gemm_rrr(a, b, scale, fast=False):
    """host_ref.hpp gemm_rrr on float32 matrices (contiguous, ld = extent)."""
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    scale = _c(scale, np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2 and scale.size == n
    c = np.empty((m, n), np.float32)
    fn = lib.orc_gemm_rrr_fast if fast else lib.orc_gemm_rrr
    fn(_p(c, _fp), _p(a, _fp), _p(b, _fp), _p(scale, _fp), m, n, k, k, n, n)
    return c


def gemm_bf16(a_bf16, w_bf16):
    """fp32 sequential-K GEMM of bf16 activations [m,k] with bf16 dequantized weights [k,n]."""
    a = _c(a_bf16, np.uint16)
    w = _c(w_bf16, np.uint16)
    m, k = a.shape
    k2, n = w.shape
    assert k == k2
    c = np.empty((m, n), np.float32)
    lib.orc_gemm_bf16(_p(c, _fp), _p(a, _u16p), _p(w, _u16p), m, n, k, k, n, n)
    return c


def gemm_bf16_f64(a_bf16, w_bf16):
    a = _c(a_bf16, np.uint16)
    w = _c(w_bf16, np.uint16)
    m, k = a.shape
    _, n = w.shape
    c = np.empty((m, n), np.float64)
    lib.orc_gemm_bf16_f64(_p(c, C.POINTER(C.c_double)), _p(a, _u16p), _p(w, _u16p), m, n, k, k, n, n)
    return c


def gemm_bf16_rows(a_bf16, w_bf16, threads=8):
    """orc_gemm_bf16 split over column blocks on a thread pool (ctypes drops the GIL); every
    output element is still one sequential-K fp32 sum, so the result is bit-identical."""
    from concurrent.futures import ThreadPoolExecutor
    a = _c(a_bf16, np.uint16)
    w = _c(w_bf16, np.uint16)
    m, k = a.shape
    _, n = w.shape
    c = np.empty((m, n), np.float32)
    blk = 512
    jobs = [(n0, min(blk, n - n0)) for n0 in range(0, n, blk)]

    def run(job):
        n0, nb = job
        lib.orc_gemm_bf16(C.cast(c.ctypes.data + 4 * n0, _fp), _p(a, _u16p),
                          C.cast(w.ctypes.data + 2 * n0, _u16p), m, nb, k, k, n, n)

    with ThreadPoolExecutor(max_workers=threads) as ex:
        list(ex.map(run, jobs))
    return c


def valid_vector(ref_c, pred_bf16, nrms=1e-3):
    r = _c(ref_c, np.float32).ravel()
    p = _c(pred_bf16, np.uint16).ravel()
    pp = C.c_int(0)
    nr = C.c_float(0)
    ok = lib.orc_valid_vector(_p(r, _fp), _p(p, _u16p), r.size, nrms, C.byref(pp), C.byref(nr))
    return bool(ok), pp.value, nr.value


def check_ulp(ref_c, pred_bf16, max_ulp=2.0, small_abs=1e-3, small_rel=1e-2):
    """Returns (failing_count, worst_error_in_ulp, flat_index_of_worst)."""
    r = _c(ref_c, np.float32).ravel()
    p = _c(pred_bf16, np.uint16).ravel()
    worst = C.c_double(0)
    idx = _sz(0)
    bad = lib.orc_check_ulp(_p(r, _fp), _p(p, _u16p), r.size, max_ulp, small_abs, small_rel, C.byref(worst),
                            C.byref(idx))
    return int(bad), worst.value, int(idx.value)
