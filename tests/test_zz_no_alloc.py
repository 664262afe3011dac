"""bfaintb_gemm_static: the GEMM on the library's own per-GPU scratch (no workspace argument, no allocation), checked
through the C ABI against bfaintb_gemm with a caller's workspace: bit for bit, on calls in a row that share the scratch."""
import ctypes as C

import numpy as np
import pytest

from helpers import Problem, from_dev_u16, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def af():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    import awesome_fusion_amd as af
    af.lib()  # raises if the HIP library was not built: no fallback
    return af


def _both(af, p):
    """(C from bfaintb_gemm_static, C from bfaintb_gemm with its own fresh workspace), straight through the C ABI."""
    import torch
    L = af.lib()
    a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
    stream = torch.cuda.current_stream().cuda_stream
    c_static = torch.full((p.m, p.n), 0x7FC0, dtype=torch.int16, device="cuda")
    c_plain = torch.full((p.m, p.n), 0x7FC0, dtype=torch.int16, device="cuda")
    rc = L.bfaintb_gemm_static(c_static.data_ptr(), a.data_ptr(), b.data_ptr(), s.data_ptr(), p.m, p.n, p.k, p.k, p.n, p.n,
                               p.bits, p.group_size, stream)
    assert rc == 0, af.error_string(rc)
    need = L.bfaintb_gemm_workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
    assert L.bfaintb_workspace_init(ws.data_ptr(), ws.numel(), stream) == 0
    rc = L.bfaintb_gemm(c_plain.data_ptr(), a.data_ptr(), b.data_ptr(), s.data_ptr(), p.m, p.n, p.k, p.k, p.n, p.n, p.bits,
                        p.group_size, ws.data_ptr() if need else None, need, stream)
    assert rc == 0, af.error_string(rc)
    torch.cuda.synchronize()
    return from_dev_u16(c_static), from_dev_u16(c_plain), need


def test_static_scratch_matches_caller_workspace_on_calls_in_a_row(af):
    # the second input is smaller than the first (it finds the scratch as the first call left it), the third larger
    # again and 4-bit with group scales, the fourth runs without split-K (the tiled kernel: the scratch is not touched),
    # the fifth is the tiled kernel with k split (its partial sums go through the scratch as well), the sixth one row of
    # small tiles with k split three ways, two rounds of workgroups
    shapes = [(16, 4096, 4096, 8, 0), (1, 1024, 2048, 8, 0), (4, 4096, 8192, 4, 128), (300, 512, 256, 8, 0), (384, 2048, 8192, 8, 0),
              (33, 16512, 8192, 8, 0), (1, 4096, 4096, 8, 0)]
    used_split = 0
    for i, (m, n, k, bits, group) in enumerate(shapes):
        p = Problem(m, n, k, bits, group, seed=40 + i)
        c_static, c_plain, need = _both(af, p)
        used_split += need > 0
        assert np.array_equal(c_static, c_plain), f"call {i}: {shapes[i]}"
        assert not np.isnan(c_plain.view(np.uint16).astype(np.uint32) << 16).any()
    assert used_split >= 6  # the comparison did exercise the scratch


def test_static_scratch_refuses_what_does_not_fit(af):
    L = af.lib()
    # 32 rows x 22016 columns of 4-bit codes, k long enough for 8 splits: 18.8 MiB of partial sums
    m, n, k = 32, 22016, 28672
    need = L.bfaintb_gemm_workspace_bytes(m, n, k, 4, 128)
    assert need > L.bfaintb_gemm_static_scratch_bytes() == 16 << 20
    P = 1 << 20  # never dereferenced: the call is refused before any launch
    assert L.bfaintb_gemm_static(P, P, P, P, m, n, k, k, n, n, 4, 128, None) == af.ERR_STATIC_SCRATCH
    assert "bfaintb_gemm" in af.error_string(af.ERR_STATIC_SCRATCH)


def test_static_scratch_status_and_reset_after_a_give_up(af):
    """The give-up path on the library's own scratch, forced from the host (producers keep their sums, the wait is capped:
    every kernel exits normally): the call's outputs are NaN, bfaintb_static_scratch_status reports the poisoned scratch,
    bfaintb_static_scratch_reset repairs it, and the next call gives bfaintb_gemm's bits again."""
    import torch
    af.init()
    p = Problem(4, 2048, 4096, seed=91)
    assert af.split_k(p.m, p.n, p.k) > 1
    c_static, c_plain, _ = _both(af, p)
    assert np.array_equal(c_static, c_plain)
    assert af.static_scratch_status() == 0
    a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
    c = torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda")
    try:
        af.debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 3)
        af.debug_control(af.DEBUG_WITHHOLD_PARTIALS, 1)
        af.gemm_static(c, a, b, s, p.m, p.n, p.k)
        torch.cuda.synchronize()
    finally:
        af.debug_control(af.DEBUG_WITHHOLD_PARTIALS, 0)
        af.debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 0)
    got = from_dev_u16(c).astype(np.uint32) << 16
    assert np.isnan(got.view(np.float32)).all(), "every output misses partial sums: all NaN"
    assert af.static_scratch_status() == af.ERR_WORKSPACE_POISONED
    af.static_scratch_reset()
    assert af.static_scratch_status() == 0
    c_static, c_plain, _ = _both(af, p)
    assert np.array_equal(c_static, c_plain)
    assert af.static_scratch_status() == 0


def test_static_entry_point_can_be_captured_and_replayed(af):
    """No allocation, no memset, no host-side wait: the call records into a HIP graph; replays, with eager calls on the
    same scratch in between, give the eager result every time."""
    import torch
    af.init()
    p = Problem(8, 2048, 4096, seed=77)
    small = Problem(1, 512, 4096, seed=78)
    a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
    c = torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda")
    af.gemm_static(c, a, b, s, p.m, p.n, p.k)
    torch.cuda.synchronize()
    want = from_dev_u16(c).copy()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        af.gemm_static(c, a, b, s, p.m, p.n, p.k)
    for rep in range(4):
        c.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(from_dev_u16(c), want), f"replay {rep}"
        cs = torch.zeros((small.m, small.n), dtype=torch.int16, device="cuda")
        af.gemm_static(cs, to_dev(small.a_bf), to_dev(small.b_bytes), to_dev(small.s_bf), small.m, small.n, small.k)
        torch.cuda.synchronize()
