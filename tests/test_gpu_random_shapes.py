"""Seeded random walk over the library's argument space: shapes, code widths, scale groups, weight orders, variants and
epilogues drawn together, each case checked against the CPU oracle through the C ABI.  The directed tests cover the
corners by design; this one covers combinations nobody thought of (it is deterministic: the seed is fixed)."""
import numpy as np
import pytest

import oracle
from helpers import Problem, assert_close_gated, assert_close_ulp, run_gemm
from test_gpu_prepacked import run_prepacked

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def af():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    import awesome_fusion_amd as af
    af.lib()  # raises if the HIP library was not built: no fallback
    return af


def run_strided(af, p, which, act, packed, pad):
    """The same product with lda = k + pad, ldc = ldr = columns + pad; the padding of C must come back untouched."""
    import torch
    from helpers import Workspace, from_dev_u16, to_dev
    out_n = p.n // 2 if act else p.n
    a = np.full((p.m, p.k + pad), 0x7FC0, np.uint16)          # NaN in the padding: it must never be read as data
    a[:, :p.k] = p.a_bf
    res = None
    if p.residual_bf is not None:
        r = np.full((p.m, out_n + pad), 0x7FC0, np.uint16)
        r[:, :out_n] = p.residual_bf
        res = to_dev(r)
    c = torch.full((p.m, out_n + pad), 0x7FC1, dtype=torch.int16, device="cuda")
    bias = None if p.bias_bf is None else to_dev(p.bias_bf)
    kw = dict(weight_bits=p.bits, group_size=p.group_size, bias=bias, residual=res, ldr=None if res is None else out_n + pad, activation=act)
    if packed:
        pk = torch.zeros(af.prepack_bytes(p.n, p.k, p.bits), dtype=torch.uint8, device="cuda")
        af.prepack(pk, to_dev(p.b_bytes), p.n, p.k, weight_bits=p.bits)
        ws = Workspace().get(af.prepacked_workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size, which))
        af.gemm_prepacked(c, to_dev(a), pk, to_dev(p.s_bf), p.m, p.n, p.k, lda=p.k + pad, ldc=out_n + pad, workspace=ws, which=which, **kw)
    else:
        ws = Workspace().get(af.workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size, which))
        af.gemm(c, to_dev(a), to_dev(p.b_bytes), to_dev(p.s_bf), p.m, p.n, p.k, lda=p.k + pad, ldc=out_n + pad, workspace=ws, which=which, **kw)
    torch.cuda.synchronize()
    got = from_dev_u16(c)
    assert np.all(got[:, out_n:] == 0x7FC1), "padding of C was written"
    return np.ascontiguousarray(got[:, :out_n])


def draw_case(rng):
    bits = int(rng.choice([8, 4]))
    packed = bool(rng.integers(0, 2))
    kunit = 128 if (bits == 4 and packed) else 64
    m = int(rng.choice([rng.integers(1, 9), rng.integers(9, 49), rng.integers(49, 200), rng.integers(200, 700)]))
    kmax = 8192 if m < 49 else 1024               # long k with few rows: the split-K plans
    k = kunit * int(rng.integers(1, kmax // kunit + 1))
    n = 16 * int(rng.integers(1, 70))
    groups = [g for g in (0, 32, 64, 128, 256) if g == 0 or k % g == 0]
    group = int(rng.choice(groups))
    epilogue = str(rng.choice(["none", "none", "none", "bias", "residual", "bias+residual", "gate", "gate+bias+residual"]))
    if epilogue.startswith("gate") and n % 32:
        n += 16                                   # the gated output has n/2 columns, itself a multiple of 16
    variant = str(rng.choice(["auto", "decode", "prefill_128", "prefill_256", "prefill_256_lds"]))
    if epilogue != "none" and not (packed and epilogue == "bias"):
        variant = "auto"                          # the fused entry points choose the kernel themselves
    pad = int(rng.choice([0, 0, 8, 24]))           # extra elements per row of A, C (and the residual): strided operands
    return dict(m=m, n=n, k=k, bits=bits, group=group, packed=packed, epilogue=epilogue, variant=variant, pad=pad)


CASES = [draw_case(np.random.Generator(np.random.PCG64(1000 + i))) for i in range(300)]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "{m}x{n}x{k}-b{bits}-g{group}-{o}-{variant}-{epilogue}".format(o="packed" if c["packed"] else "rowmajor", **c))
def test_random_case(af, case):
    m, n, k, bits, group = case["m"], case["n"], case["k"], case["bits"], case["group"]
    gated = case["epilogue"].startswith("gate")
    if gated:
        p = Problem(m, n, k, bits, group, seed=m + n + k, scale_lo=0.002, scale_hi=0.02 if bits == 8 else 0.2)
    else:
        p = Problem(m, n, k, bits, group, seed=m + n + k)
    if "bias" in case["epilogue"]:
        p.with_bias()
    if "residual" in case["epilogue"]:
        if gated:
            p.residual_bf = oracle.f32_to_bf16_rne(np.random.default_rng(m).uniform(-2, 2, size=(m, n // 2)).astype(np.float32))
        else:
            p.with_residual()
    which = {"auto": af.AUTO, "decode": af.DECODE, "prefill_128": af.PREFILL_128, "prefill_256": af.PREFILL_256,
             "prefill_256_lds": af.PREFILL_256_LDS}[case["variant"]]
    act = af.ACT_SILU_GATE if gated else af.ACT_NONE
    if case["pad"]:
        c = run_strided(af, p, which, act, case["packed"], case["pad"])
    else:
        c = run_prepacked(af, p, which, activation=act) if case["packed"] else run_gemm(p, which=which, activation=act)
    if gated:
        assert_close_gated(p, c, str(case))
    else:
        assert_close_ulp(p, c, str(case))


# ---------------------------------------------------------------------------------------------------------------------
# Ragged shapes: n a multiple of 8 (16 for 4-bit codes), k a multiple of 8 — the tails the reference kernel never handled
# (its N-tail flag compares the wrong index, bf16gemm_kernel_gfx90a.s:341-343; its K dispatch knows multiples of 64 only,
# :402-408).  Row-major weights (the packed order keeps whole chunks).  A, B and C carry padding filled with NaNs / a
# sentinel: nothing of it may be read as data or written.

def run_ragged(af, p, which, act=0, pad=0):
    import torch
    from helpers import Workspace, from_dev_u16, to_dev
    out_n = p.n // 2 if act else p.n
    lda, ldc = p.k + pad, (out_n + 7) // 8 * 8 + pad
    ldb = (p.n + 15) // 16 * 16                                  # rows of B stay 16-byte aligned
    a = np.full((p.m, lda), 0x7FC0, np.uint16)
    a[:, :p.k] = p.a_bf
    b = np.full((p.k, ldb * p.bits // 8), 0x55, np.uint8)
    b[:, :p.n * p.bits // 8] = p.b_bytes
    res = None
    if p.residual_bf is not None:
        r = np.full((p.m, ldc), 0x7FC0, np.uint16)
        r[:, :out_n] = p.residual_bf
        res = to_dev(r)
    c = torch.full((p.m, ldc), 0x7FC1, dtype=torch.int16, device="cuda")
    bias = None if p.bias_bf is None else to_dev(p.bias_bf)
    ws = Workspace().get(af.workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size, which))
    af.gemm(c, to_dev(a), to_dev(b), to_dev(p.s_bf), p.m, p.n, p.k, lda=lda, ldb=ldb, ldc=ldc, workspace=ws, which=which,
            weight_bits=p.bits, group_size=p.group_size, bias=bias, residual=res, ldr=None if res is None else ldc, activation=act)
    torch.cuda.synchronize()
    got = from_dev_u16(c)
    assert np.all(got[:, out_n:] == 0x7FC1), "padding of C was written"
    return np.ascontiguousarray(got[:, :out_n])


@pytest.mark.parametrize("m,n,k,bits,group,variant", [
    (33, 1000, 1000, 8, 0, "auto"), (33, 1000, 1000, 8, 0, "decode"), (33, 1000, 1000, 8, 0, "prefill_128"), (33, 1000, 1000, 8, 0, "prefill_256"),
    (1, 4104, 4072, 8, 0, "auto"), (16, 4104, 4072, 8, 0, "auto"), (32, 520, 1048, 8, 0, "auto"),
    (1, 8, 8, 8, 0, "auto"), (5, 24, 16, 8, 0, "decode"), (5, 24, 24, 8, 0, "prefill_128"), (70, 40, 8, 8, 0, "prefill_256"),
    (300, 1000, 1000, 8, 0, "auto"), (700, 1000, 1000, 8, 0, "prefill_256"), (700, 1000, 1000, 8, 0, "prefill_256_lds"), (130, 264, 72, 8, 0, "decode"),
    (33000, 264, 72, 8, 0, "prefill_256"), (33000, 272, 72, 4, 0, "prefill_256"), (33000, 264, 96, 8, 32, "prefill_256"),   # whole rounds of 256x256 tiles
    (16, 1008, 1000, 4, 0, "auto"), (1, 4112, 4072, 4, 0, "auto"), (300, 1008, 1000, 4, 0, "prefill_128"), (300, 1008, 1000, 4, 0, "prefill_256"),
    (48, 1000, 992, 8, 32, "auto"), (300, 1000, 992, 8, 32, "prefill_128"), (300, 1000, 96, 8, 32, "prefill_256"), (8, 1008, 96, 4, 32, "auto"),
])
def test_ragged_shapes(af, m, n, k, bits, group, variant):
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    which = {"auto": af.AUTO, "decode": af.DECODE, "prefill_128": af.PREFILL_128, "prefill_256": af.PREFILL_256, "prefill_256_lds": af.PREFILL_256_LDS}[variant]
    assert_close_ulp(p, run_ragged(af, p, which, pad=8), f"ragged {m}x{n}x{k} int{bits} g{group} {variant}")


@pytest.mark.parametrize("m,n,k,bits,group", [
    (1, 33000, 512, 8, 0),       # n % 16 != 0: only 128-column blocks can read the last columns — 258 of them, two past a round
    (5, 45072, 2048, 4, 128),    # 4-bit, 4 waves: 177 blocks of 256 columns, the last one 16 columns wide, k split four ways by rounds
    (12, 36880, 4224, 4, 128),   # 8 waves, a half-filled round of 256-column blocks split three ways, a 16-column last block
    (64, 36872, 192, 8, 0),      # one row of 289 small tiles in their 64-row form, the last tile 8 columns wide
    (40, 50320, 256, 4, 64),     # the same for 4-bit codes: 394 tiles, 16 columns in the last
    (70, 33032, 128, 8, 0),      # ... and with more than 64 rows: the whole-tile form, 259 tiles
])
def test_very_wide_ragged_shapes(af, m, n, k, bits, group):
    """Column counts beyond 32768 that do not end on a block or tile, kernel left to the library; rows of B and C padded by 8 elements."""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    assert_close_ulp(p, run_ragged(af, p, af.AUTO, pad=8), f"very wide {m}x{n}x{k} bits={bits} g={group}")


def draw_ragged(rng):
    bits = int(rng.choice([8, 8, 4]))
    m = int(rng.choice([rng.integers(1, 9), rng.integers(9, 49), rng.integers(49, 200), rng.integers(200, 500)]))
    group = int(rng.choice([0, 0, 0, 32, 128]))
    kunit = group if group else 8
    kmax = 6144 if m < 49 else 1024
    k = kunit * int(rng.integers(1, kmax // kunit + 1))
    n = (16 if bits == 4 else 8) * int(rng.integers(1, 140 if bits == 8 else 70))
    epilogue = str(rng.choice(["none", "none", "bias", "bias+residual", "gate"]))
    if epilogue == "gate":
        n = (n + 15) // 16 * 16
    variant = str(rng.choice(["auto", "decode", "prefill_128", "prefill_256", "prefill_256_lds"])) if epilogue == "none" else "auto"
    return dict(m=m, n=n, k=k, bits=bits, group=group, epilogue=epilogue, variant=variant, pad=int(rng.choice([0, 8, 24])))


RAGGED = [draw_ragged(np.random.Generator(np.random.PCG64(5000 + i))) for i in range(150)]


@pytest.mark.parametrize("case", RAGGED, ids=lambda c: "{m}x{n}x{k}-b{bits}-g{group}-{variant}-{epilogue}".format(**c))
def test_random_ragged_case(af, case):
    m, n, k, bits, group = case["m"], case["n"], case["k"], case["bits"], case["group"]
    gated = case["epilogue"] == "gate"
    p = Problem(m, n, k, bits, group, seed=m + n + k, **(dict(scale_lo=0.002, scale_hi=0.02 if bits == 8 else 0.2) if gated else {}))
    if "bias" in case["epilogue"]:
        p.with_bias()
    if "residual" in case["epilogue"]:
        p.with_residual()
    which = {"auto": af.AUTO, "decode": af.DECODE, "prefill_128": af.PREFILL_128, "prefill_256": af.PREFILL_256,
             "prefill_256_lds": af.PREFILL_256_LDS}[case["variant"]]
    c = run_ragged(af, p, which, af.ACT_SILU_GATE if gated else af.ACT_NONE, case["pad"])
    (assert_close_gated if gated else assert_close_ulp)(p, c, str(case))


@pytest.mark.parametrize("cus", [64, 304])
def test_plans_for_another_compute_unit_count_are_still_correct_launches(af, cus):
    """The launch plans follow the device's compute units; a plan made for another count (the tuning hook) changes the
    split factors, the tile sizes and the second launch over a thin last round, and never the result's contract."""
    shapes = [(1, 4096, 4096, 8, 0), (16, 1024, 4096, 8, 0), (24, 2064, 2048, 4, 128), (72, 1536, 2048, 8, 0), (300, 512, 1024, 8, 0),
              (700, 1280, 512, 4, 64), (520, 4096, 256, 8, 0), (2100, 2304, 256, 8, 0)]
    try:
        af.debug_control(af.DEBUG_PLAN_COMPUTE_UNITS, cus)
        for i, (m, n, k, bits, g) in enumerate(shapes):
            assert af.plan(m, n, k, bits, g).compute_units == cus
            p = Problem(m, n, k, bits, g, seed=300 + i)
            assert_close_ulp(p, run_gemm(p), f"planned for {cus} compute units: {m}x{n}x{k} int{bits} g{g}")
            if k % 128 == 0:  # (whole K-chunks of either code width)
                assert_close_ulp(p, run_prepacked(af, p), f"planned for {cus} compute units, packed: {m}x{n}x{k} int{bits} g{g}")
    finally:
        af.debug_control(af.DEBUG_PLAN_COMPUTE_UNITS, 0)
