"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X.

Bars: dequantised weights bit-exact; bf16 output within 2 bf16 ULP of the fp32 sequential-K oracle
(or relative error <= 1e-2 where |ref| < 1e-3); bit-exact wherever the arithmetic is exact
(one-hot activations, the reference's small-integer regime, power-of-two scaling).
"""
import numpy as np
import pytest

import oracle
from helpers import Problem, assert_close_gated, assert_close_ulp, from_dev_u16, run_gemm, to_dev, widen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def af():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    import awesome_fusion_amd as af
    af.lib()  # raises if the HIP library was not built: no fallback
    return af


# ---------------------------------------------------------------------------- dequantisation

@pytest.mark.parametrize("bits,group", [(8, 0), (8, 128), (8, 32), (4, 0), (4, 128), (4, 64)])
def test_dequant_dump_bit_exact(af, bits, group):
    import torch
    k, n = 512, 1024
    p = Problem(1, n, k, bits, group, seed=100 + bits + group, scale_lo=0.001, scale_hi=0.02)
    if bits == 8:  # every code next to every kind of scale
        p.b_bytes[:256, 0] = np.arange(256, dtype=np.uint8)
        p.b_bytes[0, :256] = np.arange(256, dtype=np.uint8)
    p.s_bf[0, :8] = np.array([0x3F80, 0x3F7F, 0x3C01, 0xBC7F, 0x0000, 0x4000, 0x3DFF, 0x38D1], np.uint16)
    p._w = None
    w_dev = torch.zeros((k, n), dtype=torch.int16, device="cuda")
    af.dequant(w_dev, to_dev(p.b_bytes), to_dev(p.s_bf), n, k, weight_bits=bits, group_size=group)
    torch.cuda.synchronize()
    got = from_dev_u16(w_dev)
    assert np.array_equal(got, p.w_bf), f"{np.count_nonzero(got != p.w_bf)} dequantised weights differ"


@pytest.mark.parametrize("bits,group", [(8, 0), (4, 128)])
@pytest.mark.parametrize("which_m", [("decode", 16), ("decode", 32), ("prefill_256", 64), ("prefill_128", 64)])
def test_gemm_kernels_dequantise_bit_exact(af, bits, group, which_m):
    """One-hot activations make C[i,:] = W[k_i,:] with nothing to round: the GEMM kernels' own
    in-register dequantisation is observed exactly."""
    which, m = which_m
    which = {"decode": af.DECODE, "prefill_256": af.PREFILL_256, "prefill_128": af.PREFILL_128}[which]
    k, n = 256, 512
    p = Problem(m, n, k, bits, group, seed=7)
    seen = np.zeros(k, bool)
    for base in range(0, k, m):
        a = np.zeros((m, k), np.float32)
        rows = (base + np.arange(m)) % k
        a[np.arange(m), rows] = 1.0
        p.a_bf = oracle.f32_to_bf16_rne(a)
        c = run_gemm(p, which=which)
        assert np.array_equal(c, p.w_bf[rows]), f"rows {base}.. differ"
        seen[rows] = True
    assert seen.all()


# ---------------------------------------------------------------------------- exact regimes

@pytest.mark.parametrize("m,n,k", [(32, 128, 512), (1, 256, 512), (64, 128, 256), (300, 272, 192)])
def test_reference_regime_bit_for_bit(af, m, n, k):
    """Data in {-2,-1,0,1} (random_gen.hpp:24,37,50): every partial sum is an exact integer, so the
    device must equal the host reference bit for bit and the reference's own valid_vector passes."""
    p = Problem(m, n, k, regime="small_int", seed=m + n)
    c_ref = oracle.gemm_rrr(widen(p.a_bf), p.q.astype(np.float32), widen(p.s_bf)[0])  # host_ref as main() calls it
    c = run_gemm(p)
    # the fp32 sums are exact; the only rounding is the store to bf16 (odd integers above 256 are not bf16 numbers)
    assert np.array_equal(widen(c), widen(oracle.f32_to_bf16_rne(c_ref)))
    if np.abs(c_ref).max() <= 256 and c_ref.any():
        ok, pp, _ = oracle.valid_vector(c_ref, c)  # the reference's own acceptance test (validation.hpp:7-46)
        assert ok and pp == 0


def test_golden_int_regime_fixture(af, golden_dir):
    g = np.load(f"{golden_dir}/int_regime_seed1.npz")
    p = Problem(32, 128, 512, regime="small_int")
    p.a_bf, p.b_bytes, p.s_bf = g["a_dev"], g["b_dev"], oracle.f32_to_bf16_rne(g["s"]).reshape(1, -1)
    c = run_gemm(p)
    assert np.array_equal(c, g["c_bf_trunc"])  # exact values: truncation == RNE here


def test_power_of_two_scaling_commutes(af):
    p = Problem(8, 512, 1024, seed=3)
    c1 = run_gemm(p)
    p.a_bf = oracle.f32_to_bf16_rne(widen(p.a_bf) * 4.0)
    c4 = run_gemm(p)
    assert np.array_equal(widen(c4), widen(c1) * 4.0)


# ---------------------------------------------------------------------------- the headline configurations

def test_config1_golden(af, golden_dir):
    g = np.load(f"{golden_dir}/c1_seed0.npz")
    p = Problem(64, 128, 256)
    p.a_bf, p.b_bytes, p.s_bf = g["a_bf"], g["b_bytes"], g["s_bf"].reshape(1, -1)
    c = run_gemm(p)
    # fixture output = the reference's gemm_rrr on (bf16 A, bf16 W, unit scales); no near-zero escape here
    bad, worst, _ = oracle.check_ulp(g["c_oracle"], c)
    assert bad == 0, (bad, worst)
    assert np.array_equal(p.w_bf, g["w_bf"])


@pytest.mark.parametrize("m", [1, 4, 8, 16, 32])
def test_config2_and_3_decode(af, m):
    for n in (4096, 11008):
        p = Problem(m, n, 4096, seed=m)
        c = run_gemm(p)
        assert af.variant(m, n, 4096) == af.DECODE
        assert_close_ulp(p, c, f"decode m={m} n={n}")


def test_config4_prefill_full_size(af):
    p = Problem(4096, 4096, 4096, seed=4)
    c = run_gemm(p)
    worst, near_zero = assert_close_ulp(p, c, "prefill 4096^3", threads=16)
    print(f"prefill 4096^3: worst {worst:.3f} ULP, {near_zero} near-zero outputs beyond 2 ULP (within fp32 summation noise)")


@pytest.mark.parametrize("m", [1, 16])
def test_config5_int4_group128_decode(af, m):
    p = Problem(m, 28672, 8192, 4, 128, seed=50 + m, scale_lo=0.001, scale_hi=0.02)
    c = run_gemm(p)
    assert_close_ulp(p, c, f"int4 g128 m={m}", threads=16)


def test_config5_int4_group128_prefill_rows(af):
    m = 2048
    p = Problem(m, 28672, 8192, 4, 128, seed=52, scale_lo=0.001, scale_hi=0.02)
    c = run_gemm(p)
    rows = np.arange(5, m, 16)  # 128 rows touching every 32-row MFMA block of every tile
    assert_close_ulp(p, np.ascontiguousarray(c[rows]), "int4 g128 m=2048 (row sample)", rows=rows, threads=16)


# ---------------------------------------------------------------------------- shapes, strides, split-K

@pytest.mark.parametrize("m,n,k", [(3, 16, 64), (17, 48, 128), (33, 272, 64), (257, 528, 192), (100, 1040, 320), (31, 4112, 2048)])
@pytest.mark.parametrize("bits,group", [(8, 0), (4, 64)])
def test_ragged_shapes(af, m, n, k, bits, group):
    p = Problem(m, n, k, bits, group, seed=m * 7 + n)
    c = run_gemm(p)
    assert_close_ulp(p, c, f"ragged {m}x{n}x{k} bits={bits}")


@pytest.mark.parametrize("m,n,k", [(17, 48, 128), (257, 528, 192), (100, 1040, 320), (300, 272, 448), (1000, 1008, 384), (130, 4112, 256)])
@pytest.mark.parametrize("bits,group", [(8, 0), (8, 64), (4, 0), (4, 64)])
@pytest.mark.parametrize("tile", [256, 128])
def test_tiled_kernels_on_ragged_shapes(af, m, n, k, bits, group, tile):
    """The tiled variant with either tile size forced: partial tiles in m and n, odd numbers of K-steps, column counts
    that end inside a 16-column block of a tile."""
    p = Problem(m, n, k, bits, group, seed=m * 3 + n + tile)
    assert_close_ulp(p, run_gemm(p, which=af.PREFILL_256 if tile == 256 else af.PREFILL_128), f"tile {tile}: {m}x{n}x{k} bits={bits} g={group}")


@pytest.mark.parametrize("m,n,k,bits,group", [(4160, 256, 256, 8, 0), (1000, 1008, 384, 4, 0), (300, 528, 512, 8, 64), (130, 4112, 256, 4, 128)])
def test_tile_sizes_agree_bit_for_bit(af, m, n, k, bits, group):
    """The 256x256 tiles and the 128x128 tiles that stage both operands in LDS add the products of an output in the same
    order (ascending k through one chain of matrix instructions), so they must agree in every bit, near-cancelling
    outputs included: an indexing slip in either one shows here even where it would stay inside the 2-ULP bound.  (The
    128x128 form with the weights in registers adds in an order of its own: test_small_tile_forms_agree.)"""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    assert np.array_equal(run_gemm(p, which=af.PREFILL_128_LDS), run_gemm(p, which=af.PREFILL_256))


@pytest.mark.parametrize("m,n,k,bits,group", [(130, 272, 72, 8, 0), (700, 1008, 1000, 8, 0), (300, 528, 512, 8, 64), (1000, 1008, 384, 4, 0),
                                              (130, 4112, 256, 4, 128), (1024, 4096, 1088, 8, 0), (257, 272, 8, 4, 0)])
def test_small_tile_forms_agree(af, m, n, k, bits, group):
    """The 128x128-tile kernel that keeps the weights in registers (row-major weights: what PREFILL_128 runs) against the
    one that stages both operands in LDS: the same products; the register form has two waves per column group, one per
    block of 32 k of a K-step, and adds the two waves' sums at the end, so its order of addition is its own — both meet
    the oracle, and the two agree except where a bf16 rounding boundary falls between two fp32 sums that differ in their
    last bits.  Partial tiles in m and n, K-steps that are not whole, one to seventeen steps, both code widths, grouped
    scales."""
    p = Problem(m, n, k, bits, group, seed=m + 2 * n + k)
    c = run_gemm(p, which=af.PREFILL_128, force_split_k=1)
    assert_close_ulp(p, c, f"128-tile, weights in registers: {m}x{n}x{k} bits={bits} g={group}")
    c_lds = run_gemm(p, which=af.PREFILL_128_LDS)
    assert_close_ulp(p, c_lds, f"128-tile, LDS form: {m}x{n}x{k} bits={bits} g={group}")
    assert np.array_equal(c, run_gemm(p, which=af.PREFILL_128, force_split_k=1)), "not reproducible"
    assert np.mean(c != c_lds) < 2e-3, f"{np.mean(c != c_lds):.2e} of the outputs differ between the two forms"


@pytest.mark.parametrize("m,n,k,bits,group,which", [
    (1, 256, 960, 8, 96, "AUTO"), (16, 528, 1920, 4, 160, "AUTO"), (40, 512, 1920, 4, 160, "AUTO"), (100, 1040, 2240, 8, 224, "AUTO"),
    (300, 272, 960, 8, 96, "PREFILL_128"), (300, 272, 960, 8, 96, "PREFILL_256"), (300, 528, 1920, 4, 160, "PREFILL_128_LDS"),
    (300, 528, 1920, 4, 160, "PREFILL_256_LDS"), (520, 272, 1120, 8, 224, "PREFILL_256X128"), (130, 4112, 672, 4, 96, "PREFILL_256")])
def test_scale_groups_that_are_no_power_of_two(af, m, n, k, bits, group, which):
    """The kernels find the scale group of a block of 32 rows by a multiplication the host prepares from the group size;
    group sizes that are no power of two (any multiple of 32 that divides k is allowed) take the general form of it."""
    p = Problem(m, n, k, bits, group, seed=m + n + k + group)
    assert_close_ulp(p, run_gemm(p, which=getattr(af, which)), f"{which}: {m}x{n}x{k} bits={bits} g={group}")


def test_tiled_variant_picks_its_tile_size_by_shape(af):
    """PREFILL runs 128x128 tiles while m x n holds at most 256 of them, then tiles of 256 rows x 128 columns while those
    are at most 256, 256x256 tiles beyond; every time the result meets the oracle and is the forced form's, bit for bit."""
    for (m, n, rows, cols) in [(1024, 4096, 128, 128), (2048, 2048, 128, 128), (2064, 2048, 256, 128), (1024, 4224, 256, 128), (2048, 4096, 256, 128),
                               (2064, 4096, 256, 256), (520, 16512, 256, 256)]:
        assert (af.prefill_tile(m, n), af.prefill_tile_cols(m, n)) == (rows, cols)
        p = Problem(m, n, 256, 8, 0, seed=m + n)
        c = run_gemm(p, which=af.PREFILL)
        assert_close_ulp(p, c, f"{m}x{n}")
        forced = af.PREFILL_128 if rows == 128 else af.PREFILL_256X128 if cols == 128 else af.PREFILL_256
        assert np.array_equal(c, run_gemm(p, which=forced, force_split_k=1)), f"{m}x{n}"
    # two rounds of 128x128 tiles: where 256x128 tiles just miss one round and 256x256 ones would use half the machine
    # (8-bit codes, 640 x 11008: 430 tiles), and for 4-bit codes up to 345 tiles (1152 x 4096: 288)
    # and one row of them however many: 256-row tiles would be half empty or worse (96 x 36992: 289 tiles; 40 x 50304, 4-bit: 393)
    for (m, n, bits, group, tiles) in [(640, 11008, 8, 0, 430), (1152, 4096, 4, 128, 288), (1152, 4096, 8, 0, 0), (96, 36992, 8, 0, 289),
                                       (40, 50304, 4, 128, 393)]:
        pl = af.plan(m, n, 256, bits, group, which=af.PREFILL)
        assert (pl.tile_rows, pl.tile_cols, pl.workgroups) == ((128, 128, tiles) if tiles else (256, 128, 160))
        p = Problem(m, n, 256, bits, group, seed=m + n + bits)
        c = run_gemm(p, which=af.PREFILL)
        assert_close_ulp(p, c, f"{m}x{n} b{bits}")
        if tiles:
            assert np.array_equal(c, run_gemm(p, which=af.PREFILL_128, force_split_k=1)), f"{m}x{n} b{bits}"


@pytest.mark.parametrize("m,n,k,bits,group", [(256, 128, 64, 8, 0), (300, 272, 448, 8, 0), (700, 1008, 1000, 8, 0), (1000, 1008, 384, 4, 0), (520, 528, 512, 8, 64),
                                              (130, 4112, 256, 4, 128), (257, 272, 8, 4, 0), (2048, 512, 1088, 8, 0), (17, 48, 128, 4, 64)])
def test_tall_tiles_agree_with_the_large_ones_bit_for_bit(af, m, n, k, bits, group):
    """Tiles of 256 rows x 128 columns (two waves by two, each converting the weights of its 64 columns) against the 256x256
    tiles: same products, same order of addition, so the same bits — partial tiles in m and n, K-steps that are not
    whole, one to seventeen steps, both code widths, grouped scales; and the oracle's tolerance on top."""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    c = run_gemm(p, which=af.PREFILL_256X128)
    assert_close_ulp(p, c, f"256x128 tiles: {m}x{n}x{k} bits={bits} g={group}")
    assert np.array_equal(c, run_gemm(p, which=af.PREFILL_256))


def test_tall_tiles_take_the_epilogues(af):
    """A shape PREFILL runs on tiles of 256 rows x 128 columns, through the fused entry point: bias and residual, then the
    SiLU gate (the kernel finishes 128 rows at a time from fp32 sums staged in LDS)."""
    m, n, k = 2100, 2048, 320
    assert af.variant(m, n, k) == af.PREFILL and (af.prefill_tile(m, n), af.prefill_tile_cols(m, n)) == (256, 128)
    p = Problem(m, n, k, 8, 0, seed=71).with_bias().with_residual()
    assert_close_ulp(p, run_gemm(p), "bias + residual")
    g = gated_problem(m, n, k, 4, 64, seed=72).with_bias()
    assert_close_gated(g, run_gemm(g, activation=af.ACT_SILU_GATE), "gated")


@pytest.mark.parametrize("m,n,k,bits,group", [(130, 272, 1000, 8, 0), (256, 1040, 2048, 8, 64), (100, 528, 4096, 4, 128), (300, 272, 1088, 4, 0),
                                              (64, 4096, 4096, 8, 0)])
def test_tiled_split_k_matches_oracle_and_is_deterministic(af, m, n, k, bits, group):
    """The 128x128-tile kernel with k split between workgroups: every split factor meets the oracle (shares of whole
    64-row steps; a last step that is not whole; as many splits as steps; more splits asked for than steps exist), the
    same factor gives the same bits every time, whatever order the workgroups arrived in, and the workspace is left at
    rest."""
    import helpers
    p = Problem(m, n, k, bits, group, seed=m + n + k + 1)
    steps = (k + 63) // 64
    for split in (2, 3, 5, 16):
        need = af.workspace_bytes(m, n, k, bits, group, af.PREFILL_128, split)
        per = -(-steps // min(split, 16))
        runs = -(-steps // per)  # splits that really run
        assert need == (256 + (((runs - 1) * m * n * 4 + 255) & ~255) if runs > 1 else 0)
        c = run_gemm(p, which=af.PREFILL_128, force_split_k=split)
        assert_close_ulp(p, c, f"128-tile split_k={split}: {m}x{n}x{k} bits={bits} g={group}")
        for _ in range(2):
            assert np.array_equal(run_gemm(p, which=af.PREFILL_128, force_split_k=split), c), f"split_k={split} not reproducible"
        assert bool((helpers._ws.t[256:] == 0xFF).all()), f"workspace not at rest after split_k={split}"
        assert af.workspace_status(helpers._ws.t) == 0


@pytest.mark.parametrize("m,n,k,group", [(1, 2048, 1024, 128), (5, 2432, 512, 0), (20, 4224, 1024, 64), (33, 4112, 512, 128), (16, 6144, 2048, 128)])
def test_4bit_128_column_form_gives_the_halves_of_a_line_to_paired_workgroups(af, m, n, k, group):
    """4-bit codes in rows, 128 columns per workgroup: within every whole run of 16 column blocks the kernel hands blocks
    2j and 2j + 1 (the two halves of a 128-byte line) to workgroups 8 apart; blocks past the last whole run keep their
    order.  One run, a run and a remainder, two runs and a partial last block, three runs: the oracle's bound."""
    p = Problem(m, n, k, 4, group, seed=m + n + k)
    assert af.plan(m, n, k, 4, group, which=af.DECODE).tile_cols == 128
    assert_close_ulp(p, run_gemm(p, which=af.DECODE), f"4-bit 128-column form {m}x{n}x{k} g{group}")


@pytest.mark.parametrize("m,n,k", [(1, 1024, 4096), (16, 640, 2048), (9, 2064, 4096)])
def test_decode_hand_over_leaves_the_workspace_at_rest_for_every_split_factor(af, m, n, k):
    """The reducer of the 128-column decode kernels keeps two fetch attempts in flight and has one instantiation per
    number of splits it fetches (1, 2, up to 4, up to 7 others); beyond 8 splits the single-attempt form runs.  Every
    split factor: the oracle's bound, the same bits on every run, and every workspace word empty again afterwards
    (an attempt still in flight when the words are emptied must not disturb the emptying stores)."""
    import torch
    p = Problem(m, n, k, seed=m + n)
    a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
    for split in (2, 3, 4, 5, 7, 8, 16):
        need = af.workspace_bytes(m, n, k, which=af.DECODE, force_split_k=split)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        af.workspace_init(ws)
        c = torch.zeros((m, n), dtype=torch.int16, device="cuda")
        first = None
        for rep in range(20):
            af.gemm(c, a, b, s, m, n, k, workspace=ws, which=af.DECODE, force_split_k=split)
            torch.cuda.synchronize()
            got = from_dev_u16(c).copy()
            if first is None:
                first = got
                assert_close_ulp(p, got, f"decode, k split {split} ways: {m}x{n}x{k}")
            assert np.array_equal(got, first), f"split {split}, run {rep}: not reproducible"
            assert bool((ws[256:] == 0xFF).all()), f"split {split}, run {rep}: workspace not at rest"
        assert af.workspace_status(ws) == 0


def test_tiled_split_k_is_what_auto_runs_and_takes_the_epilogues(af):
    """A shape whose plan is the small tiles with k split (long k, few tiles): AUTO gives the forced form's bits, and the
    bias / residual / gate epilogues run on the reduced sums."""
    m, n, k = 384, 2048, 8192
    assert af.variant(m, n, k) == af.PREFILL and af.prefill_tile(m, n) == 128
    split = af.split_k(m, n, k)
    assert split > 1 and af.workspace_bytes(m, n, k) == 256 + (split - 1) * m * n * 4
    p = Problem(m, n, k, seed=61)
    c = run_gemm(p)
    assert_close_ulp(p, c, "auto")
    assert np.array_equal(c, run_gemm(p, which=af.PREFILL_128, force_split_k=split))
    assert not np.array_equal(c, run_gemm(p, which=af.PREFILL_128, force_split_k=1)), "the split changes the order of addition"
    p.with_bias().with_residual()
    assert_close_ulp(p, run_gemm(p), "auto, bias + residual")
    g = gated_problem(m, n, k, 8, 0, seed=62).with_bias()
    assert_close_gated(g, run_gemm(g, activation=af.ACT_SILU_GATE), "auto, gated")


def test_tiled_split_k_gives_up_like_the_decode_family(af):
    """The bounded wait of the tiled kernel's reducing workgroups, driven from the host as in the decode family's test:
    producers keep their sums, the attempts are capped: NaNs, a poisoned header, and all well after initialisation."""
    import torch
    p = Problem(130, 272, 1024, seed=63)
    need = af.workspace_bytes(p.m, p.n, p.k, which=af.PREFILL_128, force_split_k=4)
    raw = torch.empty(need, dtype=torch.uint8, device="cuda")
    af.workspace_init(raw)
    a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
    c = torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda")
    run = lambda: (af.gemm(c, a, b, s, p.m, p.n, p.k, workspace=raw, which=af.PREFILL_128, force_split_k=4), torch.cuda.synchronize())
    run()
    good = from_dev_u16(c).copy()
    assert_close_ulp(p, good, "before")
    try:
        af.debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 3)
        af.debug_control(af.DEBUG_WITHHOLD_PARTIALS, 1)
        run()
    finally:
        af.debug_control(af.DEBUG_WITHHOLD_PARTIALS, 0)
        af.debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 0)
    assert np.isnan(widen(from_dev_u16(c))).all(), "every output misses partial sums: all NaN"
    assert af.workspace_status(raw) == af.ERR_WORKSPACE_POISONED
    af.workspace_init(raw)
    run()
    assert af.workspace_status(raw) == 0
    assert np.array_equal(from_dev_u16(c), good)


def test_forced_row_block_changes_the_plan_not_the_contract(af):
    """The tuning hook that pins the decode family's row-block size: every size meets the oracle, and the hook's 0 restores
    the library's own choice (same bits as before)."""
    p = Problem(100, 1040, 512, 8, 0, seed=11)
    own = run_gemm(p, which=af.DECODE)
    try:
        for mb in (1, 2, 4):
            af.debug_control(af.DEBUG_FORCE_ROW_BLOCK, mb)
            assert_close_ulp(p, run_gemm(p, which=af.DECODE), f"row blocks of {16 * mb}")
    finally:
        af.debug_control(af.DEBUG_FORCE_ROW_BLOCK, 0)
    assert np.array_equal(own, run_gemm(p, which=af.DECODE))


@pytest.mark.parametrize("m", [5, 80])
def test_leading_dimensions_and_untouched_padding(af, m):
    import torch
    n, k, lda, ldb, ldc = 272, 256, 264, 288, 280
    p = Problem(m, n, k, seed=m)
    a_pad = np.full((m, lda), 0x7FC0, np.uint16); a_pad[:, :k] = p.a_bf
    b_pad = np.full((k, ldb), 0xAB, np.uint8); b_pad[:, :n] = p.b_bytes
    c = run_gemm(p, lda=lda, ldb=ldb, ldc=ldc, a_dev=to_dev(a_pad), b_dev=to_dev(b_pad), c_fill=0x1234)
    assert_close_ulp(p, np.ascontiguousarray(c[:, :n]), "strided")
    assert (c[:, n:] == 0x1234).all(), "columns beyond n were written"


def test_split_k_is_deterministic_and_consistent(af):
    p = Problem(7, 768, 4096, seed=12)
    outs = {}
    for split in (1, 2, 5, 32):
        c = run_gemm(p, which=af.DECODE, force_split_k=split)
        assert_close_ulp(p, c, f"split_k={split}")
        for _ in range(3):  # same split: same bits, whatever order the workgroups arrived in
            assert np.array_equal(run_gemm(p, which=af.DECODE, force_split_k=split), c)
        outs[split] = c


def test_workspace_is_left_ready_for_the_next_call(af):
    # one workspace, back-to-back calls of different shapes and split factors, no re-initialisation
    import helpers
    shapes = [(1, 4096, 4096), (16, 1024, 8192), (32, 272, 512), (1, 4096, 4096)]
    for i, (m, n, k) in enumerate(shapes):
        p = Problem(m, n, k, seed=i)
        assert_close_ulp(p, run_gemm(p), f"call {i}")
        # every word behind the 256-byte header is back to "no partial sum here" (all bits set); the header says "healthy"
        assert bool((helpers._ws.t[256:] == 0xFF).all()), f"workspace not restored after call {i}"
        assert af.workspace_status(helpers._ws.t) == 0


def test_workspace_status_and_the_give_up_path(af):
    """The reducer's bounded wait, driven from the host so that every kernel exits normally: the producing workgroups are
    told to keep their sums (a test hook), the reducer's attempts are capped at a few, so it gives up: the output holds
    NaNs, the workspace's header records it until the workspace is initialised again, and then everything works."""
    import torch
    p = Problem(4, 1024, 4096, seed=5)
    need = af.workspace_bytes(p.m, p.n, p.k)
    assert need > 256 and af.split_k(p.m, p.n, p.k) > 1
    raw = torch.zeros(need, dtype=torch.uint8, device="cuda")
    assert af.workspace_status(raw) == af.ERR_WORKSPACE            # arbitrary memory: never initialised
    af.workspace_init(raw)
    assert af.workspace_status(raw) == 0
    a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
    c = torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda")
    af.gemm(c, a, b, s, p.m, p.n, p.k, workspace=raw)
    torch.cuda.synchronize()
    good = from_dev_u16(c).copy()
    assert_close_ulp(p, good, "before")
    assert af.workspace_status(raw) == 0
    try:
        af.debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 3)
        af.debug_control(af.DEBUG_WITHHOLD_PARTIALS, 1)
        af.gemm(c, a, b, s, p.m, p.n, p.k, workspace=raw)
        torch.cuda.synchronize()
    finally:
        af.debug_control(af.DEBUG_WITHHOLD_PARTIALS, 0)
        af.debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 0)
    bad = from_dev_u16(c)
    assert np.isnan(widen(bad)).all(), "every output misses partial sums: all NaN"
    assert af.workspace_status(raw) == af.ERR_WORKSPACE_POISONED
    assert af.workspace_status(raw) == af.ERR_WORKSPACE_POISONED   # sticky
    af.workspace_init(raw)
    assert af.workspace_status(raw) == 0
    af.gemm(c, a, b, s, p.m, p.n, p.k, workspace=raw)
    torch.cuda.synchronize()
    assert np.array_equal(from_dev_u16(c), good)


def test_prefill_variant_on_small_m_matches_decode(af):
    p = Problem(24, 512, 1024, seed=77)
    assert_close_ulp(p, run_gemm(p, which=af.PREFILL), "prefill kernel at m=24")
    assert_close_ulp(p, run_gemm(p, which=af.DECODE), "decode kernel at m=24")


@pytest.mark.parametrize("m,n,k,bits,group,split", [
    (33, 272, 512, 8, 0, 0),        # one row past two 16-row blocks: row blocks of 64, ragged columns
    (64, 512, 1024, 8, 0, 0),
    (100, 4096, 4096, 8, 0, 0),     # two row blocks of 64, the second ragged; split-K
    (200, 1040, 2048, 8, 128, 3),   # four row blocks, group scales, forced odd split
    (48, 1024, 2048, 4, 128, 0),    # 4-bit codes: row blocks of 32
    (130, 528, 1024, 4, 0, 2),
    (5000, 256, 256, 8, 0, 0),      # very tall A: thousands of row blocks along grid z
    (20000, 128, 128, 4, 64, 0),
])
def test_decode_family_with_row_blocks_matches_oracle(af, m, n, k, bits, group, split):
    """The decode kernel forced onto m > 32: grid z walks blocks of rows; each must agree with the oracle and,
    within tolerance of the summation order, with the prefill kernel on the same problem."""
    p = Problem(m, n, k, bits, group, seed=300 + m)
    c = run_gemm(p, which=af.DECODE, force_split_k=split)
    assert_close_ulp(p, c, f"decode family m={m}")
    assert np.array_equal(run_gemm(p, which=af.DECODE, force_split_k=split), c), "not reproducible"


@pytest.mark.parametrize("m,n,k,bits,group", [
    (1, 4096, 4096, 8, 0),      # decode, split-K: the bias joins in the reducing workgroup
    (16, 528, 512, 4, 128),     # decode without split-K
    (100, 1040, 1024, 8, 0),    # decode family in row blocks
    (300, 784, 512, 8, 128),    # prefill kernel, ragged tile edges
    (4096, 512, 256, 4, 0),
])
def test_fused_bias(af, m, n, k, bits, group):
    """bfaintb_gemm_bias: C = bf16(sum + bias).  Checked against the oracle's fp32 sums plus the bias, and through
    two closed forms: zero activations return the bias itself, and a zero bias returns bfaintb_gemm's bits."""
    p = Problem(m, n, k, bits, group, seed=700 + m).with_bias(seed=m)
    assert_close_ulp(p, run_gemm(p), f"bias m={m}")
    plain = Problem(m, n, k, bits, group, seed=700 + m)
    c_plain = run_gemm(plain)
    p.bias_bf = np.zeros(n, np.uint16)
    c_zero_bias = run_gemm(p)
    # x + (+0) == x except that -0 becomes +0
    assert np.array_equal(np.where(c_plain == 0x8000, 0, c_plain), c_zero_bias)
    p.with_bias(seed=m)
    p.a_bf = np.zeros_like(p.a_bf)
    assert np.array_equal(run_gemm(p), np.broadcast_to(p.bias_bf, (m, n)))


@pytest.mark.parametrize("m,n,k,bits,group", [
    (1, 4096, 4096, 8, 0),      # decode, split-K: the reducing workgroup adds the residual
    (7, 528, 1024, 4, 128),     # decode, 4-bit
    (24, 272, 512, 8, 0),       # decode, no split
    (80, 1040, 2048, 8, 64),    # row-blocked decode family
    (300, 272, 192, 8, 0),      # row-blocked family, ragged rows and columns
    (4200, 272, 256, 8, 0),     # tiled kernel (128x128 tiles), ragged rows and columns, half tiles
    (4200, 528, 256, 4, 128),   # tiled kernel (128x128 tiles), 4-bit
    (4200, 1040, 128, 8, 0),    # more than 256 small tiles: 256x256 tiles, ragged rows and columns
    (4200, 1296, 256, 4, 128),  # 256x256 tiles, 4-bit
    (40, 33024, 256, 8, 0),     # one row of 258 small tiles in their 64-row form
    (33, 16512, 8192, 8, 0),    # ... of 129 with k split three ways: the reducing workgroups add bias and residual
])
def test_fused_residual(af, m, n, k, bits, group):
    """C = bf16(sum + bias + residual): against the oracle's fp32 sums plus the two fp32 additions, with and without the
    bias, and in place (residual == c)."""
    import torch
    p = Problem(m, n, k, bits, group, seed=m + k).with_residual()
    assert_close_ulp(p, run_gemm(p), f"residual {m}x{n}x{k}")
    p.with_bias()
    want = run_gemm(p)
    assert_close_ulp(p, want, f"bias + residual {m}x{n}x{k}")
    # in place: the residual is the output buffer
    from helpers import Workspace
    c = to_dev(p.residual_bf).clone()
    ws = Workspace().get(af.workspace_bytes(m, n, k, bits, group))
    af.gemm(c, to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf), m, n, k, weight_bits=bits, group_size=group, workspace=ws,
            bias=to_dev(p.bias_bf), residual=c)
    torch.cuda.synchronize()
    assert np.array_equal(from_dev_u16(c), want)


def test_residual_closed_forms(af):
    """Zero activations: C = bf16(bias + residual) exactly; zero residual: the bits of the bias-only call."""
    p = Problem(40, 272, 256, seed=8).with_bias().with_residual()
    base = Problem(40, 272, 256, seed=8).with_bias()
    p.a_bf = np.zeros_like(p.a_bf)
    want = oracle.f32_to_bf16_rne((widen(p.bias_bf)[None, :] + widen(p.residual_bf)).astype(np.float32))
    assert np.array_equal(run_gemm(p), want)
    q = Problem(40, 272, 256, seed=8).with_bias().with_residual()
    q.residual_bf = np.zeros_like(q.residual_bf)
    got, ref = run_gemm(q), run_gemm(base)
    assert np.array_equal(got & 0x7FFF, ref & 0x7FFF) and np.all((got == ref) | ((ref & 0x7FFF) == 0))  # up to the sign of zero


GATED_SHAPES = [
    (1, 4096, 4096, 8, 0),      # decode, split-K
    (7, 544, 1024, 4, 128),     # decode, 4-bit
    (24, 288, 512, 8, 0),       # decode, no split
    (80, 1056, 2048, 8, 64),    # row-blocked decode family
    (4200, 288, 256, 8, 0),     # tiled kernel (128x128 tiles), ragged rows and columns, half tiles
    (4200, 544, 256, 4, 128),   # tiled kernel (128x128 tiles), 4-bit
    (4200, 1056, 128, 8, 0),    # more than 256 small tiles: 256x256 tiles
    (4200, 1312, 256, 4, 128),  # 256x256 tiles, 4-bit
    (40, 33024, 256, 8, 0),     # one row of 258 small tiles in their 64-row form
]


def gated_problem(m, n, k, bits, group, seed):
    # sums of a few units, so that silu is exercised on both sides of zero and in its curved part
    return Problem(m, n, k, bits, group, seed=seed, scale_lo=0.002, scale_hi=0.02 if bits == 8 else 0.2)


@pytest.mark.parametrize("m,n,k,bits,group", GATED_SHAPES)
def test_silu_gate_epilogue(af, m, n, k, bits, group):
    """C[m, j] = bf16(silu(S[m, 2j]) * S[m, 2j+1] (+ residual)), S = A.W + bias: against fp64 arithmetic on the oracle's
    fp32 sums, with the tolerance gated_reference states."""
    p = gated_problem(m, n, k, bits, group, seed=m + k)
    c = run_gemm(p, activation=af.ACT_SILU_GATE)
    assert c.shape == (m, n // 2)
    assert_close_gated(p, c, f"gated {m}x{n}x{k}")
    p.with_bias()
    p.residual_bf = oracle.f32_to_bf16_rne(np.random.default_rng(3).uniform(-2, 2, size=(m, n // 2)).astype(np.float32))
    worst = assert_close_gated(p, run_gemm(p, activation=af.ACT_SILU_GATE), f"gated + bias + residual {m}x{n}x{k}")
    print(f"gated {m}x{n}x{k}: worst {worst:.2f} x tolerance")


def test_silu_gate_closed_forms(af):
    """What the mathematics fixes, independent of the oracle's formula: with zero up-weights and an up-bias of 1 the output
    is silu(gate) (checked against torch's own silu on exactly known gates); a zero gate gives 0; a large gate lets the
    up value through; a very negative one gives 0."""
    import torch
    m, n, k = 8, 32, 64
    p = Problem(m, n, k, 8, 0, seed=1)
    gates = np.array([-30.0, -4.0, -1.0, -0.25, 0.0, 0.5, 2.0, 40.0], np.float32)
    a = np.zeros((m, k), np.float32)
    a[:, 0] = gates                                   # A[i, 0] = gate_i, everything else 0
    p.a_bf = oracle.f32_to_bf16_rne(a)
    q = np.zeros((k, n), np.int8)
    q[0, 0::2] = 64                                   # gate columns: W[0, 2j] = 64 * (1/64) = 1, so S[i, 2j] = gate_i
    p.q = q
    p.b_bytes = oracle.mem_transfer_int8(q.astype(np.float32))
    p.s_bf = oracle.f32_to_bf16_rne(np.full((1, n), 1.0 / 64, np.float32))
    p._w = None
    bias = np.zeros(n, np.float32)
    bias[1::2] = 1.0                                  # up columns: S[i, 2j+1] = 0 + 1
    p.bias_bf = oracle.f32_to_bf16_rne(bias)
    c = widen(run_gemm(p, activation=af.ACT_SILU_GATE))
    want = torch.nn.functional.silu(torch.from_numpy(gates)).to(torch.bfloat16).float().numpy()
    for j in range(n // 2):
        assert np.allclose(c[:, j], want, rtol=2 ** -7, atol=1e-12), (c[:, j], want)
    assert np.all(c[4] == 0.0) and np.all(np.abs(c[0]) < 1e-11) and np.all(c[7] == 40.0)


def test_row_permutation_permutes_output(af):
    # size-independent property at a prefill shape: rows of A are independent
    p = Problem(512, 512, 512, seed=5)
    c = run_gemm(p)
    perm = np.random.Generator(np.random.PCG64(1)).permutation(512)
    p.a_bf = p.a_bf[perm]
    assert np.array_equal(run_gemm(p), c[perm])


def test_hip_graph_replays_match_eager(af):
    """The path holds no memset and leaves its workspace as it found it (every word empty again), so it can be
    captured once and replayed: every replay must reproduce the eager result, with other work and
    synchronisations in between."""
    import torch
    from helpers import Workspace
    shapes = [(1, 4096, 4096, 8, 0), (4, 1040, 2048, 4, 128), (16, 768, 1024, 8, 0), (96, 512, 512, 8, 0),
              (4200, 272, 256, 8, 0), (4200, 1040, 128, 4, 64),   # the tiled kernels: 128x128 tiles, 256x256 tiles (two launches)
              (384, 2048, 8192, 8, 0)]                            # 128x128 tiles with k split (partial sums through the workspace)
    probs = [Problem(m, n, k, bits, g, seed=90 + i) for i, (m, n, k, bits, g) in enumerate(shapes)]
    eager = [run_gemm(p) for p in probs]
    ws = Workspace()
    bufs = []
    for p in probs:
        need = af.workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size)
        bufs.append(dict(a=to_dev(p.a_bf), b=to_dev(p.b_bytes), s=to_dev(p.s_bf),
                         c=torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda"),
                         w=None if need == 0 else torch.empty(need, dtype=torch.uint8, device="cuda")))
        if need:
            af.workspace_init(bufs[-1]["w"])
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):  # warm up on the capture stream's device (lazy kernel attributes), then capture
        for p, d in zip(probs, bufs):
            af.gemm(d["c"], d["a"], d["b"], d["s"], p.m, p.n, p.k, weight_bits=p.bits, group_size=p.group_size, workspace=d["w"])
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for p, d in zip(probs, bufs):
            af.gemm(d["c"], d["a"], d["b"], d["s"], p.m, p.n, p.k, weight_bits=p.bits, group_size=p.group_size, workspace=d["w"])
    for replay in range(4):
        for d in bufs:
            d["c"].fill_(0x7FC0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for i, (p, d) in enumerate(zip(probs, bufs)):
            assert np.array_equal(from_dev_u16(d["c"]), eager[i]), f"replay {replay}, problem {i}"
        # unrelated eager work on the same workspaces between replays
        af.gemm(bufs[0]["c"], bufs[0]["a"], bufs[0]["b"], bufs[0]["s"], 1, 4096, 4096, workspace=bufs[0]["w"])
        torch.cuda.synchronize()


def test_two_streams_with_their_own_workspaces(af):
    """Launches are stream-ordered and keep no state outside their arguments: GEMMs issued alternately on two streams,
    each stream with its own workspace and output, give the single-stream results."""
    import torch
    # (the last shape runs the small tiles with k split: 192 workgroups of one per CU, so two launches in flight compete
    # for CUs while their reducing workgroups wait — for workgroups that wait for nothing, hence never for long)
    shapes = [(1, 4096, 4096, 8, 0), (8, 1040, 4096, 4, 128), (200, 528, 1024, 8, 0), (4200, 272, 256, 8, 0), (384, 2048, 8192, 8, 0)]
    assert af.variant(384, 2048, 8192) == af.PREFILL and af.split_k(384, 2048, 8192) > 1
    probs = [Problem(m, n, k, bits, g, seed=300 + i) for i, (m, n, k, bits, g) in enumerate(shapes)]
    want = [run_gemm(p) for p in probs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    bufs = []
    for si in range(2):
        for p in probs:
            need = af.workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size)
            w = None if need == 0 else torch.empty(need, dtype=torch.uint8, device="cuda")
            if need:
                af.workspace_init(w)
            bufs.append(dict(a=to_dev(p.a_bf), b=to_dev(p.b_bytes), s=to_dev(p.s_bf), w=w,
                             c=torch.full((p.m, p.n), 0x7FC0, dtype=torch.int16, device="cuda")))
    torch.cuda.synchronize()
    for rep in range(3):
        for i, p in enumerate(probs):
            for si, st in enumerate(streams):
                d = bufs[si * len(probs) + i]
                with torch.cuda.stream(st):
                    af.gemm(d["c"], d["a"], d["b"], d["s"], p.m, p.n, p.k, weight_bits=p.bits, group_size=p.group_size, workspace=d["w"])
    torch.cuda.synchronize()
    for si in range(2):
        for i in range(len(probs)):
            assert np.array_equal(from_dev_u16(bufs[si * len(probs) + i]["c"]), want[i]), f"stream {si}, problem {i}"


def test_empty_and_minimal_shapes(af):
    import torch
    p = Problem(1, 16, 64, seed=1)       # the smallest shape the library takes
    assert_close_ulp(p, run_gemm(p), "1x16x64")
    a = torch.zeros(16, dtype=torch.int16, device="cuda")
    assert af.gemm(a, a, a, a, 0, 16, 64) == 0     # m = 0: nothing to do, nothing launched
    assert af.gemm(a, a, a, a, 4, 0, 64) == 0      # n = 0
    torch.cuda.synchronize()


def test_first_call_under_capture_is_refused_until_init():
    """A fresh process whose first library call comes under stream capture: the call is refused (the per-device set-up
    makes runtime calls that are not stream operations) and nothing is recorded; after bfaintb_init the same capture
    works and replays correctly."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import sys
sys.path.insert(0, %r); sys.path.insert(0, %r)
import numpy as np, torch
import awesome_fusion_amd as af
from helpers import Problem, to_dev, from_dev_u16, assert_close_ulp
p = Problem(4, 1024, 4096, seed=3)
a, b, s = to_dev(p.a_bf), to_dev(p.b_bytes), to_dev(p.s_bf)
c = torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda")
ws = torch.empty(af.workspace_bytes(p.m, p.n, p.k), dtype=torch.uint8, device="cuda")
torch.cuda.synchronize()
g = torch.cuda.CUDAGraph()
with torch.cuda.graph(g):
    rc_ws = af.lib().bfaintb_workspace_init(ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    rc = af.gemm(c, a, b, s, p.m, p.n, p.k, workspace=ws, check=False)
    rc_static = af.gemm_static(c, a, b, s, p.m, p.n, p.k, check=False)
assert rc_ws == 0 and rc == af.ERR_NOT_INITIALISED and rc_static == af.ERR_NOT_INITIALISED, (rc_ws, rc, rc_static)
g.replay()   # what was recorded: the workspace's initialisation (fill kernels), nothing of the refused calls
torch.cuda.synchronize()
assert af.workspace_status(ws) == 0
af.init()
g2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(g2):
    af.gemm(c, a, b, s, p.m, p.n, p.k, workspace=ws)
for rep in range(3):
    c.zero_()
    g2.replay()
    torch.cuda.synchronize()
    assert_close_ulp(p, from_dev_u16(c), "replay %%d" %% rep)
print("capture-first ok")
''' % (root, os.path.join(root, "tests"))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "capture-first ok" in r.stdout, r.stdout[-2000:] + r.stderr[-3000:]
