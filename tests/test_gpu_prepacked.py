"""Pre-packed weights on the GPU, through the C ABI: the packing kernels bit-exact against the oracle's restatement
of the byte map, and bfaintb_gemm_prepacked (both kernels behind it) against the oracle GEMM on the same seeded
inputs, to the bar of the row-major path (2 bf16 ULP of the fp32-accumulated reference)."""
import numpy as np
import pytest

import oracle
from helpers import Problem, Workspace, assert_close_gated, assert_close_ulp, from_dev_u16, run_gemm, to_dev

_ws = Workspace()

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def af():
    import torch
    import awesome_fusion_amd as af_
    assert torch.cuda.is_available()
    af_.lib()
    return af_


def packed_on_device(af, p):
    import torch
    pk = torch.zeros(af.prepack_bytes(p.n, p.k, p.bits), dtype=torch.uint8, device="cuda")
    af.prepack(pk, to_dev(p.b_bytes), p.n, p.k, weight_bits=p.bits)
    return pk


def run_prepacked(af, p, which=0, pk=None, ldc=None, activation=0):
    import torch
    pk = packed_on_device(af, p) if pk is None else pk
    ldc_ = (p.n // 2 if activation else p.n) if ldc is None else ldc
    c = torch.full((p.m, ldc_), 0x7FC0, dtype=torch.int16, device="cuda")
    bias = None if p.bias_bf is None else to_dev(p.bias_bf)
    ws = _ws.get(af.prepacked_workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size, which))
    res = None if p.residual_bf is None else to_dev(p.residual_bf)
    af.gemm_prepacked(c, to_dev(p.a_bf), pk, to_dev(p.s_bf), p.m, p.n, p.k, ldc=ldc, weight_bits=p.bits, group_size=p.group_size,
                      bias=bias, workspace=ws, which=which, residual=res, activation=activation)
    torch.cuda.synchronize()
    return from_dev_u16(c)


@pytest.mark.parametrize("bits,k,n", [(8, 64, 16), (8, 448, 272), (4, 128, 16), (4, 640, 304), (8, 4096, 4096)])
def test_pack_kernels_bit_exact_and_inverse(af, bits, k, n):
    import torch
    p = Problem(1, n, k, bits, 0, seed=k + n)
    pk = packed_on_device(af, p)
    torch.cuda.synchronize()
    assert np.array_equal(pk.cpu().numpy(), oracle.pack_mfma16(p.b_bytes, k, n, bits))
    back = torch.zeros_like(to_dev(p.b_bytes))
    af.unpack(back, pk, n, k, weight_bits=bits)
    torch.cuda.synchronize()
    assert np.array_equal(back.cpu().numpy(), p.b_bytes)


@pytest.mark.parametrize("bits,k,n,ldb", [(8, 64, 16, None), (8, 448, 272, 512), (4, 128, 16, None), (4, 640, 304, 768), (8, 4096, 4096, None)])
def test_pack_from_column_major_is_the_same_buffer(af, bits, k, n, ldb):
    """bfaintb_prepack_colmajor on [n, ldb] codes (k contiguous) gives byte for byte what bfaintb_prepack gives on the
    row-major form of the same weights (= the oracle's packed order); a GEMM over it meets the oracle."""
    import torch
    p = Problem(64, n, k, bits, 0, seed=k + n + 1)
    cm = oracle.colmajor_codes(p.q, bits)                     # [n, k * bits / 8]
    if ldb is not None:                                       # padded columns: the padding must not be read as codes
        wide = np.full((n, ldb * bits // 8), 0xAB, np.uint8)
        wide[:, :cm.shape[1]] = cm
        cm = wide
    pk = torch.zeros(af.prepack_bytes(n, k, bits), dtype=torch.uint8, device="cuda")
    af.prepack_colmajor(pk, to_dev(cm), n, k, ldb=ldb, weight_bits=bits)
    torch.cuda.synchronize()
    assert np.array_equal(pk.cpu().numpy(), oracle.pack_mfma16(p.b_bytes, k, n, bits))
    if k <= 640:
        assert_close_ulp(p, run_prepacked(af, p, pk=pk), f"GEMM over column-major-packed weights {n}x{k} b{bits}")


def test_pack_honours_the_row_stride(af):
    import torch
    k, n, ldb = 128, 48, 64
    p = Problem(1, n, k, 8, 0, seed=3)
    wide = np.full((k, ldb), 0xEE, np.uint8)
    wide[:, :n] = p.b_bytes
    pk = torch.zeros(af.prepack_bytes(n, k, 8), dtype=torch.uint8, device="cuda")
    af.prepack(pk, to_dev(wide), n, k, ldb=ldb, weight_bits=8)
    back = torch.full((k, ldb), 0x11, dtype=torch.uint8, device="cuda")
    af.unpack(back, pk, n, k, ldb=ldb, weight_bits=8)
    torch.cuda.synchronize()
    assert np.array_equal(pk.cpu().numpy(), oracle.pack_mfma16(p.b_bytes, k, n, 8))
    got = back.cpu().numpy()
    assert np.array_equal(got[:, :n], p.b_bytes) and np.all(got[:, n:] == 0x11)


@pytest.mark.parametrize("m,n,k,bits,group", [
    (1, 16, 64, 8, 0), (1, 256, 512, 8, 0), (3, 48, 192, 8, 64), (16, 64, 1024, 4, 0), (17, 80, 640, 4, 32),
    (33, 96, 1152, 4, 128), (70, 64, 1600, 8, 32), (1, 32, 8256, 8, 0), (40, 128, 4096, 8, 128), (5, 1024, 2048, 4, 128),
    # every launch form: one batch per wave (k = 4096 / 2048 for 8-bit with 1 / 2 row blocks, 4096 for 4-bit), pipelined
    # (long k, per-channel scales), with one and two row blocks
    (20, 48, 2048, 8, 0), (3, 32, 4096, 4, 128), (2, 32, 8192, 4, 0), (40, 32, 8256, 8, 0), (24, 32, 8192, 4, 0), (9, 64, 4096, 8, 0),
    # 8-bit codes, narrow with long columns: the split family instead of the slab kernel, also for a few rows
    (1, 1024, 12288, 8, 0), (4, 272, 12288, 8, 64), (8, 512, 16384, 8, 0)])
def test_decode_kernel_matches_oracle(af, m, n, k, bits, group):
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    assert_close_ulp(p, run_prepacked(af, p, af.DECODE), f"packed decode {m}x{n}x{k} b{bits} g{group}")
    p.with_bias()
    assert_close_ulp(p, run_prepacked(af, p, af.DECODE), f"packed decode + bias {m}x{n}x{k} b{bits} g{group}")


@pytest.mark.parametrize("m,n,k,bits,group", [
    (24, 1024, 4096, 8, 0),      # 8-bit, 17..32 rows, small matrix: two 16-row blocks that split k to fill one round
    (32, 528, 8192, 8, 64),
    (48, 768, 5120, 8, 0),       # so few columns that only 16-row blocks are used beyond 32 rows too
    (128, 256, 7168, 8, 128),
    (12, 528, 2048, 4, 64),      # 4-bit, 8..16 rows: 256 columns x 8 waves (row-major), ragged last column block
    (16, 4096, 4096, 4, 128),
    (24, 1040, 4096, 4, 0),      # 4-bit, 17..32 rows, narrow: two 8-wave blocks of 16 rows
    (1, 1024, 8192, 4, 128),     # narrow with long columns: the split factor stops at 16
    (8, 11008, 4096, 4, 128),    # 8-wave workgroups: the split stays within one round of workgroups
    (4, 1024, 12288, 8, 0),      # packed 8-bit, narrow and long: the split family instead of the slab kernel
    (2, 9216, 4096, 8, 0),       # 8-bit, 256 columns x 4 waves on a large matrix: the split that fills one round (7 x 36 workgroups)
    (16, 16640, 2048, 8, 0),     # 8 rows and more, over 64 blocks of 256 columns: those blocks (row-major) instead of 128-column ones
    (24, 16640, 2048, 8, 64),    # the same with two 16-row accumulators per wave
    (1, 22016, 4096, 4, 128),    # 4-bit, 4 waves, 86 blocks of 256 columns: 5 splits, not the 6 that land 4 workgroups past two rounds
    (4, 45056, 2048, 4, 128),    # ... 176 blocks: 4 splits, 2.75 rounds
    (8, 33024, 4224, 8, 0),      # 129 blocks of 256 columns, half a round: three splits once k is beyond 4096
    (16, 33024, 4224, 4, 128),   # the same for 4-bit codes with 8 waves
    (1, 131328, 512, 8, 0),      # 513 blocks of 256 columns, one past two rounds: k is split (two ways at this k)
    (24, 33024, 4096, 4, 128),   # one 32-row block of 4-bit codes over 129 blocks of 256 columns: three splits also at this k
    (40, 16512, 8192, 8, 0),     # one row of 129 small tiles and a long k: k split three ways, 387 workgroups in two rounds
    (40, 17408, 8192, 4, 128),   # the same with 4-bit codes and scale groups, 136 tiles
])
def test_plan_corners_both_weight_orders(af, m, n, k, bits, group):
    """Shapes on either side of the launch-plan rules for small, narrow and long matrices, kernel left to the library."""
    p = Problem(m, n, k, bits, group, seed=m * 3 + n + k)
    assert_close_ulp(p, run_gemm(p), f"row-major {m}x{n}x{k} b{bits} g{group}")
    assert_close_ulp(p, run_prepacked(af, p), f"packed {m}x{n}x{k} b{bits} g{group}")


@pytest.mark.parametrize("m,n,k,bits,group", [(1, 640, 1024, 4, 128), (3, 1040, 512, 8, 64), (2, 496, 1024, 4, 256), (1, 1024, 2048, 8, 128)])
def test_slab_kernel_hands_neighbouring_slabs_to_one_xcd_with_grouped_scales(af, m, n, k, bits, group):
    """With grouped scales the slab kernel gives the four slabs that share a 128-byte line of scales to workgroups 8 apart
    in dispatch order, within whole runs of 32 slabs; the slabs past the last whole run keep their place (40 slabs: one run
    and 8; 65: two and one; 31: none; 64: two whole runs).  Every column must still come out of its own slab."""
    assert af.plan(m, n, k, bits, group, packed=True).kernel == af.KERNEL_DECODE_SLAB
    p = Problem(m, n, k, bits, group, seed=n + k + bits)
    assert_close_ulp(p, run_prepacked(af, p), f"slab kernel {m}x{n}x{k} b{bits} g{group}")


@pytest.mark.parametrize("m,n,k,bits,group", [
    (49, 128, 512, 8, 0), (64, 4096, 1024, 8, 0), (100, 272, 448, 8, 64), (130, 48, 1024, 8, 32), (200, 1040, 256, 8, 0), (300, 144, 2048, 8, 128),
    (64, 256, 512, 4, 0), (97, 528, 1024, 4, 128), (150, 80, 640, 4, 32), (260, 1296, 384, 4, 128),
    # shapes whose plan splits along k (few column groups, long k): partial sums meet in the workspace
    (64, 256, 4096, 4, 128), (80, 128, 8192, 8, 0), (100, 512, 4096, 4, 0),
    # 8-bit codes whose waves walk several steps from a start of their own (one scale per column, and scale groups that
    # begin before, at and after that start: 32, 128, 192 and 2048 rows), 4-bit codes walking whole chunks with one and two row blocks
    (20, 1024, 8192, 8, 0), (33, 1024, 8192, 8, 128), (16, 2048, 6144, 8, 192), (70, 512, 8192, 8, 32), (24, 1024, 8192, 8, 2048),
    (16, 2048, 8192, 4, 128), (32, 1024, 8192, 4, 256), (40, 2048, 4096, 4, 64),
    # ... and three and four steps per wave (the walk wraps round inside a scale group of 384 rows, and between groups of 32)
    (20, 4096, 12288, 8, 384), (20, 11008, 4096, 8, 32), (16, 4096, 11008, 8, 0)])
def test_row_blocked_family_over_packed_weights(af, m, n, k, bits, group):
    """Beyond 48 rows of A the forced DECODE variant is the row-blocked decode family reading packed slabs (8 column
    blocks per workgroup for 8-bit codes, 16 for 4-bit; partial last groups re-read the last block)."""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    assert_close_ulp(p, run_prepacked(af, p, af.DECODE), f"packed family {m}x{n}x{k} b{bits} g{group}")
    p.with_bias()
    assert_close_ulp(p, run_prepacked(af, p, af.DECODE), f"packed family + bias {m}x{n}x{k} b{bits} g{group}")


@pytest.mark.parametrize("m,n,k,bits,group", [
    (256, 256, 64, 8, 0), (300, 272, 192, 8, 0), (64, 128, 256, 8, 0), (512, 512, 256, 4, 128), (1000, 1008, 384, 4, 0),
    (513, 784, 448, 8, 64), (130, 528, 512, 8, 32), (260, 304, 512, 4, 32), (4160, 256, 256, 8, 0), (2304, 512, 512, 4, 128)])
@pytest.mark.parametrize("tile", [256, 128])
def test_tiled_kernel_matches_oracle(af, m, n, k, bits, group, tile):
    """Both tile sizes of the tiled variant, each forced (left to itself the library runs 128x128 tiles on all of these
    shapes: none has more than 256 of them)."""
    which = af.PREFILL_256 if tile == 256 else af.PREFILL_128
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    assert_close_ulp(p, run_prepacked(af, p, which), f"packed prefill{tile} {m}x{n}x{k} b{bits} g{group}")
    p.with_bias()
    assert_close_ulp(p, run_prepacked(af, p, which), f"packed prefill{tile} + bias {m}x{n}x{k} b{bits} g{group}")
    if tile == 128:
        assert np.array_equal(run_prepacked(af, p, which), run_prepacked(af, p, af.PREFILL)), "PREFILL picks 128x128 tiles here"


@pytest.mark.parametrize("m,n,k,bits,group", [(4160, 256, 256, 8, 0), (1000, 1008, 384, 4, 0), (300, 528, 512, 8, 64), (130, 4112, 256, 4, 128)])
def test_tile_sizes_and_weight_orders_agree_bit_for_bit(af, m, n, k, bits, group):
    """The tiled kernels add an output's products in the same order whatever the tile size and whichever order the
    weights are stored in: four launches, one result, bias included."""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    want = run_gemm(p, which=af.PREFILL_256)
    assert np.array_equal(run_prepacked(af, p, af.PREFILL_128_LDS), want) and np.array_equal(run_prepacked(af, p, af.PREFILL_256), want)
    p.with_bias()
    assert np.array_equal(run_prepacked(af, p, af.PREFILL_128_LDS), run_prepacked(af, p, af.PREFILL_256))


@pytest.mark.parametrize("m,n,k,bits,group", [(130, 272, 64, 8, 0), (700, 1008, 1024, 8, 0), (300, 528, 512, 8, 64), (1000, 1008, 384, 4, 0),
                                              (130, 4112, 256, 4, 128), (1024, 4096, 1088, 8, 0), (257, 272, 128, 4, 0), (100, 528, 4096, 4, 128),
                                              (256, 1040, 2048, 8, 64), (64, 4096, 4096, 8, 0), (384, 2048, 8192, 4, 128), (900, 1408, 2432, 4, 128)])
def test_small_tiles_keep_packed_weights_in_registers_too(af, m, n, k, bits, group):
    """128x128 tiles over packed weights run the kernel that converts the weights into operand registers: the codes of a
    step come into LDS as the packed order stores them and a lane takes its two columns' operands with two reads.  Same
    plan as for row-major weights, the split along k included (the long-k shapes here split), so the two weight orders
    must agree bit for bit; and against the oracle.  Partial tiles in m and n, one to 128 K-steps, 4-bit chunks that
    straddle two steps and two splits."""
    if (m, k) == (900, 2432):  # two splits of 19 steps: the second starts in the middle of a 4-bit chunk
        assert af.prepacked_workspace_bytes(m, n, k, bits, group, af.PREFILL_128) == af.workspace_bytes(m, n, k, bits, group, af.PREFILL_128, 2)
    p = Problem(m, n, k, bits, group, seed=m + 2 * n + k)
    c = run_prepacked(af, p, af.PREFILL_128)
    assert_close_ulp(p, c, f"packed, 128x128 tiles, weights in registers: {m}x{n}x{k} bits={bits} g={group}")
    assert np.array_equal(c, run_gemm(p, which=af.PREFILL_128))
    p.with_bias()
    assert_close_ulp(p, run_prepacked(af, p, af.PREFILL_128), f"... + bias: {m}x{n}x{k} bits={bits} g={group}")


@pytest.mark.parametrize("m,n,k,bits,group", [(100, 1040, 320, 8, 0), (128, 272, 448, 8, 64), (60, 528, 512, 4, 128), (100, 1040, 384, 4, 0),
                                              (17, 48, 128, 4, 64), (2064, 4096, 256, 8, 0), (520, 16512, 256, 4, 128), (2100, 4112, 192, 8, 32)])
def test_large_tiles_keep_packed_weights_in_registers_too(af, m, n, k, bits, group):
    """Whole 256x256 tiles over packed weights run the kernel that converts the weights into operand registers (a lane
    takes its operands from the packed order as they are stored; its four columns are 16 apart): against the oracle, and
    bit for bit against the form with both operands in LDS and against the row-major path.  Shapes whose tiles run whole:
    up to 128 rows of A, or more than 128 tiles in the last round; partial tiles in m and n, odd numbers of K-steps."""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    c = run_prepacked(af, p, af.PREFILL_256)
    assert_close_ulp(p, c, f"packed, 256x256 tiles, weights in registers: {m}x{n}x{k} bits={bits} g={group}")
    assert np.array_equal(c, run_prepacked(af, p, af.PREFILL_256_LDS))
    assert np.array_equal(c, run_gemm(p, which=af.PREFILL_256))
    p.with_bias()
    c = run_prepacked(af, p, af.PREFILL_256)
    assert_close_ulp(p, c, f"... + bias: {m}x{n}x{k} bits={bits} g={group}")
    assert np.array_equal(c, run_prepacked(af, p, af.PREFILL_256_LDS))


@pytest.mark.parametrize("m,n,k,bits,group", [(256, 128, 64, 8, 0), (300, 272, 448, 8, 0), (700, 1008, 1024, 8, 0), (1000, 1008, 384, 4, 0), (520, 528, 512, 8, 64),
                                              (130, 4112, 256, 4, 128), (257, 272, 128, 4, 0), (2048, 512, 1088 + 64, 8, 0), (17, 48, 128, 4, 64)])
def test_tall_tiles_keep_packed_weights_in_registers_too(af, m, n, k, bits, group):
    """Tiles of 256 rows x 128 columns over packed weights (a lane's four neighbouring columns are four neighbouring pieces of
    a packed chunk): against the oracle and bit for bit against the row-major path — partial tiles in m and n, one to
    eighteen steps, 4-bit chunks of two steps, grouped scales."""
    p = Problem(m, n, k, bits, group, seed=m + n + k)
    c = run_prepacked(af, p, af.PREFILL_256X128)
    assert_close_ulp(p, c, f"packed, 256x128 tiles: {m}x{n}x{k} bits={bits} g={group}")
    assert np.array_equal(c, run_gemm(p, which=af.PREFILL_256X128))
    p.with_bias()
    assert_close_ulp(p, run_prepacked(af, p, af.PREFILL_256X128), f"... + bias: {m}x{n}x{k} bits={bits} g={group}")


def test_tall_tiles_over_packed_weights_are_what_auto_runs_and_take_the_epilogues(af):
    m, n, k = 2100, 2048, 320
    assert af.prepacked_variant(m, n, k) == af.PREFILL and (af.prefill_tile(m, n), af.prefill_tile_cols(m, n)) == (256, 128)
    p = Problem(m, n, k, 8, 0, seed=81)
    assert np.array_equal(run_prepacked(af, p), run_prepacked(af, p, af.PREFILL_256X128))
    p.with_bias().with_residual()
    assert_close_ulp(p, run_prepacked(af, p), "packed, tall tiles, bias + residual")
    g = Problem(m, n, 384, 4, 128, seed=82, scale_lo=0.002, scale_hi=0.2).with_bias()
    assert_close_gated(g, run_prepacked(af, g, activation=af.ACT_SILU_GATE), "packed, tall tiles, gated")


@pytest.mark.parametrize("m,n,k,bits,group", [(2064, 4112, 192, 8, 0), (2100, 4128, 128, 4, 128)])
def test_large_tiles_over_packed_weights_take_the_epilogues(af, m, n, k, bits, group):
    """Shapes the library runs on whole 256x256 tiles by itself (the fused entry point takes no forced variant): 9 x 17 of
    them, the last ones partial in m and n."""
    assert af.prepacked_variant(m, n, k, bits, group) == af.PREFILL and af.prefill_tile(m, n) == 256
    p = Problem(m, n, k, bits, group, seed=m + k).with_bias().with_residual()
    assert_close_ulp(p, run_prepacked(af, p), f"packed, 256x256 tiles, bias + residual {m}x{n}x{k}")
    g = Problem(m, n, k, bits, group, seed=m + k + 1, scale_lo=0.002, scale_hi=0.02 if bits == 8 else 0.2).with_bias()
    g.residual_bf = oracle.f32_to_bf16_rne(np.random.default_rng(5).uniform(-2, 2, size=(m, n // 2)).astype(np.float32))
    assert_close_gated(g, run_prepacked(af, g, activation=af.ACT_SILU_GATE), f"packed, 256x256 tiles, gated {m}x{n}x{k}")


@pytest.mark.parametrize("bits,group", [(8, 0), (4, 128)])
@pytest.mark.parametrize("which,m", [(1, 16), (1, 32), (1, 64), (3, 64), (4, 64)])
def test_kernels_dequantise_bit_exact(af, bits, group, which, m):
    """One-hot activations make C[i, :] = W[k_i, :] with nothing to round: the in-register conversion of both
    kernels is observed exactly, against the oracle's dequantised weights."""
    k, n = 256, 512
    p = Problem(m, n, k, bits, group, seed=7)
    pk = packed_on_device(af, p)
    for base in range(0, k, m):
        a = np.zeros((m, k), np.float32)
        rows = (base + np.arange(m)) % k
        a[np.arange(m), rows] = 1.0
        p.a_bf = oracle.f32_to_bf16_rne(a)
        assert np.array_equal(run_prepacked(af, p, which, pk=pk), p.w_bf[rows]), f"rows {base}.. differ"


@pytest.mark.parametrize("m,n,k,bits,group,which", [
    (1, 256, 960, 8, 96, "AUTO"), (20, 528, 1920, 4, 160, "AUTO"), (80, 1040, 2240, 8, 224, "AUTO"), (64, 256, 1920, 4, 160, "AUTO"),
    (300, 272, 960, 8, 96, "PREFILL_128"), (300, 528, 1920, 4, 160, "PREFILL_256"), (520, 272, 2240, 8, 224, "PREFILL_256X128"),
    (300, 528, 1920, 4, 160, "PREFILL_128_LDS")])
def test_scale_groups_that_are_no_power_of_two(af, m, n, k, bits, group, which):
    p = Problem(m, n, k, bits, group, seed=m + n + k + group)
    assert_close_ulp(p, run_prepacked(af, p, getattr(af, which)), f"packed, {which}: {m}x{n}x{k} bits={bits} g={group}")


@pytest.mark.parametrize("m", [1, 16])
def test_headline_shapes(af, m):
    p = Problem(m, 4096, 4096, seed=20 + m)
    assert af.prepacked_variant(m, 4096, 4096) == af.DECODE
    assert_close_ulp(p, run_prepacked(af, p), f"packed 4096x4096 m={m}", threads=16)
    p = Problem(m, 28672, 8192, 4, 128, seed=50 + m, scale_lo=0.001, scale_hi=0.02)
    assert_close_ulp(p, run_prepacked(af, p), f"packed int4 g128 m={m}", threads=16)


def test_tiled_full_size(af):
    p = Problem(4096, 4096, 4096, seed=4)
    assert af.prepacked_variant(4096, 4096, 4096) == af.PREFILL
    assert_close_ulp(p, run_prepacked(af, p), "packed prefill 4096^3", threads=16)


def test_matches_the_row_major_path_in_the_exact_regime(af):
    """Small-integer data (the reference's own test regime) has exact sums: packed and row-major agree bit for bit."""
    from helpers import run_gemm
    for m in (1, 40, 300):
        p = Problem(m, 272, 512, 8, 0, seed=m, regime="small_int")
        assert np.array_equal(run_prepacked(af, p), run_gemm(p))


def test_workspace_is_required_where_the_plan_splits_and_left_ready(af):
    import torch
    m, n, k, bits, g = 64, 256, 4096, 4, 128
    need = af.prepacked_workspace_bytes(m, n, k, bits, g)
    assert need > 0 and af.prepacked_workspace_bytes(1, n, k, bits, g) == 0 and af.prepacked_workspace_bytes(4096, 4096, 4096) == 0
    p = Problem(m, n, k, bits, g, seed=11)
    pk = packed_on_device(af, p)
    c = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    args = (c, to_dev(p.a_bf), pk, to_dev(p.s_bf), m, n, k)
    assert af.gemm_prepacked(*args, weight_bits=bits, group_size=g, check=False) == -6
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    af.workspace_init(ws)
    for _ in range(2):  # the second call finds the workspace as the first left it
        af.gemm_prepacked(*args, weight_bits=bits, group_size=g, workspace=ws)
        torch.cuda.synchronize()
        assert_close_ulp(p, from_dev_u16(c), "packed split-K")
    assert bool((ws[256:] == 0xFF).all()) and af.workspace_status(ws) == 0  # header, then empty words


@pytest.mark.parametrize("m,n,k,bits,group", [
    (1, 4096, 4096, 8, 0), (20, 528, 1024, 4, 128),   # slab kernel
    (80, 1040, 2048, 8, 64), (64, 256, 4096, 4, 128),  # row-blocked family, without and with a split along k
    (4200, 272, 256, 8, 0), (4200, 528, 256, 4, 128),  # tiled kernel over packed weights, 128x128 tiles
    (4200, 1040, 128, 8, 0), (4200, 1296, 256, 4, 128),  # more than 256 of those: 256x256 tiles
])
def test_fused_residual(af, m, n, k, bits, group):
    p = Problem(m, n, k, bits, group, seed=m + k).with_residual()
    assert_close_ulp(p, run_prepacked(af, p), f"packed residual {m}x{n}x{k}")
    p.with_bias()
    assert_close_ulp(p, run_prepacked(af, p), f"packed bias + residual {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k,bits,group", [
    (1, 4096, 4096, 8, 0), (20, 544, 1024, 4, 128),    # slab kernel
    (80, 1056, 2048, 8, 64), (64, 256, 4096, 4, 128),   # row-blocked family, without and with a split along k
    (4200, 288, 256, 8, 0), (4200, 544, 256, 4, 128),   # tiled kernel over packed weights, 128x128 tiles
    (4200, 1056, 128, 8, 0), (4200, 1312, 256, 4, 128),  # more than 256 of those: 256x256 tiles
])
def test_silu_gate_epilogue(af, m, n, k, bits, group):
    p = Problem(m, n, k, bits, group, seed=m + k, scale_lo=0.002, scale_hi=0.02 if bits == 8 else 0.2)
    c = run_prepacked(af, p, activation=af.ACT_SILU_GATE)
    assert c.shape == (m, n // 2)
    assert_close_gated(p, c, f"packed gated {m}x{n}x{k}")
    p.with_bias()
    p.residual_bf = oracle.f32_to_bf16_rne(np.random.default_rng(3).uniform(-2, 2, size=(m, n // 2)).astype(np.float32))
    assert_close_gated(p, run_prepacked(af, p, activation=af.ACT_SILU_GATE), f"packed gated + bias + residual {m}x{n}x{k}")


def test_output_stride_and_padding(af):
    p = Problem(5, 48, 128, 8, 0, seed=9)
    c = run_prepacked(af, p, ldc=64)
    assert_close_ulp(p, np.ascontiguousarray(c[:, :48]), "packed ldc")
    assert np.all(c[:, 48:] == 0x7FC0)


def test_hip_graph_replays_match_eager(af):
    """Packing and the packed GEMMs hold no memset and no scratch state: captured once, every replay reproduces the
    eager bits, with other work and synchronisations in between."""
    import torch
    # (the last one: 128x128 tiles with k split between workgroups, the hand-over through the workspace inside the graph)
    shapes = [(1, 4096, 4096, 8, 0), (4, 1040, 2048, 4, 128), (40, 64, 8256, 8, 0), (64, 256, 4096, 4, 128), (600, 512, 512, 8, 0), (384, 2048, 8192, 4, 128)]
    probs = [Problem(m, n, k, bits, g, seed=190 + i) for i, (m, n, k, bits, g) in enumerate(shapes)]
    eager = [run_prepacked(af, p) for p in probs]
    bufs = [dict(a=to_dev(p.a_bf), b=to_dev(p.b_bytes), s=to_dev(p.s_bf), pk=torch.zeros(af.prepack_bytes(p.n, p.k, p.bits), dtype=torch.uint8, device="cuda"),
                 c=torch.zeros((p.m, p.n), dtype=torch.int16, device="cuda"), w=None) for p in probs]
    for p, d in zip(probs, bufs):
        need = af.prepacked_workspace_bytes(p.m, p.n, p.k, p.bits, p.group_size)
        if need:
            d["w"] = torch.empty(need, dtype=torch.uint8, device="cuda")
            af.workspace_init(d["w"])

    def run_all():
        for p, d in zip(probs, bufs):
            af.prepack(d["pk"], d["b"], p.n, p.k, weight_bits=p.bits)
            af.gemm_prepacked(d["c"], d["a"], d["pk"], d["s"], p.m, p.n, p.k, weight_bits=p.bits, group_size=p.group_size, workspace=d["w"])

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run_all()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run_all()
    for replay in range(3):
        for d in bufs:
            d["c"].fill_(0x7FC0)
            d["pk"].zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for i, d in enumerate(bufs):
            assert np.array_equal(from_dev_u16(d["c"]), eager[i]), f"replay {replay}, problem {i}"
        run_prepacked(af, probs[0])  # unrelated eager work between replays
