"""The C-ABI library on a machine without a GPU: it loads, exports what the header declares, and
rejects bad arguments before touching the device (so none of this launches anything)."""
import ctypes as C
import os
import re

import pytest

import awesome_fusion_amd as af

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = 0x10000  # a fake, non-null, 16-byte aligned "device pointer": validation never dereferences


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "bfaintb_gemm.h")).read()
    return re.findall(r"BFAINTB_API\s+[\w\s\*]+?\b(bfaintb_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 17 and "bfaintb_gemm_prepacked" in names and "bfaintb_gemm" in names and "bfaintb_dequant" in names
    lib = C.CDLL(af.library_path())
    for name in names:
        assert hasattr(lib, name), name
    assert af.lib().bfaintb_version() == 200
    assert "bfaintb_gemm_bias" in names


def test_public_header_is_plain_c(tmp_path):
    """include/bfaintb_gemm.h is the boundary a C caller binds to: it must compile as C99 on its own, and as C++."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "use_header.c"
    src.write_text('#include "bfaintb_gemm.h"\n'
                   'int main(void) { bfaintb_epilogue e = {0, 0, 0, BFAINTB_ACT_NONE}; bfaintb_packed_header h; (void)e; (void)h;\n'
                   '  return bfaintb_gemm_variant(1, 16, 64, 8, 0) == BFAINTB_VARIANT_DECODE ? 0 : 1; }\n')
    inc = os.path.join(root, "include")
    for cmd in (["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-I", inc, str(src)],
                ["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc, str(src)]):
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr


def test_variant_choice_and_split():
    assert af.variant(1, 4096, 4096) == af.DECODE
    assert af.variant(32, 4096, 4096) == af.DECODE
    assert af.variant(33, 4096, 4096) == af.DECODE      # row blocks of the decode family: 256x256 tiles would idle most CUs
    assert af.variant(128, 4096, 4096) == af.DECODE     # 15.7 us against 22 for 32 small tiles with k split four ways
    assert af.variant(2048, 4096, 4096) == af.PREFILL
    assert af.variant(512, 28672, 8192, 4, 128) == af.PREFILL
    assert af.variant(4096, 4096, 4096) == af.PREFILL
    assert af.variant(1, 28672, 8192, 4, 128) == af.DECODE
    # the tiled variant where the row-blocked family's last round would be mostly empty (320 workgroups on 256 CUs), and
    # before that where its small tiles, k split two ways, fill the CUs
    # (64 x 8192 x 8192: the small tiles by 6 % — 27.2 against 29.1 us — since the family's hand-over is priced at 0.9 of its term)
    assert af.variant(64, 4096, 4096) == af.DECODE and af.variant(64, 8192, 8192) == af.PREFILL
    assert af.variant(384, 4096, 4096) == af.PREFILL == af.variant(640, 4096, 4096)
    assert af.split_k(512, 4096, 4096) == 2 and af.split_k(640, 4096, 4096) == 1
    # 128x128 tiles up to one per CU, 256x256 beyond; forced forms are accepted as variants
    assert af.prefill_tile(1024, 4096) == 128 and af.prefill_tile(1025, 4096) == 256
    # (the gap: 258 tall tiles just miss one round and the large ones would use half the machine: two rounds of small tiles)
    assert af.prefill_tile(640, 11008) == 128 and af.plan(640, 11008, 4096).workgroups == 430 and af.plan(640, 11008, 4096).splits == 1
    assert af.prefill_tile(704, 11008) == 256 and af.prefill_tile(512, 11008) == 256 and af.prefill_tile_cols(512, 11008) == 128
    # (... while the large tiles would fill at most 60 % of the CUs: 141 of them at 640 x 12032, 500 small ones at 600 x 12800)
    assert af.prefill_tile(640, 12032) == 128 and af.plan(600, 12800, 4096).workgroups == 500
    # 4-bit codes beyond 256 rows: ten row blocks over few column blocks, unsplit, lose to the tiles (39.9 against 29.0 us)
    assert af.variant(320, 2816, 6144, 4, 128) == af.PREFILL and af.variant(512, 1280, 5120, 4, 128) == af.PREFILL
    assert af.variant(320, 1024, 14336, 4, 128) == af.DECODE     # (with k split the family stays ahead: 30.4 against 38.3)
    assert af.prefill_tile(128, 28672) == 128 and af.prefill_tile(4096, 4096) == 256 and af.prefill_tile(1, 16) == 128
    # the small tiles over row-major weights split k while tiles x splits fit one workgroup per CU: same workspace layout as
    # the decode family's; the large tiles, the both-operands-in-LDS form and an unsplit launch need none
    assert af.workspace_bytes(64, 4096, 4096, which=af.PREFILL_128, force_split_k=3) == 256 + 2 * 64 * 4096 * 4
    assert af.workspace_bytes(64, 4096, 4096, which=af.PREFILL_128, force_split_k=1) == 0
    assert af.workspace_bytes(64, 4096, 4096, which=af.PREFILL_128, force_split_k=1000) == 256 + 15 * 64 * 4096 * 4   # at most 16
    assert af.workspace_bytes(64, 4096, 64, which=af.PREFILL_128, force_split_k=4) == 0                               # one K-step: nothing to split
    auto = af.workspace_bytes(64, 4096, 4096, which=af.PREFILL_128)
    assert auto > 0 and (auto - 256) % (64 * 4096 * 4) == 0 and ((auto - 256) // (64 * 4096 * 4) + 1) * 32 <= 256
    assert af.workspace_bytes(1024, 4096, 4096, which=af.PREFILL_128) == 0   # a tile on every CU already
    assert af.workspace_bytes(64, 4096, 4096, which=af.PREFILL_128_LDS, force_split_k=4) == 0 == af.workspace_bytes(64, 4096, 4096, which=af.PREFILL_256)
    # AUTO: tiles with k split where the plan says so, reported by split_k and workspace_bytes alike
    assert af.variant(384, 2048, 8192) == af.PREFILL and af.split_k(384, 2048, 8192) > 1
    assert af.workspace_bytes(384, 2048, 8192) == 256 + (af.split_k(384, 2048, 8192) - 1) * 384 * 2048 * 4
    assert af.workspace_bytes(384, 2048, 8192) <= af.lib().bfaintb_gemm_static_scratch_bytes() == 16 << 20
    assert af.kernel_name(64, which=af.PREFILL_128) == "bfaintb_prefill128_wreg_kernel"
    assert af.kernel_name(64, which=af.PREFILL_128_LDS) == "bfaintb_prefill128_kernel"
    assert af.kernel_name(64, which=af.PREFILL_256) == af.kernel_name(64, which=af.PREFILL) == "bfaintb_prefill_wreg_kernel"
    assert af.kernel_name(64, which=af.PREFILL_256_LDS) == "bfaintb_prefill_kernel"
    assert af.split_k(4096, 4096, 4096) == 1
    s = af.split_k(1, 4096, 4096)
    assert 1 < s <= 64 and 4096 % s == 0
    # none for the prefill variant or without split-K
    assert af.workspace_bytes(1, 4096, 4096) == 256 + (s - 1) * 1 * 4096 * 4   # the header, then one fp32 word per (split but the last, row, column)
    assert af.workspace_bytes(4096, 4096, 4096) == 0
    assert af.workspace_bytes(8, 4096, 4096, force_split_k=1) == 0
    assert af.kernel_name(1) == "bfaintb_decode_kernel" and af.kernel_name(4096) == "bfaintb_prefill_wreg_kernel"


def rc(**kw):
    d = dict(c=P, a=P, b=P, scale=P, m=64, n=128, k=256, weight_bits=8, group_size=0, workspace=None, stream=0, check=False)
    d.update(kw)
    return af.gemm(d.pop("c"), d.pop("a"), d.pop("b"), d.pop("scale"), d.pop("m"), d.pop("n"), d.pop("k"), **d)


def test_ragged_shapes_are_accepted_by_the_host_side_queries():
    # n % 8 == 0 and k % 8 == 0 for 8-bit codes (the reference kernel needs multiples of 64), n % 16 == 0 for 4-bit codes
    assert af.variant(1, 4104, 4072) == af.DECODE and af.variant(33, 1000, 1000) in (af.DECODE, af.PREFILL)
    assert af.variant(300, 1000, 1000) in (af.DECODE, af.PREFILL) and af.variant(16, 1008, 1000, 4, 0) == af.DECODE
    assert af.variant(1, 4100, 4072) == -2 and af.variant(1, 4104, 4071) == -2 and af.variant(1, 1000, 1000, 4, 0) == -2
    assert af.workspace_bytes(1, 4104, 4072) > 256          # split along k: the partial last step belongs to the last split
    # the packed order keeps whole chunks and column blocks
    assert af.prepack_bytes(4104, 4096) == 0 and af.prepack_bytes(4096, 4072) == 0 and af.prepacked_variant(1, 4104, 4096) == -2


def test_rejects_bad_arguments_without_launching():
    L = af.lib()
    assert rc(weight_bits=5) == -5
    assert rc(group_size=48) == -5            # not a multiple of 32
    assert rc(group_size=96) == -5            # does not divide k = 256
    assert rc(n=100) == -2                    # n % 8
    assert rc(n=104, weight_bits=4, ldb=112, ldc=104) == -2   # 4-bit codes: n % 16
    assert rc(k=100) == -2                    # k % 8 (the reference kernel needs k % 64: asm main loop)
    assert rc(k=0) == -2
    assert rc(lda=128) == -3                  # lda < k
    assert rc(ldb=64) == -3
    assert rc(ldc=64) == -3
    assert rc(ldb=1 << 27) == -3              # a lane's offset within 32 rows of B is kept in 32 bits
    assert rc(lda=260) == -3                  # rows of A would lose 16-byte alignment
    assert rc(a=None) == -1
    assert rc(c=0) == -1
    assert rc(b=P + 4) == -4
    assert rc(which=9) == -7
    assert rc(m=40000, which=af.DECODE) == -7  # beyond what the decode variant accepts when forced
    assert rc(m=8, k=1024, which=af.DECODE, force_split_k=2) == -6   # split-K needs a workspace
    assert rc(m=8, k=1024, which=af.DECODE, force_split_k=2, workspace=P, workspace_nbytes=64) == -6
    assert rc(m=0) == 0                       # nothing to do
    assert rc(bias=P + 2) == -4               # bias must be 16-byte aligned too
    assert rc(residual=P + 2) == -4           # and the residual
    assert rc(residual=P, ldr=64) == -3       # ldr < n
    assert rc(activation=7) == -5             # unknown activation
    assert rc(activation=af.ACT_SILU_GATE, ldc=56) == -3   # gated C has n/2 = 64 columns
    assert rc(activation=af.ACT_SILU_GATE, residual=P, ldr=56) == -3
    assert rc(residual=P, ldr=132) == -3      # rows of the residual would lose 16-byte alignment
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert len(af.error_string(code)) > 10
    with pytest.raises(af.BfaintbError) as e:
        rc(n=100, check=True)
    assert e.value.code == -2
    # the reference-arithmetic entry point: same validation, fp32 scales
    def ref_rc(**kw):
        d = dict(c=P, a=P, b=P, scale=P, m=64, n=128, k=256, stream=0, check=False)
        d.update(kw)
        return af.gemm_reference(d.pop("c"), d.pop("a"), d.pop("b"), d.pop("scale"), d.pop("m"), d.pop("n"), d.pop("k"), **d)
    assert ref_rc(n=100) == -2 and ref_rc(k=100) == -2 and ref_rc(ldb=64) == -3 and ref_rc(ldc=120) == -3
    assert ref_rc(scale=None) == -1 and ref_rc(scale=P + 4) == -4 and ref_rc(which=9) == -7 and ref_rc(m=0) == 0
    assert ref_rc(m=8, k=1024, which=af.DECODE, force_split_k=2) == -6
    # dequant entry point
    assert af.dequant(P, P, P, 128, 256, stream=0, weight_bits=3, check=False) == -5
    assert af.dequant(P, P, P, 100, 256, stream=0, check=False) == -2
    assert af.dequant(P, P, None, 128, 256, stream=0, check=False) == -1
    assert L.bfaintb_workspace_init(P, 66, None) == -6   # not a whole number of words
    assert L.bfaintb_workspace_init(None, 0, None) == 0
    # tuning and test hooks: values outside their ranges are refused, valid ones change no result (GPU tests)
    assert L.bfaintb_debug_control(af.DEBUG_FORCE_ROW_BLOCK, 3) == -5 and L.bfaintb_debug_control(99, 0) == -5
    assert L.bfaintb_debug_control(af.DEBUG_FORCE_ROW_BLOCK, 2) == 0 and L.bfaintb_debug_control(af.DEBUG_FORCE_ROW_BLOCK, 0) == 0


def test_plan_query_agrees_with_the_other_queries_and_follows_the_compute_units():
    """bfaintb_gemm_plan describes a launch without making it: it must say what variant / split_k / workspace_bytes say,
    and plans made for another number of compute units (the tuning hook; on a device, its own count) stay within it."""
    for (m, n, k, bits, g) in [(1, 4096, 4096, 8, 0), (16, 11008, 4096, 8, 0), (32, 28672, 8192, 4, 128), (256, 4096, 4096, 8, 0),
                               (384, 2048, 8192, 8, 0), (1024, 4096, 4096, 8, 0), (2048, 4096, 4096, 8, 0), (4096, 4096, 4096, 8, 0),
                               (2048, 28672, 8192, 4, 128)]:
        pl = af.plan(m, n, k, bits, g)
        v = af.variant(m, n, k, bits, g)
        assert (pl.variant == af.DECODE) == (v == af.DECODE), (m, n, k)
        assert pl.splits == af.split_k(m, n, k, bits, g) and pl.workspace_bytes == af.workspace_bytes(m, n, k, bits, g)
        assert pl.compute_units == 256 or pl.compute_units > 0
        if pl.variant != af.DECODE:
            assert pl.tile_rows == af.prefill_tile(m, n) and pl.tile_cols == af.prefill_tile_cols(m, n)
        pk = af.plan(m, n, k, bits, g, packed=True)
        assert pk.workspace_bytes == af.prepacked_workspace_bytes(m, n, k, bits, g)
    # the headline shapes on a 256-unit part (what this container, without a device, plans for)
    if af.plan(1, 4096, 4096).compute_units == 256:
        d = af.plan(1, 4096, 4096)
        assert (d.kernel, d.tile_cols, d.waves, d.splits, d.workgroups) == (af.KERNEL_DECODE_FAMILY, 128, 8, 8, 256)
        t = af.plan(4096, 4096, 4096)
        assert (t.kernel, t.tile_rows, t.tile_cols, t.workgroups, t.launches) == (af.KERNEL_TILES_256, 256, 256, 256, 1)
        c5 = af.plan(2048, 28672, 8192, 4, 128)
        assert (c5.kernel, c5.workgroups, c5.tail_workgroups, c5.launches) == (af.KERNEL_TILES_256, 768, 256, 2)
        assert af.plan(1, 4096, 4096, packed=True).kernel == af.KERNEL_DECODE_SLAB
        # many 256-column blocks of 4-bit codes, 4 waves: never a few workgroups past a round of one per unit
        for (n, k, wgs) in ((22016, 4096, 430), (26624, 4096, 416), (33280, 4096, 390), (45056, 4096, 704), (28672, 8192, 448)):
            w = af.plan(1, n, k, 4, 128)
            assert (w.tile_cols, w.waves, w.workgroups) == (256, 4, wgs), (n, k, w.as_dict())
            assert w.workgroups % 256 >= 128
        # 8-bit codes: 128-column blocks only where they fit one round (36864 columns would take 6.75 rounds of them) ...
        w = af.plan(1, 36864, 4096)
        assert (w.tile_cols, w.waves, w.splits, w.workgroups) == (256, 4, 1, 144)
        # ... and a half-filled round of 256-column blocks takes three splits once k is beyond 4096
        assert [af.plan(mm, 36864, 8192, bb, gg).workgroups for (mm, bb, gg) in ((1, 8, 0), (16, 8, 0), (8, 4, 128), (16, 4, 128))] == [432] * 4
        # more than two rounds of 256-column blocks, fewer than 8 rows: the split that wastes the least of its last round
        assert [af.plan(1, n, 4096).splits for n in (128256, 131328, 151936)] == [1, 4, 3] and af.plan(8, 151936, 4096).splits == 1
        # ... also for one 32-row block of 4-bit codes while k is short (the estimate alone would not split there)
        assert [af.plan(mm, 36864, 4096, 4, 128).workgroups for mm in (17, 32)] == [432, 432]
        # one row of small tiles on half to five eighths of a round, k of 8192 or more: three splits, while the sums stay within 14 MiB
        t = af.plan(48, 18432, 8192)
        assert (t.kernel, t.splits, t.workgroups) == (af.KERNEL_TILES_128, 3, 432) and t.workspace_bytes == 256 + 2 * 48 * 18432 * 4
        assert af.plan(48, 18432, 4096).splits == 1 and af.plan(128, 18432, 8192).splits == 1 and af.plan(48, 21760, 8192).splits == 1
        assert af.plan(96, 18432, 8192).workspace_bytes <= af.lib().bfaintb_gemm_static_scratch_bytes()
        # one row of tiles is always 128 x 128 tiles, whatever their number; more rows go back to large tiles
        assert (af.prefill_tile(96, 36864), af.prefill_tile(128, 128256), af.prefill_tile(129, 36864)) == (128, 128, 256)
        for packed in (False, True):
            t = af.plan(96, 36864, 8192, packed=packed)
            assert (t.tile_rows, t.tile_cols, t.workgroups) == (128, 128, 288), (packed, t.as_dict())
            t = af.plan(64, 128256, 4096, 4, 128, packed=packed)
            assert t.workgroups == 1002 and (t.tile_rows == 128) == (not packed), (packed, t.as_dict())
    try:
        for cus in (64, 304):
            af.debug_control(af.DEBUG_PLAN_COMPUTE_UNITS, cus)
            d = af.plan(1, 4096, 4096)
            assert d.compute_units == cus and d.workgroups <= cus, (cus, d.as_dict())       # 8-wave workgroups: one round
            assert d.workspace_bytes == af.workspace_bytes(1, 4096, 4096)
            for (m, n) in ((512, 2048), (1024, 4096), (2048, 4096)):
                t = af.plan(m, n, 4096, which=af.PREFILL)
                tiles = -(-m // t.tile_rows) * -(-n // t.tile_cols)
                assert t.tile_rows == 256 and t.tile_cols == 256 or tiles * t.splits <= cus, (cus, m, n, t.as_dict())
    finally:
        af.debug_control(af.DEBUG_PLAN_COMPUTE_UNITS, 0)
    assert af.plan(1, 4096, 4096).compute_units != 64


def test_split_k_test_hooks_are_refused_without_the_environment_switch():
    """The hooks that withhold partial sums or cap the reducer's wait change what every later split-K launch of the
    process does: a process that has not asked for them (BFAINTB_TEST_HOOKS=1) gets BFAINTB_ERR_UNSUPPORTED."""
    import subprocess
    import sys
    code = ("import os, sys; sys.path.insert(0, %r); os.environ.pop('BFAINTB_TEST_HOOKS', None); os.environ['BFAINTB_TEST_HOOKS'] = sys.argv[1];"
            "import awesome_fusion_amd as af; L = af.lib();"
            "print(L.bfaintb_debug_control(af.DEBUG_SPLIT_WAIT_LIMIT, 3), L.bfaintb_debug_control(af.DEBUG_WITHHOLD_PARTIALS, 1),"
            " L.bfaintb_debug_control(af.DEBUG_FORCE_ROW_BLOCK, 0))") % ROOT
    for value, want in (("0", "-5 -5 0"), ("1", "0 0 0")):
        r = subprocess.run([sys.executable, "-c", code, value], capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert r.stdout.split("\n")[-2].strip() == want, (value, r.stdout, r.stderr[-500:])


def test_prepacked_entry_points_validate_before_launching():
    L = af.lib()
    assert af.prepack_bytes(4096, 4096, 8) == 4096 * 4096 and af.prepack_bytes(4096, 4096, 4) == 4096 * 4096 // 2
    assert af.prepack_bytes(4096, 4160, 4) == 0          # 4-bit packed order has K-chunks of 128 rows
    assert af.prepack_bytes(100, 4096, 8) == 0 and af.prepack_bytes(16, 64, 5) == 0
    assert af.prepack(P, P, 128, 256, stream=0, weight_bits=3, check=False) == -5
    assert af.prepack(P, P, 100, 256, stream=0, check=False) == -2
    assert af.prepack(P, P, 128, 192, stream=0, weight_bits=4, check=False) == -2
    assert af.prepack(P, P, 128, 256, ldb=64, stream=0, check=False) == -3
    assert af.prepack(None, P, 128, 256, stream=0, check=False) == -1
    assert af.prepack(P, P + 8, 128, 256, stream=0, check=False) == -4
    # column-major source: ldb counts the elements between columns (>= k)
    assert af.prepack_colmajor(P, P, 128, 256, stream=0, weight_bits=3, check=False) == -5
    assert af.prepack_colmajor(P, P, 100, 256, stream=0, check=False) == -2
    assert af.prepack_colmajor(P, P, 128, 256, ldb=128, stream=0, check=False) == -3
    assert af.prepack_colmajor(P, P, 128, 256, ldb=264, stream=0, check=False) == -3
    assert af.prepack_colmajor(P, None, 128, 256, stream=0, check=False) == -1
    assert af.prepack_colmajor(P + 4, P, 128, 256, stream=0, check=False) == -4
    assert af.prepack_colmajor(P, P, 0, 256, stream=0, check=False) == 0
    assert af.unpack(P, None, 128, 256, stream=0, check=False) == -1

    def rcp(**kw):
        d = dict(c=P, a=P, packed_b=P, scale=P, m=64, n=128, k=256, stream=0, check=False)
        d.update(kw)
        return af.gemm_prepacked(d.pop("c"), d.pop("a"), d.pop("packed_b"), d.pop("scale"), d.pop("m"), d.pop("n"), d.pop("k"), **d)
    assert rcp(weight_bits=5) == -5
    assert rcp(group_size=48) == -5
    assert rcp(n=100) == -2
    assert rcp(k=192, weight_bits=4) == -2
    assert rcp(lda=128) == -3
    assert rcp(ldc=64) == -3
    assert rcp(packed_b=None) == -1
    assert rcp(bias=P + 2) == -4
    assert rcp(which=9) == -7
    assert rcp(m=0) == 0
    assert af.prepacked_workspace_bytes(1, 4096, 4096) == 0 and af.prepacked_workspace_bytes(4096, 4096, 4096) == 0
    # (4-bit codes of so small a matrix run 128 columns per workgroup in either weight order; packed ones walk k in whole
    # K-chunks of 128 rows per wave, so their split factors are coarser)
    assert 0 < af.prepacked_workspace_bytes(64, 256, 4096, 4, 128) <= af.workspace_bytes(64, 256, 4096, 4, 128, af.DECODE)
    assert af.plan(16, 8192, 8192, 4, 128, packed=True).k_per_workgroup % 1024 == 0 and af.plan(64, 256, 4096, 4, 128, packed=True).k_per_workgroup % 512 == 0
    assert af.plan(64, 256, 4096, 4, 128, which=af.DECODE).tile_cols == 128 == af.plan(64, 256, 4096, 4, 128, packed=True, which=af.DECODE).tile_cols
    # packed 4-bit codes up to 32 rows: the slab kernel (16 columns) while the rows are few, then the 128-column form
    assert af.plan(8, 4096, 4096, 4, 128, packed=True).tile_cols == 16 and af.plan(12, 28672, 8192, 4, 128, packed=True).tile_cols == 128
    assert af.plan(16, 5120, 13824, 4, 128, packed=True).tile_cols == 128 and af.plan(32, 4096, 2048, 4, 128, packed=True).tile_cols == 16
    # (one round of workgroups, and only the split factors k divides into)
    assert af.plan(16, 11008, 8192, 4, 128, packed=True).splits == 2 and af.plan(16, 12288, 12288, 4, 128, packed=True).workgroups == 192
    assert af.plan(1, 28672, 8192, 4, 128).tile_cols == 256 and af.plan(24, 11008, 4096, 4, 128).tile_cols == 128
    # the small tiles split k over packed weights as over row-major ones: same plan, same scratch
    assert af.prepacked_variant(384, 2048, 8192, 4, 128) == af.PREFILL
    assert af.prepacked_workspace_bytes(384, 2048, 8192, 4, 128) == af.workspace_bytes(384, 2048, 8192, 4, 128, af.PREFILL) > 0
    assert rcp(m=64, n=256, k=4096, weight_bits=4, group_size=128) == -6     # the plan splits along k: workspace required
    assert af.prepacked_variant(1, 4096, 4096) == af.DECODE
    assert af.prepacked_variant(64, 4096, 4096) == af.DECODE
    # 48 .. 64 rows of 4-bit codes against many columns: row-major weights run the small tiles (54.5 against 74.5 us measured
    # at 64 x 28672 x 8192); packed ones have the family's 128-column form at every size, which is level with the tiles
    # there (54.1 / 53.1 us) and ahead on fewer columns (48 x 11008 x 8192: 30.7 / 33.3); from 96 rows the tiles
    assert af.variant(64, 28672, 8192, 4, 128) == af.PREFILL and af.prepacked_variant(96, 28672, 8192, 4, 128) == af.PREFILL
    assert af.prepacked_variant(48, 11008, 8192, 4, 128) == af.DECODE and af.plan(48, 11008, 8192, 4, 128, packed=True).tile_cols == 128
    assert af.variant(64, 4096, 4096) == af.DECODE and af.variant(192, 4096, 4096, 4, 128) == af.DECODE and af.variant(512, 4096, 4096, 4, 128) == af.PREFILL
    assert af.prepacked_variant(4096, 4096, 4096) == af.PREFILL
    assert af.prepacked_variant(1, 4096, 4160, 4, 0) == -2
    assert L.bfaintb_gemm_prepacked_variant(1, 100, 4096, 8, 0) == -2


def test_packed_file_header_and_round_trip(tmp_path):
    import torch
    L = af.lib()
    h = af.PackedHeader()
    assert C.sizeof(h) == 64
    assert L.bfaintb_packed_header_init(C.byref(h), 4096, 8192, 4, 128, 1) == 0
    assert (h.magic, h.header_bytes, h.layout, h.weight_bits, h.group_size, h.k, h.n) == (b"BFAINTB1", 64, 1, 4, 128, 8192, 4096)
    assert h.payload_bytes == 4096 * 8192 // 2 and h.scale_bytes == 64 * 4096 * 2 and h.has_bias == 1
    assert L.bfaintb_packed_header_check(C.byref(h)) == 0
    assert L.bfaintb_packed_header_init(C.byref(h), 4096, 4160, 4, 0, 0) == -2     # 4-bit: k % 128
    assert L.bfaintb_packed_header_init(C.byref(h), 4096, 4096, 8, 48, 0) == -5
    assert L.bfaintb_packed_header_init(None, 16, 64, 8, 0, 0) == -1
    L.bfaintb_packed_header_init(C.byref(h), 64, 128, 8, 0, 0)
    for field, bad in (("magic", b"BFAINTB2"), ("layout", 2), ("payload_bytes", 1), ("scale_bytes", 64), ("n", 72), ("has_bias", 2)):
        g = af.PackedHeader.from_buffer_copy(bytes(h))
        setattr(g, field, bad)
        assert L.bfaintb_packed_header_check(C.byref(g)) < 0, field
    # file round trip (host tensors: nothing here touches a device)
    n, k = 64, 128
    packed = torch.arange(n * k, dtype=torch.int64).to(torch.uint8)
    scale = torch.linspace(0.001, 0.01, n).to(torch.bfloat16).view(1, n)
    bias = torch.linspace(-1, 1, n).to(torch.bfloat16)
    path = str(tmp_path / "w.bfaintb")
    af.save_packed(path, packed, scale, n, k, 8, 0, bias)
    assert os.path.getsize(path) == 64 + n * k + 2 * n + 2 * n
    h2, p2, s2, b2 = af.load_packed(path, device="cpu")
    assert (h2.n, h2.k, h2.weight_bits, h2.has_bias) == (n, k, 8, 1)
    assert torch.equal(p2, packed) and torch.equal(s2.view(torch.int16), scale.view(torch.int16)) and torch.equal(b2.view(torch.int16), bias.view(torch.int16))
    with open(path, "ab") as f:
        f.write(b"x")
    with pytest.raises(ValueError):
        af.load_packed(path, device="cpu")


def test_product_does_not_reach_for_the_oracle():
    # the shipped package and the C/HIP sources must not import, include or link anything under oracle/
    pkg = os.path.join(ROOT, "awesome_fusion_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cc", ".cpp", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
