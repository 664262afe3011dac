// Tiled variant, 256x256 tiles, weights kept in registers: the prefill kernel, for row-major B (described first) and for B
// in the packed order (PACKED: what changes is said where the codes are loaded).
//
// Same job and the same reference kernel replaced as bfaintb_prefill_kernel
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630).  That kernel stages both operands in LDS and is bound
// by LDS traffic as much as by the matrix pipe (per K-step a CU reads 192 KiB and writes 64 KiB of LDS).  Here only A
// goes through LDS:
//   256 threads = 4 waves side by side along n; a wave owns ALL 256 rows x 64 columns of the tile, i.e. 16 x 4
//   accumulators of v_mfma_f32_16x16x32_bf16 (256 accumulator registers: one wave per SIMD, the whole register file).
//   Because a wave owns its 64 columns outright, it converts exactly the weights it multiplies by, straight into the
//   matrix instruction's operand registers: no W tile in LDS, no duplicate conversion, no LDS writes by the waves at all.
//   Lane (c16 = lane % 16, kq = lane / 16) loads, per block of 32 k and for each of the 8 rows k0 + 8 kq + r, one dword =
//   the codes of columns 4 c16 .. 4 c16 + 3 of the wave's 64 (16-bit loads for 4-bit codes): byte j of those 8 dwords is
//   the 8-element operand of column 4 c16 + j, rows 8 kq .. 8 kq + 7 — the layout v_mfma_f32_16x16x32_bf16 wants.
//   A: global -> LDS directly (buffer_load ... lds), four stages of 256 rows x 64 k (32 KiB each), rows of 128 bytes in 8
//   chunks of 16, chunk c of row r at position c ^ ((r >> 1) & 7); a fragment read is one ds_read_b128 (16 rows x 32 k).
//   Per K-step a CU reads 128 KiB of LDS and the copy engine writes 32 KiB.
// Pipeline per K-step of 64 (registers: operands of this step; raw codes of the next, loaded one step ago): request the
//   A tile of step+2 into the stage read two steps ago and the raw codes of step+2; convert the raw codes of step+1 into
//   the second operand set between the matrix instructions; 128 matrix instructions (2 blocks of 32 k x 16 row blocks x
//   4 columns), A fragments fetched one group of 16 ahead — the last group fetches the next step's first fragments, so no
//   step starts by waiting for LDS; one barrier, in the middle of the step.
// Accumulator (mt, j), register r of lane (c16, q = lane / 16): row 16 mt + 4 q + r, column 64 w + 4 c16 + j of the tile.
// Epilogue: bias, rounding to bf16, staging through LDS in [m][n] order, 16-byte row-contiguous stores; with a residual or
// the SiLU gate the fp32 sums are staged instead, 128 rows at a time, and finished 8 columns per thread.
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

namespace {
constexpr uint32_t kWrTile = 256, kWrK = 64;
constexpr uint32_t kWrStageBytes = 256 * 128;  // one A stage
constexpr uint32_t kWrCRowBytes = 256 * 2;     // epilogue staging row

__device__ __forceinline__ uint32_t wr_swz(uint32_t row, uint32_t chunk) { return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4); }

// acc += a x b with the accumulator pinned to the accumulation registers and updated in place.  Written as assembly
// because the compiler, given 256 accumulator registers, keeps part of them in ordinary registers and shuttles them
// back and forth around every matrix instruction (measured on this kernel's first form: 1772 copies for 384 matrix
// instructions).  What the compiler's hazard bookkeeping cannot see behind the assembly is kept safe by construction:
// the operands a and b are written (LDS reads, conversions) long before, under wait counts the compiler does insert
// for assembly operands; the accumulators are read by ordinary instructions only in the epilogue, behind explicit idle
// cycles (wreg_settle) that cover a matrix instruction's write latency.
__device__ __forceinline__ void mfma16(f32x4_t& acc, const bf16x8_t& a, const bf16x8_t& b)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void wreg_settle()
{
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
}
}  // namespace

template <int BITS, bool GROUPED, bool PACKED>
__global__ void __launch_bounds__(256) bfaintb_prefill_wreg_kernel(const GemmParams p)
{
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a0[kWrStageBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a1[kWrStageBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a2[kWrStageBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a3[kWrStageBytes];
    // (four separate arrays rather than one block: the compiler then knows that fragment reads of one stage cannot alias
    // the asynchronous copies into another, and does not make them wait for those)
    auto a_tile = [&](auto stage_c) -> uint8_t* {
        constexpr uint32_t St = decltype(stage_c)::value;
        return St == 0 ? lds_a0 : St == 1 ? lds_a1 : St == 2 ? lds_a2 : lds_a3;
    };

    using C0 = std::integral_constant<uint32_t, 0>;
    using C1 = std::integral_constant<uint32_t, 1>;
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // 0..3: the wave's 64 columns
    const uint32_t c16 = lane & 15u, kq = lane >> 4;

    // ---- tile of this workgroup: ids that share an XCD (id mod 8) cover consecutive logical ids, which walk groups of
    //      4 tile-rows column by column (as in bfaintb_prefill_kernel)
    const uint32_t tiles_m = (p.m + kWrTile - 1) / kWrTile, tiles_n = (p.n + kWrTile - 1) / kWrTile;
    const uint32_t wgs = p.tile_count;
    const uint32_t per_xcd = (wgs + 7u) / 8u;
    const uint32_t local = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (local >= wgs) return;
    const uint32_t logical = p.tile_first + local;
    const uint32_t group = logical / (4u * tiles_n);
    const uint32_t first_m = group * 4u;
    const uint32_t group_rows = tiles_m - first_m < 4u ? tiles_m - first_m : 4u;
    const uint32_t in_group = logical - group * 4u * tiles_n;
    const uint32_t tm = first_m + in_group % group_rows;
    const uint32_t tn = in_group / group_rows;
    const uint32_t m0 = tm * kWrTile, n0 = tn * kWrTile;

    const uint32_t rows_valid = p.m - m0 < kWrTile ? p.m - m0 : kWrTile;
    const uint32_t a_extent = ((rows_valid - 1u) * p.lda + p.k) * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.a + (size_t)m0 * p.lda), 0, (int)a_extent, kBufferFlags);
    const uint32_t cols_valid = p.n - n0 < kWrTile ? p.n - n0 : kWrTile;
    // packed weights: a block of 16 columns is one run of k x 16 codes (chunks of 1024 bytes: 64 rows of 8-bit, 128 rows of
    // 4-bit codes); the tile's column blocks follow one another, and one past n reads as zero through the extent
    const uint32_t slab_bytes = p.k * (BITS == 8 ? 16u : 8u);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (size_t)(n0 / 16u) * slab_bytes), 0,
                                                   (int)(cols_valid / 16u * slab_bytes), kBufferFlags)
               : __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (BITS == 8 ? n0 : n0 / 2u)), 0,
                                                   (int)((p.k - 1u) * p.ldb_bytes + (BITS == 8 ? cols_valid : cols_valid / 2u)), kBufferFlags);

    const uint32_t ksteps = (p.k + kWrK - 1u) / kWrK;
    const uint32_t last_chunks = (p.k - (ksteps - 1u) * kWrK) / 8u;  // valid 16-byte chunks per row of A in the last step

    // A copy: instruction j of wave w fills rows 64 w + 8 j .. + 7; lane l lands at row + l / 8, chunk position l % 8, so it
    // fetches chunk (l % 8) ^ ((row >> 1) & 7) = (l % 8) ^ (l / 16) for even j and that ^ 4 for odd j: two lane offsets, the
    // row advance of j (and the K advance) in the scalar offset.
    const uint32_t a_row = 64u * wave + (lane >> 3);
    const uint32_t chunk_e = (lane & 7u) ^ ((lane >> 4) & 7u), chunk_o = chunk_e ^ 4u;
    const uint32_t a_voff_e = (a_row * p.lda + chunk_e * 8u) * 2u, a_voff_o = (a_row * p.lda + chunk_o * 8u) * 2u;
    // a chunk past the end of k (partial last step) is fetched from beyond the extent: it reads as zero
    const uint32_t a_last_e = chunk_e < last_chunks ? a_voff_e : a_extent, a_last_o = chunk_o < last_chunks ? a_voff_o : a_extent;
    auto dma_a = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = a_tile(stage_c) + wave * 8192u;
        const bool last = kt + 1u == ksteps;
        const uint32_t ve = last ? a_last_e : a_voff_e, vo = last ? a_last_o : a_voff_o;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16,
                                                     (j & 1u) ? vo : ve, kt * kWrK * 2u + j * 16u * p.lda, 0, 0);
        __builtin_amdgcn_sched_barrier(0);  // the copy's requests stay ahead of the loads that follow: the wait below counts on it
    };

    // W: this lane's 4 columns, rows 8 kq .. 8 kq + 7 of a block of 32 k.  Row-major weights: four neighbouring columns
    // (one dword of a row holds them).  Packed weights: column c16 of each of the wave's four column blocks — the packed
    // order gives lane 16 kq + c16 of a column block, in 16 bytes, exactly these rows of that column for the chunk's
    // K-blocks (two for 8-bit codes = this step; four for 4-bit codes, of which a step takes 8 bytes).
    const uint32_t wcol = PACKED ? 64u * wave + c16 : 64u * wave + 4u * c16;  // the lane's column j is wcol + kColStep * j
    constexpr uint32_t kColStep = PACKED ? 16u : 1u;
    const uint32_t b_voff = PACKED ? lane * 16u : 8u * kq * p.ldb_bytes + (BITS == 8 ? wcol : wcol / 2u);
    const bool w_ok = n0 + wcol < p.n;  // (packed: the lane's four columns are whole column blocks apart, checked each on its own)
    auto col_ok = [&](uint32_t j) { return n0 + wcol + kColStep * j < p.n; };
    // packed: where column block j of this wave starts, and where a step's codes are within it
    auto slab_off = [&](uint32_t j) { return (4u * wave + j) * slab_bytes; };
    auto step_off = [&](uint32_t kt) { return BITS == 8 ? kt * 1024u : (kt >> 1) * 1024u + (kt & 1u) * 8u; };
    struct Raw {
        // row-major: [block of 32 k][row] (8-bit: a dword of four columns; 4-bit: 16 bits)
        // packed: [block][2 j + half] = rows 4 half .. + 3 of column j (8-bit); [block][j] = the 8 rows of column j (4-bit)
        uint32_t d[2][8];
        uint32_t s[2][PACKED ? 4 : 2];  // grouped scales of the two blocks: row-major 4 bf16 in two dwords, packed one each
    };
    // packed: the codes of column block j for step kt, one request
    auto gload_packed = [&](Raw& raw, uint32_t kt, uint32_t j) {
        if constexpr (BITS == 8) {
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, b_voff, slab_off(j) + step_off(kt), 0);
            raw.d[0][2 * j] = v[0], raw.d[0][2 * j + 1] = v[1], raw.d[1][2 * j] = v[2], raw.d[1][2 * j + 1] = v[3];
        } else {
            const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_b, b_voff, slab_off(j) + step_off(kt), 0);
            raw.d[0][j] = v[0], raw.d[1][j] = v[1];
        }
    };
    // Scales go through a buffer resource so that the load is issued whatever the lane's column (the wait counts
    // below count requests): columns past n read other columns' scales, or zero beyond the array; their results are
    // never stored.
    const uint32_t scale_rows = GROUPED ? p.k / p.group_size : 1u;
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.scale), 0, (int)(((scale_rows - 1u) * p.lds + p.n) * 2u), kBufferFlags);
    const uint32_t s_voff = (n0 + wcol) * 2u;
    // the grouped scales of block blk of step kt (packed: of the lane's column j alone)
    auto load_group_scales = [&](Raw& raw, uint32_t kt, uint32_t blk, uint32_t j = 0) {
        uint32_t g = group_of_row(p, kt * kWrK + 32u * blk);
        if (g >= scale_rows) g = scale_rows - 1u;  // rows past k in a partial last step: any scale will do
        if constexpr (PACKED) {
            raw.s[blk][j] = __builtin_amdgcn_raw_buffer_load_b16(rsrc_s, s_voff, g * p.lds * 2u + 32u * j, 0);
        } else {
            const u32x2_t sr = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, s_voff, g * p.lds * 2u, 0);
            raw.s[blk][0] = sr[0];
            raw.s[blk][1] = sr[1];
        }
    };
    auto gload = [&](Raw& raw, uint32_t kt) {
        if constexpr (PACKED) {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) gload_packed(raw, kt, j);
        }
#pragma unroll
        for (uint32_t blk = 0; blk < 2; ++blk) {
            if constexpr (!PACKED) {
                const uint32_t row0 = (kt * kWrK + 32u * blk) * p.ldb_bytes;
#pragma unroll
                for (uint32_t r = 0; r < 8; ++r) {
                    if constexpr (BITS == 8) raw.d[blk][r] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_b, b_voff, row0 + r * p.ldb_bytes, 0);
                    else raw.d[blk][r] = __builtin_amdgcn_raw_buffer_load_b16(rsrc_b, b_voff, row0 + r * p.ldb_bytes, 0);
                }
            }
            if constexpr (GROUPED) {
                if constexpr (PACKED) {
#pragma unroll
                    for (uint32_t j = 0; j < 4; ++j) load_group_scales(raw, kt, blk, j);
                } else {
                    load_group_scales(raw, kt, blk);
                }
            }
        }
    };
    float cs[4];
    if constexpr (!GROUPED) {
        if constexpr (PACKED) {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) cs[j] = make_col_scale<BITS>(__builtin_amdgcn_raw_buffer_load_b16(rsrc_s, s_voff, 32u * j, 0));
        } else {
            const u32x2_t sr = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, s_voff, 0, 0);
            cs[0] = make_col_scale<BITS>(sr[0] & 0xffffu);
            cs[1] = make_col_scale<BITS>(sr[0] >> 16);
            cs[2] = make_col_scale<BITS>(sr[1] & 0xffffu);
            cs[3] = make_col_scale<BITS>(sr[1] >> 16);
        }
    }
    struct Ops {
        bf16x8_t w[2][4];  // [block of 32 k][column j]
    };
    // byte `col` (a compile-time value at every call site) of a dword of signed bytes, as fp32
    auto sbyte_sel = [&](uint32_t x, uint32_t col) -> float {
        return col == 0 ? sbyte_to_f32<0>(x) : col == 1 ? sbyte_to_f32<1>(x) : col == 2 ? sbyte_to_f32<2>(x) : sbyte_to_f32<3>(x);
    };
    // The signed bytes of a block, s8[8].  Row-major: s8[r] = row r of the lane's 8, byte j = column j.  Packed: s8[2 j + h]
    // = column j, byte t = row 4 h + t.  weight(s8, r, j): row r of column j as fp32 (r and j compile-time at every call).
    auto weight = [&](const uint32_t (&s8)[8], uint32_t r, uint32_t j) -> float {
        return PACKED ? sbyte_sel(s8[2u * j + (r >> 2)], r & 3u) : sbyte_sel(s8[r], j);
    };
    // entry e of s8 from the raw codes of block BLK
    auto signed_bytes = [&](const Raw& raw, auto blk_c, uint32_t e) -> uint32_t {
        constexpr int BLK = decltype(blk_c)::value;
        if constexpr (BITS == 8) return codes8_to_s8(raw.d[BLK][e]);
        else if constexpr (PACKED) return codes4_quad_to_s8x16(raw.d[BLK][e >> 1] >> (16u * (e & 1u)));  // 8 codes of a column: 4 per entry
        else return codes4_quad_to_s8x16(raw.d[BLK][e]);
    };
    auto block_scales = [&](float (&sc)[4], const Raw& raw, auto blk_c) {
        constexpr int BLK = decltype(blk_c)::value;
        if constexpr (PACKED) {
#pragma unroll
            for (int j = 0; j < 4; ++j) sc[j] = make_col_scale<BITS>(raw.s[BLK][j]);
        } else {
            sc[0] = make_col_scale<BITS>(raw.s[BLK][0] & 0xffffu);
            sc[1] = make_col_scale<BITS>(raw.s[BLK][0] >> 16);
            sc[2] = make_col_scale<BITS>(raw.s[BLK][1] & 0xffffu);
            sc[3] = make_col_scale<BITS>(raw.s[BLK][1] >> 16);
        }
    };
    // one column of one block: 8 weights -> operand
    auto convert_col = [&](Ops& ops, const uint32_t (&s8)[8], const float (&sc)[4], auto blk_c, auto j_c) {
        constexpr int BLK = decltype(blk_c)::value, J = decltype(j_c)::value;
        uint4 w;
        w.x = pack_bf16_rne(weight(s8, 0, J) * sc[J], weight(s8, 1, J) * sc[J]);
        w.y = pack_bf16_rne(weight(s8, 2, J) * sc[J], weight(s8, 3, J) * sc[J]);
        w.z = pack_bf16_rne(weight(s8, 4, J) * sc[J], weight(s8, 5, J) * sc[J]);
        w.w = pack_bf16_rne(weight(s8, 6, J) * sc[J], weight(s8, 7, J) * sc[J]);
        ops.w[BLK][J] = __builtin_bit_cast(bf16x8_t, w);
    };
    // the raw codes of one block -> signed bytes, and the block's four column scales
    auto prepare_block = [&](uint32_t (&s8)[8], float (&sc)[4], const Raw& raw, auto blk_c) {
#pragma unroll
        for (int e = 0; e < 8; ++e) s8[e] = signed_bytes(raw, blk_c, e);
        if constexpr (GROUPED) {
            block_scales(sc, raw, blk_c);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) sc[j] = cs[j];
        }
    };
    auto convert_block = [&](Ops& ops, const Raw& raw, auto blk_c) {
        uint32_t s8[8];
        float sc[4];
        prepare_block(s8, sc, raw, blk_c);
        convert_col(ops, s8, sc, blk_c, std::integral_constant<int, 0>{});
        convert_col(ops, s8, sc, blk_c, std::integral_constant<int, 1>{});
        convert_col(ops, s8, sc, blk_c, std::integral_constant<int, 2>{});
        convert_col(ops, s8, sc, blk_c, std::integral_constant<int, 3>{});
    };

    f32x4_t acc[16][4];
#pragma unroll
    for (int mt = 0; mt < 16; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[mt][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // fragment (mt, blk): row 16 mt + c16 of the tile, chunk 4 blk + kq
    uint32_t a_rd[2];
#pragma unroll
    for (uint32_t blk = 0; blk < 2; ++blk) a_rd[blk] = wr_swz(c16, 4u * blk + kq);  // + mt * 2048 (16 rows; the swizzle repeats every 16 rows)
    auto read_frag = [&](auto stage_c, uint32_t blk, uint32_t mt) -> bf16x8_t {
        return *reinterpret_cast<const bf16x8_t*>(a_tile(stage_c) + a_rd[blk] + mt * 2048u);
    };

    // One K-step: stage S and `cur` hold this step; `nxt` receives the operands of step kt + 1 from `raw1` (loaded one
    // step ago); `raw2` receives the codes of step kt + 2.
    // With one wave per SIMD nothing overlaps by itself: the wave issues in order, and the matrix pipe idles whenever the
    // wave is busy issuing something else for longer than a matrix instruction runs (16 cycles).  So the step is written
    // as 128 slots of one matrix instruction plus at most a few other instructions, fenced so the compiler keeps them
    // that way: slot (g, i, j) — group g of 16 (block of 32 k = g / 4, row blocks 4 (g % 4) .. + 3), row block i, column j:
    //   j = 0  fetch the A fragment (g + 1, i) of the next group
    //   j = 1, 3  a quarter of a column's conversion: column g % 4 of block g / 4 of the NEXT step's weights, rows 2 i,
    //          2 i + 1 of the lane's 8 (five instructions, three in slot 1 and two in slot 3)
    //   j = 2  one request to memory: the 8 A copies in groups 0-1, the 16 raw-code loads in groups 2-5, the scales in group 6
    //   j = 3  also, in group 3: two rows of the next block's codes made signed
    bf16x8_t af[2][4];  // A fragments of the group being multiplied and of the next one; af[0] carries over from step to step
    auto step = [&](auto stage_c, uint32_t kt, const Ops& cur, Ops& nxt, const Raw& raw1, Raw& raw2) {
        constexpr uint32_t S = decltype(stage_c)::value;
        using Next = std::integral_constant<uint32_t, (S + 1u) & 3u>;
        using Target = std::integral_constant<uint32_t, (S + 2u) & 3u>;
        const uint32_t kt2 = kt + 2 < ksteps ? kt + 2 : ksteps - 1;
        const bool last = kt2 + 1u == ksteps;
        const uint32_t a_ve = last ? a_last_e : a_voff_e, a_vo = last ? a_last_o : a_voff_o;
        uint8_t* const a_dst = a_tile(Target{}) + wave * 8192u;
        uint32_t s8[8];
        float sc[4];
        uint32_t wq[2][4][4];  // the next step's operands as they are built: [block][column][dword]
        float f_lo = 0.f, f_hi = 0.f;
        prepare_block(s8, sc, raw1, B0{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t g = 0; g < 8; ++g) {
            const uint32_t blk = g >> 2, mt0 = 4u * (g & 3u);
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) {
                    mfma16(acc[mt0 + i][j], af[g & 1][i], cur.w[blk][j]);
                    if (j == 0) {
                        if (g + 1 < 8) af[(g + 1) & 1][i] = read_frag(stage_c, (g + 1) >> 2, 4u * ((g + 1) & 3u) + i);
                        else af[0][i] = read_frag(Next{}, 0, i);  // the next step's first group (its stage is complete: see the barrier)
                    }
                    if (j == 1) {  // (the five instructions of a quarter column are split 3 + 2 over slots j = 1 and j = 3)
                        const uint32_t col = g & 3u;
                        f_lo = weight(s8, 2 * i, col) * sc[col];
                        f_hi = weight(s8, 2 * i + 1, col);
                    }
                    if (j == 2) {
                        const uint32_t q = 4u * g + i;  // 0..31
                        if (q < 8) {
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(a_dst + q * 1024u), 16,
                                                                     (q & 1u) ? a_vo : a_ve, kt2 * kWrK * 2u + q * 16u * p.lda, 0, 0);
                        } else if constexpr (PACKED) {  // 4 requests for the codes, then 8 for the scales
                            if (q < 12) gload_packed(raw2, kt2, q - 8u);
                            else if (GROUPED && q < 20) load_group_scales(raw2, kt2, (q - 12u) >> 2, (q - 12u) & 3u);
                        } else if (q < 24) {
                            const uint32_t lb = (q - 8u) >> 3, r = (q - 8u) & 7u;
                            const uint32_t soff = (kt2 * kWrK + 32u * lb + r) * p.ldb_bytes;
                            if constexpr (BITS == 8) raw2.d[lb][r] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_b, b_voff, soff, 0);
                            else raw2.d[lb][r] = __builtin_amdgcn_raw_buffer_load_b16(rsrc_b, b_voff, soff, 0);
                        } else if (GROUPED && q < 26) {
                            load_group_scales(raw2, kt2, q - 24u);
                        }
                    }
                    if (j == 3) wq[blk][g & 3u][i] = pack_bf16_rne(f_lo, f_hi * sc[g & 3u]);
                    if (j == 3 && g == 3) {
                        // block 1's codes made signed, two entries per slot, into the part of s8 whose conversion is done
                        // (row-major: rows 2 i, 2 i + 1 of block 0 were last used by slot (3, i, 1); packed: column i of
                        // block 0 was converted in group i, its last rows by slot (i, 3, 1))
                        s8[2 * i] = signed_bytes(raw1, B1{}, 2 * i);
                        s8[2 * i + 1] = signed_bytes(raw1, B1{}, 2 * i + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (g == 3) {
                if constexpr (GROUPED) block_scales(sc, raw1, B1{});
                // The step's one barrier, in the middle.  Before it the wave makes sure that its part of the A tile of step
                // kt + 1 has landed (requested during step kt - 1; since then it has requested the rest of that step's codes and
                // scales, this step's A copy and 8 loads of codes: at most that many requests may still be in flight).  Behind
                // it every wave's part has: the next step's first fragments can be fetched at the end of this one, and the
                // copy this step started (into the stage read two steps ago) overwrites nothing a wave still reads — every
                // wave that reaches this barrier has passed the previous one, i.e. finished the step before it.
                // (row-major: 16 loads of codes and 2 of scales per step, 8 of the codes before this point; packed: 4 of codes
                // and 8 of scales, 4 + 4 of them before this point)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PACKED ? (GROUPED ? 12 + 16 : 4 + 12) : (GROUPED ? 18 : 16) + 16) : "memory");
                barrier_no_fence();  // (a fenced barrier would also wait for the copy this step has just started)
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int b2 = 0; b2 < 2; ++b2)
#pragma unroll
            for (int c2 = 0; c2 < 4; ++c2)
                nxt.w[b2][c2] = __builtin_bit_cast(bf16x8_t, make_uint4(wq[b2][c2][0], wq[b2][c2][1], wq[b2][c2][2], wq[b2][c2][3]));
    };

    // ---- prologue: A tiles 0 and 1 -> stages 0 and 1; operands of step 0; raw codes of step 1; the first fragments
    Ops ops0, ops1;
    Raw rawa, rawb;
    dma_a(C0{}, 0);
    dma_a(C1{}, ksteps > 1 ? 1 : 0);
    gload(rawa, 0);
    convert_block(ops0, rawa, B0{});
    convert_block(ops0, rawa, B1{});
    gload(rawa, ksteps > 1 ? 1 : 0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PACKED ? (GROUPED ? 12 : 4) : (GROUPED ? 18 : 16)) : "memory");
    __syncthreads();
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) af[0][i] = read_frag(C0{}, 0, i);

    using C2 = std::integral_constant<uint32_t, 2>;
    using C3 = std::integral_constant<uint32_t, 3>;
#ifdef BFAINTB_TRACE
    const long long tr_c0 = clock64(), tr_w0 = wall_clock64();
#endif
    uint32_t kt = 0;
    for (; kt + 3 < ksteps; kt += 4) {
        step(C0{}, kt, ops0, ops1, rawa, rawb);
        step(C1{}, kt + 1, ops1, ops0, rawb, rawa);
        step(C2{}, kt + 2, ops0, ops1, rawa, rawb);
        step(C3{}, kt + 3, ops1, ops0, rawb, rawa);
    }
    if (kt < ksteps) step(C0{}, kt, ops0, ops1, rawa, rawb);
    if (kt + 1 < ksteps) step(C1{}, kt + 1, ops1, ops0, rawb, rawa);
    if (kt + 2 < ksteps) step(C2{}, kt + 2, ops0, ops1, rawa, rawb);
#ifdef BFAINTB_TRACE
    {   // shader cycles and 100 MHz ticks the K loop took, per wave: words 0, 1 of the wave's 8
        const long long tr_c1 = clock64(), tr_w1 = wall_clock64();
        if (lane == 0 && p.trace != nullptr) {
            unsigned long long* t = p.trace + (size_t)(blockIdx.x * 4u + wave) * 8u;
            t[0] = (unsigned long long)(tr_c1 - tr_c0);
            t[1] = (unsigned long long)(tr_w1 - tr_w0);
            t[2] = (unsigned long long)tr_w0;
            t[3] = (unsigned long long)tr_w1;
        }
    }
#endif

    // ---- epilogue: bf16 tile through LDS (rows 64 q .. 64 q + 63 in the q-th array), then 16-byte row-contiguous stores
    wreg_settle();  // the last matrix instructions have written their accumulators
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing asynchronous may still be writing LDS
    __syncthreads();
    auto c_rows = [&](uint32_t q) -> uint8_t* { return q == 0 ? lds_a0 : q == 1 ? lds_a1 : q == 2 ? lds_a2 : lds_a3; };
    const bool gated = p.activation == kActSiluGate;
    if (p.residual == nullptr && !gated) {
        // the bare sums, or sums + bias: rounded in registers, staged as bf16 (rows 64 q .. 64 q + 63 in the q-th array)
        float bias[4] = {0.f, 0.f, 0.f, 0.f};
        const bool has_bias = p.bias != nullptr;
        if constexpr (PACKED) {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                if (has_bias && col_ok(j)) bias[j] = bf16_bits_to_f32(p.bias[n0 + wcol + kColStep * j]);
        } else if (has_bias && w_ok) {
            const uint2 raw = *reinterpret_cast<const uint2*>(p.bias + n0 + wcol);
            bias[0] = bf16_bits_to_f32(raw.x & 0xffffu);
            bias[1] = bf16_bits_to_f32(raw.x >> 16);
            bias[2] = bf16_bits_to_f32(raw.y & 0xffffu);
            bias[3] = bf16_bits_to_f32(raw.y >> 16);
        }
        // Packed weights: a lane's four columns are 16 apart, so it stages four single values per row, and the four
        // k-groups of a wave (rows 4 apart: the same banks) would collide; the 32-byte groups of a row are therefore
        // stored at position (group ^ ((row >> 2) & 3)), which the readers below undo.
        uint32_t pk_base[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) pk_base[j] = 4u * kq * kWrCRowBytes + (((4u * wave + j) ^ kq) << 5) + c16 * 2u;
#pragma unroll
        for (uint32_t mt = 0; mt < 16; ++mt) {
            uint8_t* base = c_rows(mt >> 2);
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t row = 16u * (mt & 3u) + 4u * kq + r;  // within the 64 rows of this array
                uint2 o;
                // without a bias the sums are stored as they are (adding +0 would turn a -0 sum into +0)
                if (has_bias) {
                    o.x = pack_bf16_rne(acc[mt][0][r] + bias[0], acc[mt][1][r] + bias[1]);
                    o.y = pack_bf16_rne(acc[mt][2][r] + bias[2], acc[mt][3][r] + bias[3]);
                } else {
                    o.x = pack_bf16_rne(acc[mt][0][r], acc[mt][1][r]);
                    o.y = pack_bf16_rne(acc[mt][2][r], acc[mt][3][r]);
                }
                if constexpr (PACKED) {
                    uint8_t* at = base + (16u * (mt & 3u) + r) * kWrCRowBytes;  // + the lane's part, in pk_base
                    *reinterpret_cast<uint16_t*>(at + pk_base[0]) = (uint16_t)(o.x & 0xffffu);
                    *reinterpret_cast<uint16_t*>(at + pk_base[1]) = (uint16_t)(o.x >> 16);
                    *reinterpret_cast<uint16_t*>(at + pk_base[2]) = (uint16_t)(o.y & 0xffffu);
                    *reinterpret_cast<uint16_t*>(at + pk_base[3]) = (uint16_t)(o.y >> 16);
                } else {
                    *reinterpret_cast<uint2*>(base + row * kWrCRowBytes + wcol * 2u) = o;
                }
            }
        }
        __syncthreads();
#pragma unroll 4
        for (uint32_t pass = 0; pass < 32u; ++pass) {
            const uint32_t row = pass * 8u + (tid >> 5);
            const uint32_t ch = tid & 31u;
            const uint32_t gm = m0 + row, gn = n0 + ch * 8u;
            if (gm < p.m && gn < p.n) {
                const uint32_t at = PACKED ? ((((ch >> 1) ^ ((row >> 2) & 3u)) << 5) + (ch & 1u) * 16u) : ch * 16u;
                const uint4 v = *reinterpret_cast<const uint4*>(c_rows(row >> 6) + (row & 63u) * kWrCRowBytes + at);
                *reinterpret_cast<uint4*>(p.c + (size_t)gm * p.ldc + gn) = v;
            }
        }
        return;
    }
    // Residual and / or the SiLU gate: the fp32 sums are staged in [m][n] order, 128 rows at a time (128 x 256 x 4 bytes
    // = the four arrays, rows 32 q .. 32 q + 31 of the half in the q-th), and each thread finishes 8 neighbouring columns
    // of a row — bias, gate, residual, the one rounding — as the small-tile kernels do.
    const uint32_t ch = tid & 31u;  // 8 columns: 8 ch .. 8 ch + 7 of the tile
    const uint32_t gn = n0 + 8u * ch;
    float bias8[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) bias8[i] = 0.f;
    if (p.bias != nullptr && gn < p.n) {
        const uint4 raw = *reinterpret_cast<const uint4*>(p.bias + gn);
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bias8[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
            bias8[2 * i + 1] = bf16_bits_to_f32(d[i] >> 16);
        }
    }
#pragma unroll
    for (uint32_t half = 0; half < 2; ++half) {
#pragma unroll
        for (uint32_t mh = 0; mh < 8; ++mh) {
            const uint32_t mt = 8u * half + mh;
            float* base = reinterpret_cast<float*>(c_rows(mh >> 1));
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t row = 16u * (mh & 1u) + 4u * kq + r;  // within the 32 rows of this array
                if constexpr (PACKED) {
#pragma unroll
                    for (uint32_t j = 0; j < 4; ++j) base[row * kWrTile + wcol + kColStep * j] = acc[mt][j][r];
                } else {
                    *reinterpret_cast<float4*>(base + row * kWrTile + wcol) = make_float4(acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]);
                }
            }
        }
        __syncthreads();
#pragma unroll 4
        for (uint32_t pass = 0; pass < 16u; ++pass) {
            const uint32_t row = pass * 8u + (tid >> 5);  // within the half
            const uint32_t gm = m0 + 128u * half + row;
            if (gm >= p.m || gn >= p.n) continue;
            const float* src = reinterpret_cast<const float*>(c_rows(row >> 5)) + (row & 31u) * kWrTile + 8u * ch;
            const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
            float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] += bias8[i];
            if (gated) {
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = silu_gate(v[2 * i], v[2 * i + 1]);
                if (p.residual != nullptr) {
                    const uint2 r = *reinterpret_cast<const uint2*>(p.residual + (size_t)gm * p.ldr + gn / 2u);
                    o[0] += bf16_bits_to_f32(r.x & 0xffffu);
                    o[1] += bf16_bits_to_f32(r.x >> 16);
                    o[2] += bf16_bits_to_f32(r.y & 0xffffu);
                    o[3] += bf16_bits_to_f32(r.y >> 16);
                }
                *reinterpret_cast<uint2*>(p.c + (size_t)gm * p.ldc + gn / 2u) = make_uint2(pack_bf16_rne(o[0], o[1]), pack_bf16_rne(o[2], o[3]));
            } else {
                const uint4 r = *reinterpret_cast<const uint4*>(p.residual + (size_t)gm * p.ldr + gn);
                const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    v[2 * i] += bf16_bits_to_f32(d[i] & 0xffffu);
                    v[2 * i + 1] += bf16_bits_to_f32(d[i] >> 16);
                }
                *reinterpret_cast<uint4*>(p.c + (size_t)gm * p.ldc + gn) =
                    make_uint4(pack_bf16_rne(v[0], v[1]), pack_bf16_rne(v[2], v[3]), pack_bf16_rne(v[4], v[5]), pack_bf16_rne(v[6], v[7]));
            }
        }
        __syncthreads();  // the second half overwrites the staging area
    }
}

// Runs `tile_count` whole 256x256 tiles from `tile_first` on (the caller splits off a last, thin round for the half-tile kernel).
template <int BITS, bool GROUPED, bool PACKED>
static hipError_t launch_wreg_t(const GemmParams& p, hipStream_t stream)
{
    const uint32_t grid = (p.tile_count + 7u) / 8u * 8u;  // a whole number of workgroups per XCD; ids past the last tile exit at once
    void (*kernel)(const GemmParams) = bfaintb_prefill_wreg_kernel<BITS, GROUPED, PACKED>;
    return launch_kernel(kernel, dim3(grid, 1, 1), dim3(256, 1, 1), 0, stream, p);
}

// Whether this kernel can serve a launch: this library's own arithmetic (either order of the weights).
bool prefill_wreg_serves(const GemmParams& p) { return !p.reference_arith; }

template <bool PACKED>
static hipError_t launch_wreg_order(const GemmParams& p, int bits, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    if (bits == 8) return grouped ? launch_wreg_t<8, true, PACKED>(p, stream) : launch_wreg_t<8, false, PACKED>(p, stream);
    return grouped ? launch_wreg_t<4, true, PACKED>(p, stream) : launch_wreg_t<4, false, PACKED>(p, stream);
}

// packed: p.b is the buffer in the packed order (p.ldb_bytes is unused)
hipError_t launch_prefill_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream)
{
    return packed ? launch_wreg_order<true>(p, bits, stream) : launch_wreg_order<false>(p, bits, stream);
}

}  // namespace bfaintb
