// Prefill variant (m > 32): 256x256x64 LDS-tiled bf16 MFMA kernel for gfx950.
//
// Replaces the reference kernel's 32x64x64 tile, two waves, v_mfma_f32_32x32x8bf16_1k,
// single-buffered LDS with two barriers per K-step
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:410-489, tile origin :222-223,
// LDS layouts :346-393, epilogue :594-630).
//
// Shape of the computation
//   One workgroup of 512 threads (8 waves, 2 along m x 4 along n) per 256x256 tile of C; each wave
//   owns a 128 x 64 block = 4 x 2 accumulators of v_mfma_f32_32x32x16_bf16.  K advances 64 per step.
//   LDS holds two stages of {A tile, dequantised W tile}; a tile is 256 rows x 64 k of bf16 (a row is
//   128 bytes = 8 chunks of 16 bytes), so one barrier per step suffices.  Chunk c of row r lives at
//   chunk position c ^ ((r >> 1) & 7): 16 lanes that read, or 8 lanes that write, the same chunk of
//   consecutive rows land in different 16-byte bank groups.
//   Workgroup ids are remapped so that the workgroups an XCD receives (id mod 8) form a compact
//   4 x 8 block of tiles: each XCD's L2 then fetches 4 row-panels of A and 8 column-panels of B
//   instead of every row-panel of A.
// Global loads are raw buffer loads: a lane's byte offset sits in one VGPR, the K advance (and for B
// the row) in an SGPR offset, so the loop carries no vector address arithmetic and no predication.
// The buffers' extents end with the tile's last valid row of A and the last row of B (gfx9-family
// range checks add the SGPR offset to the lane offset): rows of A past m read as zero; columns of B
// past n read whatever lies there, or zero past the end of B, and feed only columns that are never stored.
// A path: global -> LDS directly (buffer_load ... lds, 16 bytes per lane, 8 lanes per row), each lane fetching the chunk
//   that the swizzle places at its LDS position.
// W path (row-major B; the PACKED instantiation reads the packed order instead, see the kernel): wave w loads rows 8w..8w+7 of the step, one dword (4 codes) per lane per row, so a lane
//   ends up with 8 consecutive k of 4 columns; it dequantises them (xor, cvt with sign-extending
//   byte select, multiply, cvt_pk) and writes one 16-byte chunk per column.  Column (4*lane + j)
//   goes to LDS row rho = (j>>1)*128 + (j&1)*32 + (lane&31) + (lane>>5)*64, so consecutive lanes
//   write consecutive rows.  The MFMA "column" index is the LDS row: wave wn, accumulator t, lane
//   column jl hold tile column 4*(32*(wn&1) + jl) + 2*(wn>>1) + t.
// Pipeline per step (registers hold the raw W tile of step+1, loaded one step earlier): the 32 MFMAs
//   of the current stage run in four quarters; the raw tile is converted and written to the other
//   stage between the MFMAs of the second and third quarter, the registers it frees are refilled
//   with step+2 at once, and the barrier sits before the last quarter so that the first fragments
//   of the next stage are fetched behind those MFMAs.
// Launches: whole 256-row tiles, then (a last round of 256 workgroups that would be less than half full, or fewer
//   than 128 tiles in all) 128-row half tiles, MT = 2.
// Epilogue: accumulators are rounded to bf16 (v_cvt_pk_bf16_f32; t = 0,1 are neighbouring columns
//   and share a dword), staged in LDS in true [m][n] order and stored with 16-byte row-contiguous writes.
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr uint32_t kTileBytes = 256 * 128;              // one A or W tile in LDS
constexpr int kCRowBytes = 256 * 2;                     // epilogue staging row: 64 rows fill one 32 KiB tile array


__device__ __forceinline__ uint32_t swizzled_off(uint32_t row, uint32_t chunk)
{
    return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4);
}

// MT = blocks of 32 rows per wave along m: 4 for the 256-row tile, 2 for a 128-row half tile.  Half tiles take
// over the tiles of a last, less than half full round of 256 workgroups: twice as many workgroups, each with half
// the matrix instructions (and all of the weight conversion), finish sooner than half-idle CUs running whole tiles.
// REF: the reference kernel's arithmetic (p.reference_arith): one fp32 scale per column, W and C narrowed by truncation.
template <int BITS, bool GROUPED, int MT, bool PACKED, bool REF>
__global__ void __launch_bounds__(512) bfaintb_prefill_kernel(const GemmParams p)
{
    static_assert(!REF || (BITS == 8 && !GROUPED && !PACKED), "the reference's arithmetic: 8-bit codes, row-major, one scale per column");
    constexpr uint32_t kRows = 64u * MT;  // rows of C per workgroup
    // Four separate LDS arrays (A and W tiles, two stages each) rather than one block: the compiler
    // then knows that fragment reads of one stage cannot alias the asynchronous global->LDS writes
    // into the other, and does not make them wait for those writes.
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w1[kTileBytes];
    auto a_tile = [&](auto stage_c) -> uint8_t* { return decltype(stage_c)::value == 0 ? lds_a0 : lds_a1; };
    auto w_tile = [&](auto stage_c) -> uint8_t* { return decltype(stage_c)::value == 0 ? lds_w0 : lds_w1; };

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
    const uint32_t wm = wave >> 2;   // 0..1
    const uint32_t wn = wave & 3u;   // 0..3

    // ---- tile of this workgroup: ids that share an XCD (id mod 8) cover consecutive logical ids;
    //      logical ids walk groups of 4 tile-rows column by column
    //      This launch covers logical tiles tile_first .. tile_first + tile_count - 1 (two workgroups per tile when MT = 2).
    const uint32_t tiles_m = (p.m + kBM - 1) / kBM, tiles_n = (p.n + kBN - 1) / kBN;
    const uint32_t wgs = p.tile_count * (4u / MT);
    const uint32_t per_xcd = (wgs + 7u) / 8u;
    const uint32_t local = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (local >= wgs) return;
    const uint32_t logical = p.tile_first + local / (4u / MT);
    const uint32_t mhalf = MT == 4 ? 0u : (local & 1u);
    const uint32_t group = logical / (4u * tiles_n);
    const uint32_t first_m = group * 4u;
    const uint32_t group_rows = tiles_m - first_m < 4u ? tiles_m - first_m : 4u;
    const uint32_t in_group = logical - group * 4u * tiles_n;
    const uint32_t tm = first_m + in_group % group_rows;
    const uint32_t tn = in_group / group_rows;
    const uint32_t m0 = tm * kBM + mhalf * kRows, n0 = tn * kBN;
    if (m0 >= p.m) return;  // the lower half of a tile that ends in its upper half

    // ---- buffer resources over this tile's rows of A and columns of B
    const uint32_t rows_valid = p.m - m0 < kRows ? p.m - m0 : kRows;
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.a + (size_t)m0 * p.lda), 0, (int)(((rows_valid - 1u) * p.lda + p.k) * 2u), kBufferFlags);
    const uint32_t cols_valid = p.n - n0 < (uint32_t)kBN ? p.n - n0 : (uint32_t)kBN;
    // packed weights: the tile's column blocks of 16 are consecutive slabs of slab_bytes each; the buffer ends with the
    // last valid one, so blocks past n read as zero
    const uint32_t slab_bytes = p.k * 16u * BITS / 8u;
    const __amdgpu_buffer_rsrc_t rsrc_b =
        PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (size_t)(n0 / 16u) * slab_bytes), 0,
                                                   (int)((cols_valid / 16u) * slab_bytes), kBufferFlags)
               : __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (BITS == 8 ? n0 : n0 / 2u)), 0,
                                                   (int)((p.k - 1u) * p.ldb_bytes + (BITS == 8 ? cols_valid : cols_valid / 2u)),
                                                   kBufferFlags);

    // A goes global -> LDS directly (buffer_load_dwordx4 ... lds): instruction j of wave w fills the 1 KiB
    // of rows 8*MT*w + 8j .. +7; lane l lands at byte 16*l of it, i.e. row 8*MT*w + 8j + l/8, chunk POSITION l%8,
    // so the lane fetches the chunk that the swizzle puts there: chunk (l%8) ^ ((row >> 1) & 7).
    // (arrays below keep the 256-row tile's extent whatever MT is: with array bounds that depend on MT this compiler's host
    // pass stops emitting the kernel's launch stub; the unused elements cost nothing)
    // The last K-step may be partial (k a multiple of 8, not of 64): there the chunks of 8 k past the end are fetched
    // from beyond the buffer's extent, which reads as zero; B's rows past k read as zero codes — finite weights — and
    // their products with those zeros vanish.
    const uint32_t ksteps = (p.k + (uint32_t)kBK - 1u) / (uint32_t)kBK;
    const uint32_t last_chunks = (p.k - (ksteps - 1u) * (uint32_t)kBK) / 8u;  // valid 16-byte chunks per row in the last step: 1..8
    const uint32_t a_extent = ((rows_valid - 1u) * p.lda + p.k) * 2u;
    uint32_t a_voff[4], a_voff_last[4];
#pragma unroll
    for (uint32_t j = 0; j < MT; ++j) {
        const uint32_t row = 8u * MT * wave + 8u * j + (lane >> 3);
        const uint32_t chunk = (lane & 7u) ^ ((row >> 1) & 7u);
        a_voff[j] = (row * p.lda + chunk * 8u) * 2u;
        a_voff_last[j] = chunk < last_chunks ? a_voff[j] : a_extent;
    }
    // W, row-major: k-group = wave (rows 8*wave..+7 of the step), 4 columns per lane
    const uint32_t b_voff = BITS == 8 ? 4u * lane : 2u * lane;
    const uint32_t w_dst = swizzled_off((lane & 31u) + (lane >> 5) * 64u, wave);  // + (j&1)*4096 + (j>>1)*16384
    // W, packed: wave w converts column blocks 2w and 2w+1 of the tile; lane (nl, kg) holds, per block, column nl, rows
    // 8 kg .. +7 of both K-blocks of the step, and writes them as chunks kg and 4 + kg of the column's LDS row.  Column
    // nl of block cb lives in LDS row (cb>>2)*64 + (cb&1)*32 + ((cb>>1)&1)*16 + nl: the 16 lanes that write one chunk
    // hit 16 consecutive rows (distinct bank groups), and wave wn's accumulator t, MFMA column jl is tile column
    // 16*(4 wn + 2 (jl>>4) + t) + (jl & 15).
    uint32_t pk_voff[2], pk_dst[2];
#pragma unroll
    for (uint32_t i = 0; i < 2; ++i) {
        const uint32_t cb = 2u * wave + i;
        pk_voff[i] = cb * slab_bytes + lane * 16u;
        const uint32_t rho = (cb >> 2) * 64u + (cb & 1u) * 32u + ((cb >> 1) & 1u) * 16u + (lane & 15u);
        pk_dst[i] = swizzled_off(rho, lane >> 4);  // chunk kg; chunk 4 + kg is this address ^ 64
    }
    // fragment reads: row (lane&31) of a 32-row block, chunk 2*kk + lane/32
    uint32_t a_rd[4], w_rd[4];
#pragma unroll
    for (uint32_t kk = 0; kk < 4; ++kk) {
        const uint32_t x = swizzled_off(lane & 31u, 2u * kk + (lane >> 5));
        a_rd[kk] = wm * (MT * 4096u) + x;  // + mt*4096
        w_rd[kk] = wn * 8192u + x;   // + t*4096
    }

    // ---- scales of this lane's 4 columns
    const uint32_t ncol = n0 + 4u * lane;
    const bool w_ok = ncol < p.n;
    // row-major: cs[j] scales column 4*lane + j.  Packed: cs[2 i + h] scales column nl of block 2 wave + i in K-block h.
    float cs[4];
    uint32_t cur_group = 0xffffffffu, cur_group1 = 0xffffffffu;
    auto fetch_scales = [&](uint32_t g, uint32_t g1) {
        if constexpr (PACKED) {
            // g = group of the step's first K-block, g1 of the second one
#pragma unroll
            for (uint32_t i = 0; i < 2; ++i) {
                const uint32_t c = n0 + 16u * (2u * wave + i) + (lane & 15u);
                uint32_t s0 = 0, s1 = 0;
                if (c < p.n) {
                    s0 = p.scale[(size_t)g * p.lds + c];
                    s1 = p.scale[(size_t)g1 * p.lds + c];
                }
                cs[2 * i] = make_col_scale<BITS>(s0);
                cs[2 * i + 1] = make_col_scale<BITS>(s1);
            }
        } else if constexpr (REF) {
            float4 sf = make_float4(0.f, 0.f, 0.f, 0.f);
            if (w_ok) sf = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.scale) + ncol);
            cs[0] = sf.x; cs[1] = sf.y; cs[2] = sf.z; cs[3] = sf.w;
        } else {
            uint2 sr = make_uint2(0, 0);
            if (w_ok) sr = *reinterpret_cast<const uint2*>(p.scale + (size_t)g * p.lds + ncol);
            cs[0] = make_col_scale<BITS>(sr.x & 0xffffu);
            cs[1] = make_col_scale<BITS>(sr.x >> 16);
            cs[2] = make_col_scale<BITS>(sr.y & 0xffffu);
            cs[3] = make_col_scale<BITS>(sr.y >> 16);
        }
    };
    if constexpr (!GROUPED) fetch_scales(0, 0);

    uint32_t b_reg[8];

    // A tile of K-step `kt` -> LDS stage (asynchronous; counted by vmcnt like any other load)
    auto dma_a = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = a_tile(stage_c) + wave * (MT * 1024u);
#pragma unroll
        for (uint32_t j = 0; j < MT; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16,
                                                     kt + 1u == ksteps ? a_voff_last[j] : a_voff[j], kt * (uint32_t)kBK * 2u, 0, 0);
    };
    // raw W codes of K-step `kt` -> registers (kt is clamped by the callers, so every load is in range)
    auto gload = [&](uint32_t kt) {
        if constexpr (PACKED) {
#pragma unroll
            for (uint32_t i = 0; i < 2; ++i) {
                if constexpr (BITS == 8) {  // K-chunk = this step: the lane's 16 bytes
                    const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, pk_voff[i], kt * 1024u, 0);
                    b_reg[4 * i] = v[0]; b_reg[4 * i + 1] = v[1]; b_reg[4 * i + 2] = v[2]; b_reg[4 * i + 3] = v[3];
                } else {  // K-chunk = two steps: the half of the lane's 16 bytes that belongs to this one
                    const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_b, pk_voff[i], (kt >> 1) * 1024u + (kt & 1u) * 8u, 0);
                    b_reg[2 * i] = v[0]; b_reg[2 * i + 1] = v[1];
                }
            }
            return;
        }
        const uint32_t row0 = (kt * (uint32_t)kBK + 8u * wave) * p.ldb_bytes;
#pragma unroll
        for (uint32_t r = 0; r < 8; ++r) {
            if constexpr (BITS == 8) b_reg[r] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_b, b_voff, row0 + r * p.ldb_bytes, 0);
            else b_reg[r] = __builtin_amdgcn_raw_buffer_load_b16(rsrc_b, b_voff, row0 + r * p.ldb_bytes, 0);
        }
    };
    // column J of the raw W registers -> bf16 -> LDS
    auto store_w_col = [&](auto stage_c, auto j_c, const uint32_t (&b_s8)[8]) {
        constexpr int J = decltype(j_c)::value;
        uint4 w;
        if constexpr (PACKED) {
            // J = 2 i + h: column block i of this wave, K-block h of the step
            constexpr int I = J >> 1, H = J & 1;
            const float s = cs[J];
            if constexpr (BITS == 8) {
                const uint32_t lo = b_s8[4 * I + 2 * H], hi = b_s8[4 * I + 2 * H + 1];  // rows 0-3, rows 4-7
                w.x = pack_bf16<REF>(sbyte_to_f32<0>(lo) * s, sbyte_to_f32<1>(lo) * s);
                w.y = pack_bf16<REF>(sbyte_to_f32<2>(lo) * s, sbyte_to_f32<3>(lo) * s);
                w.z = pack_bf16<REF>(sbyte_to_f32<0>(hi) * s, sbyte_to_f32<1>(hi) * s);
                w.w = pack_bf16<REF>(sbyte_to_f32<2>(hi) * s, sbyte_to_f32<3>(hi) * s);
            } else {
                const uint32_t ev = b_s8[2 * J], od = b_s8[2 * J + 1];  // rows 0,2,4,6 and rows 1,3,5,7
                w.x = pack_bf16<REF>(sbyte_to_f32<0>(ev) * s, sbyte_to_f32<0>(od) * s);
                w.y = pack_bf16<REF>(sbyte_to_f32<1>(ev) * s, sbyte_to_f32<1>(od) * s);
                w.z = pack_bf16<REF>(sbyte_to_f32<2>(ev) * s, sbyte_to_f32<2>(od) * s);
                w.w = pack_bf16<REF>(sbyte_to_f32<3>(ev) * s, sbyte_to_f32<3>(od) * s);
            }
            *reinterpret_cast<uint4*>(w_tile(stage_c) + (pk_dst[I] ^ (H * 64u))) = w;
            return;
        }
        w.x = pack_bf16<REF>(sbyte_to_f32<J>(b_s8[0]) * cs[J], sbyte_to_f32<J>(b_s8[1]) * cs[J]);
        w.y = pack_bf16<REF>(sbyte_to_f32<J>(b_s8[2]) * cs[J], sbyte_to_f32<J>(b_s8[3]) * cs[J]);
        w.z = pack_bf16<REF>(sbyte_to_f32<J>(b_s8[4]) * cs[J], sbyte_to_f32<J>(b_s8[5]) * cs[J]);
        w.w = pack_bf16<REF>(sbyte_to_f32<J>(b_s8[6]) * cs[J], sbyte_to_f32<J>(b_s8[7]) * cs[J]);
        *reinterpret_cast<uint4*>(w_tile(stage_c) + w_dst + (J & 1) * 4096u + (J >> 1) * 16384u) = w;
    };
    auto prepare = [&](uint32_t (&b_s8)[8]) {
        if constexpr (PACKED && BITS == 4) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {  // dword d = 2 i + h: 8 nibbles = rows 0..7 of one column
                codes4_to_s8x16(b_reg[d], b_s8[2 * d], b_s8[2 * d + 1]);
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) b_s8[r] = BITS == 8 ? codes8_to_s8(b_reg[r]) : codes4_quad_to_s8x16(b_reg[r]);
    };
    auto update_scales = [&](uint32_t kt) {
        if constexpr (GROUPED) {
            uint32_t g = group_of_row(p, kt * (uint32_t)kBK + (PACKED ? 0u : 8u * wave));
            uint32_t g1 = PACKED ? group_of_row(p, kt * (uint32_t)kBK + 32u) : g;  // packed: a wave converts both K-blocks of the step
            const uint32_t groups = p.k / p.group_size;
            if (g >= groups) g = groups - 1u;  // rows past k in a partial last step: any scale will do, their products vanish
            if (g1 >= groups) g1 = groups - 1u;
            if (g != cur_group || g1 != cur_group1) {
                cur_group = g;
                cur_group1 = g1;
                fetch_scales(g, g1);
            }
        }
    };

    f32x16_t acc[4][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

    auto read_frags = [&](auto stage_c, auto kk_c, bf16x8_t (&af)[4], bf16x8_t (&wf)[2]) {
        constexpr uint32_t KK = decltype(kk_c)::value;
#pragma unroll
        for (uint32_t mt = 0; mt < MT; ++mt) af[mt] = *reinterpret_cast<const bf16x8_t*>(a_tile(stage_c) + a_rd[KK] + mt * 4096u);
#pragma unroll
        for (uint32_t t = 0; t < 2; ++t) wf[t] = *reinterpret_cast<const bf16x8_t*>(w_tile(stage_c) + w_rd[KK] + t * 4096u);
    };
    auto mma = [&](const bf16x8_t (&af)[4], const bf16x8_t (&wf)[2]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int t = 0; t < 2; ++t) acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mt], wf[t], acc[mt][t], 0, 0, 0);
    };

    using C0 = std::integral_constant<uint32_t, 0>;
    using C1 = std::integral_constant<uint32_t, 1>;
    using C2 = std::integral_constant<uint32_t, 2>;
    using C3 = std::integral_constant<uint32_t, 3>;
    using J0 = std::integral_constant<int, 0>;
    using J1 = std::integral_constant<int, 1>;
    using J2 = std::integral_constant<int, 2>;
    using J3 = std::integral_constant<int, 3>;

    // One K-step in four quarters of 8 MFMAs (stage S is current, O = S^1 receives step kt+1, whose
    // raw tile sits in a_reg/b_reg; fragments are double-buffered in f0/f1; on entry f0 holds kk=0):
    //   Q1  MFMA kk=0 (f0)          | LDS reads kk=1 -> f1
    //   Q2  MFMA kk=1 (f1)          | LDS reads kk=2 -> f0; A registers -> LDS(O); raw W -> signed bytes;
    //                                 buffer loads of step kt+2 into the freed registers; W columns 0,1 -> LDS(O)
    //   Q3  MFMA kk=2 (f0)          | LDS reads kk=3 -> f1; W columns 2,3 -> LDS(O)
    //   barrier                       (every wave has filled O)
    //   Q4  MFMA kk=3 (f1)          | LDS reads kk=0 of O -> f0 for the next step
    // The raw tile is loaded a full step before it is used, and the first fragments of the next
    // stage are fetched behind the last 8 MFMAs of this one.
    bf16x8_t af0[4], wf0[2], af1[4], wf1[2];
#ifdef BFAINTB_TRACE
    long long tq[5] = {0, 0, 0, 0, 0};
#define PF_MARK(i) do { const long long now_ = clock64(); tq[i] += now_ - tlast; tlast = now_; } while (0)
    long long tlast = clock64();
#else
#define PF_MARK(i) do { } while (0)
#endif
    auto step = [&](auto stage_c, uint32_t kt) {
        constexpr uint32_t S = decltype(stage_c)::value;
        using Other = std::integral_constant<uint32_t, S ^ 1u>;
        uint32_t b_s8[8];
        // Q1
        __builtin_amdgcn_s_setprio(0);
        dma_a(Other{}, kt + 1 < ksteps ? kt + 1 : kt);
        read_frags(stage_c, C1{}, af1, wf1);
        mma(af0, wf0);
        __builtin_amdgcn_sched_barrier(0);
        PF_MARK(0);
        // Q2
        read_frags(stage_c, C2{}, af0, wf0);
        update_scales(kt + 1 < ksteps ? kt + 1 : kt);
        prepare(b_s8);
        // the raw W tile of step kt+2 goes into the registers just freed: here for 8-bit codes, a quarter later for
        // 4-bit codes, whose conversion makes this quarter the longest (measured: each placement wins for its format)
        if constexpr (BITS == 8) gload(kt + 2 < ksteps ? kt + 2 : ksteps - 1);
        store_w_col(Other{}, J0{}, b_s8);
        store_w_col(Other{}, J1{}, b_s8);
        mma(af1, wf1);
        // interleave: 2 x {MFMA, 4 xor, 3 LDS reads}, the 8 buffer loads, then per W column 3 x {MFMA, 7 VALU} and its write
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
        }
        if constexpr (BITS == 8) __builtin_amdgcn_sched_group_barrier(0x020, PACKED ? 2 : 8, 0);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        PF_MARK(1);
        // Q3
        read_frags(stage_c, C3{}, af1, wf1);
        if constexpr (BITS == 4) gload(kt + 2 < ksteps ? kt + 2 : ksteps - 1);
        store_w_col(Other{}, J2{}, b_s8);
        store_w_col(Other{}, J3{}, b_s8);
        mma(af0, wf0);
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
        if constexpr (BITS == 4) __builtin_amdgcn_sched_group_barrier(0x020, PACKED ? 2 : 8, 0);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        PF_MARK(2);
        // From here to the end of the step this wave outranks its SIMD neighbour: past the barrier it holds the
        // fragments of the next stage's first quarter and should start on them at once, ahead of a neighbour
        // still converting weights (measured: 5-6 % at M = 4096 and 8192; raising other quarters gains less).
        __builtin_amdgcn_s_setprio(1);
        // this wave's part of the next A tile has landed in LDS (the 8 W loads issued after it may still fly)
        if constexpr (PACKED) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        __syncthreads();
        PF_MARK(3);
        // Q4
        read_frags(Other{}, C0{}, af0, wf0);
        mma(af1, wf1);
        PF_MARK(4);
    };

    // ---- prologue: tile 0 -> stage 0, raw W of tile 1 -> registers
    dma_a(C0{}, 0);
    gload(0);
    {
        uint32_t b_s8[8];
        update_scales(0);
        prepare(b_s8);
        store_w_col(C0{}, J0{}, b_s8);
        store_w_col(C0{}, J1{}, b_s8);
        store_w_col(C0{}, J2{}, b_s8);
        store_w_col(C0{}, J3{}, b_s8);
    }
    gload(ksteps > 1 ? 1 : 0);
    if constexpr (PACKED) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __syncthreads();
    read_frags(C0{}, C0{}, af0, wf0);

    uint32_t kt = 0;
    for (; kt + 1 < ksteps; kt += 2) {
        step(C0{}, kt);
        step(C1{}, kt + 1);
    }
    if (kt < ksteps) step(C0{}, kt);

#ifdef BFAINTB_TRACE
    if (lane == 0 && p.trace != nullptr)
        for (int i = 0; i < 5; ++i) p.trace[(size_t)(blockIdx.x * 8 + wave) * 8 + i] = (unsigned long long)tq[i];
#endif
    __builtin_amdgcn_s_setprio(0);
    // ---- epilogue: bf16 tile through LDS (rows 64q..64q+63 in the q-th of the four arrays), then
    //      16-byte row-contiguous stores
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing asynchronous may still be writing LDS
    __syncthreads();
    auto c_rows = [&](uint32_t q) -> uint8_t* { return q == 0 ? lds_a0 : q == 1 ? lds_a1 : q == 2 ? lds_w0 : lds_w1; };
    // gated: columns (2j, 2j+1) of the sums are (gate, up) of output column j; the staged tile is then 128 columns wide
    const bool gated = p.activation == kActSiluGate;
    if constexpr (PACKED) {
        // accumulator t of this wave, MFMA column jl is tile column 16 * (4 wn + 2 (jl >> 4) + t) + (jl & 15): the two
        // accumulators are 16 columns apart, so each value is staged on its own
        const uint32_t jl = lane & 31u, half = lane >> 5;
        const uint32_t col0 = 16u * (4u * wn + 2u * (jl >> 4)) + (jl & 15u);
        float bias0 = 0.f, bias1 = 0.f;
        const bool has_bias = p.bias != nullptr, has_res = p.residual != nullptr;
        if (has_bias) {
            if (n0 + col0 < p.n) bias0 = bf16_bits_to_f32(p.bias[n0 + col0]);
            if (n0 + col0 + 16u < p.n) bias1 = bf16_bits_to_f32(p.bias[n0 + col0 + 16u]);
        }
        if (gated) {
            // neighbouring columns (gate, up) sit in neighbouring lanes: even lanes fetch the partner's sums with a DPP swap and
            // produce output columns (n0 + col0) / 2 and (n0 + col0 + 16) / 2
            const bool is_gate = (lane & 1u) == 0u;
#pragma unroll
            for (uint32_t mt = 0; mt < MT; ++mt) {
                const uint32_t block32 = wm * MT + mt;
                uint8_t* base = c_rows(block32 >> 1);
                uint32_t rres[16];
                if (has_res && is_gate) {
#pragma unroll
                    for (uint32_t i = 0; i < 16; ++i) {
                        const uint32_t gm = m0 + 32u * block32 + 8u * (i >> 2) + 4u * half + (i & 3u);
                        uint32_t lo = 0, hi = 0;
                        if (gm < p.m) {
                            if (n0 + col0 < p.n) lo = p.residual[(size_t)gm * p.ldr + (n0 + col0) / 2u];
                            if (n0 + col0 + 16u < p.n) hi = p.residual[(size_t)gm * p.ldr + (n0 + col0 + 16u) / 2u];
                        }
                        rres[i] = lo | (hi << 16);
                    }
                }
#pragma unroll
                for (uint32_t i = 0; i < 16; ++i) {
                    const uint32_t row = 32u * (block32 & 1u) + 8u * (i >> 2) + 4u * half + (i & 3u);
                    const float x0 = acc[mt][0][i] + bias0, x1 = acc[mt][1][i] + bias1;
                    const float y0 = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x0), 0xB1, 0xF, 0xF, true));
                    const float y1 = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x1), 0xB1, 0xF, 0xF, true));
                    if (is_gate) {
                        float o0 = silu_gate(x0, y0), o1 = silu_gate(x1, y1);
                        if (has_res) {
                            o0 += bf16_bits_to_f32(rres[i] & 0xffffu);
                            o1 += bf16_bits_to_f32(rres[i] >> 16);
                        }
                        const uint32_t both = pack_bf16<REF>(o0, o1);
                        *reinterpret_cast<uint16_t*>(base + row * kCRowBytes + col0) = (uint16_t)(both & 0xffffu);
                        *reinterpret_cast<uint16_t*>(base + row * kCRowBytes + col0 + 16u) = (uint16_t)(both >> 16);
                    }
                }
            }
        } else
        // the residual of this lane's outputs (two columns each) is fetched for two 32-row blocks at a time, before the first
        // value is used: the epilogue has the registers the main loop's fragments have freed, and pays two memory
        // latencies instead of one per block
#pragma unroll
        for (uint32_t mt0 = 0; mt0 < MT; mt0 += 2) {
            uint32_t rres[2][16];
            if (has_res) {
#pragma unroll
                for (uint32_t mt = mt0; mt < mt0 + 2; ++mt)
#pragma unroll
                    for (uint32_t i = 0; i < 16; ++i) {
                        const uint32_t gm = m0 + 32u * (wm * MT + mt) + 8u * (i >> 2) + 4u * half + (i & 3u);
                        uint32_t lo = 0, hi = 0;
                        if (gm < p.m) {
                            if (n0 + col0 < p.n) lo = p.residual[(size_t)gm * p.ldr + n0 + col0];
                            if (n0 + col0 + 16u < p.n) hi = p.residual[(size_t)gm * p.ldr + n0 + col0 + 16u];
                        }
                        rres[mt - mt0][i] = lo | (hi << 16);
                    }
            }
#pragma unroll
            for (uint32_t mt = mt0; mt < mt0 + 2; ++mt) {
                const uint32_t block32 = wm * MT + mt;
                uint8_t* base = c_rows(block32 >> 1);
#pragma unroll
                for (uint32_t i = 0; i < 16; ++i) {
                    const uint32_t row = 32u * (block32 & 1u) + 8u * (i >> 2) + 4u * half + (i & 3u);
                    uint32_t both;
                    if (has_res) {  // bias0/1 are +0 without a bias: a sum that gets a residual added need not keep -0
                        both = pack_bf16<REF>(acc[mt][0][i] + bias0 + bf16_bits_to_f32(rres[mt - mt0][i] & 0xffffu),
                                             acc[mt][1][i] + bias1 + bf16_bits_to_f32(rres[mt - mt0][i] >> 16));
                    } else {
                        both = has_bias ? pack_bf16<REF>(acc[mt][0][i] + bias0, acc[mt][1][i] + bias1) : pack_bf16<REF>(acc[mt][0][i], acc[mt][1][i]);
                    }
                    *reinterpret_cast<uint16_t*>(base + row * kCRowBytes + 2u * col0) = (uint16_t)(both & 0xffffu);
                    *reinterpret_cast<uint16_t*>(base + row * kCRowBytes + 2u * col0 + 32u) = (uint16_t)(both >> 16);
                }
            }
        }
    } else
    {
        const uint32_t jl = lane & 31u, half = lane >> 5;
        const uint32_t colbyte = 8u * (32u * (wn & 1u) + jl) + 4u * (wn >> 1);
        // this lane's two columns of the tile are colbyte/2 and the next: their bias, if the launch has one
        float bias0 = 0.f, bias1 = 0.f;
        const bool has_bias = p.bias != nullptr, has_res = p.residual != nullptr;
        if (has_bias && n0 + colbyte / 2u < p.n) {
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.bias + n0 + colbyte / 2u);
            bias0 = bf16_bits_to_f32(raw & 0xffffu);
            bias1 = bf16_bits_to_f32(raw >> 16);
        }
        if (gated) {
            // the lane's two neighbouring columns are (gate, up) of tile output column colbyte / 4
#pragma unroll
            for (uint32_t mt = 0; mt < MT; ++mt) {
                const uint32_t block32 = wm * MT + mt;
                uint8_t* base = c_rows(block32 >> 1);
                uint32_t rres[16];
                if (has_res) {
#pragma unroll
                    for (uint32_t i = 0; i < 16; ++i) {
                        const uint32_t gm = m0 + 32u * block32 + 8u * (i >> 2) + 4u * half + (i & 3u);
                        rres[i] = (gm < p.m && n0 + colbyte / 2u < p.n) ? p.residual[(size_t)gm * p.ldr + (n0 + colbyte / 2u) / 2u] : 0u;
                    }
                }
#pragma unroll
                for (uint32_t i = 0; i < 16; ++i) {
                    const uint32_t row = 32u * (block32 & 1u) + 8u * (i >> 2) + 4u * half + (i & 3u);
                    float o = silu_gate(acc[mt][0][i] + bias0, acc[mt][1][i] + bias1);
                    if (has_res) o += bf16_bits_to_f32(rres[i]);
                    *reinterpret_cast<uint16_t*>(base + row * kCRowBytes + colbyte / 2u) = (uint16_t)(pack_bf16<REF>(o, 0.f) & 0xffffu);
                }
            }
        } else {
        // the residual of this lane's 32 x MT outputs (two neighbouring columns each), fetched in one go before the first
        // is used (see the packed branch)
        uint32_t rres[4][16];
        if (has_res) {
#pragma unroll
            for (uint32_t mt = 0; mt < MT; ++mt)
#pragma unroll
                for (uint32_t i = 0; i < 16; ++i) {
                    const uint32_t gm = m0 + 32u * (wm * MT + mt) + 8u * (i >> 2) + 4u * half + (i & 3u);
                    rres[mt][i] = (gm < p.m && n0 + colbyte / 2u < p.n)
                                      ? *reinterpret_cast<const uint32_t*>(p.residual + (size_t)gm * p.ldr + n0 + colbyte / 2u) : 0u;
                }
        }
#pragma unroll
        for (uint32_t mt = 0; mt < MT; ++mt) {
            const uint32_t block32 = wm * MT + mt;  // which 32 rows of the tile
            uint8_t* base = c_rows(block32 >> 1);
#pragma unroll
            for (uint32_t i = 0; i < 16; ++i) {
                const uint32_t row = 32u * (block32 & 1u) + 8u * (i >> 2) + 4u * half + (i & 3u);
                // without a bias or residual the sums are stored as they are (adding +0 would turn a -0 sum into +0)
                uint32_t both;
                if (has_res) {
                    both = pack_bf16<REF>(acc[mt][0][i] + bias0 + bf16_bits_to_f32(rres[mt][i] & 0xffffu),
                                         acc[mt][1][i] + bias1 + bf16_bits_to_f32(rres[mt][i] >> 16));
                } else {
                    both = has_bias ? pack_bf16<REF>(acc[mt][0][i] + bias0, acc[mt][1][i] + bias1) : pack_bf16<REF>(acc[mt][0][i], acc[mt][1][i]);
                }
                *reinterpret_cast<uint32_t*>(base + row * kCRowBytes + colbyte) = both;
            }
        }
        }
    }
    __syncthreads();
#pragma unroll
    for (uint32_t pass = 0; pass < 4u * MT; ++pass) {
        const uint32_t row = pass * 16u + (tid >> 5);
        const uint32_t ch = tid & 31u;
        const uint32_t gm = m0 + row;
        const uint32_t gn = gated ? n0 / 2u + ch * 8u : n0 + ch * 8u;  // gated rows hold 128 outputs: chunks 0..15
        if (gm < p.m && (gated ? (ch < 16u && gn < p.n / 2u) : gn < p.n)) {
            const uint4 v = *reinterpret_cast<const uint4*>(c_rows(pass >> 2) + (row & 63u) * kCRowBytes + ch * 16u);
            *reinterpret_cast<uint4*>(p.c + (size_t)gm * p.ldc + gn) = v;
        }
    }
}

bool prefill_wreg_serves(const GemmParams& p);
hipError_t launch_prefill_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream);
hipError_t launch_prefill256x128_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream);

template <int BITS, bool GROUPED, bool PACKED, bool REF = false>
static hipError_t launch_prefill_t(const GemmParams& p0, hipStream_t stream, bool wreg = false)
{
    GemmParams p = p0;
    const uint32_t tiles = ((p.m + kBM - 1) / kBM) * ((p.n + kBN - 1) / kBN);
    // whole rounds of one workgroup per CU run 256x256 tiles; a last round that would fill at most half of the
    // CUs runs as twice as many half tiles instead (also when there is no whole round at all)
#ifdef BFAINTB_TRACE
    const uint32_t halves = 0u;  // instrumented builds time the whole-tile kernel at every tile count
#else
    const uint32_t halves = thin_round_tiles(tiles, p.m, p.cus ? p.cus : 256u);
#endif
    const uint32_t whole = tiles - halves;
    if (whole) {
        p.tile_first = 0;
        p.tile_count = whole;
        const uint32_t grid = (whole + 7u) / 8u * 8u;  // a whole number of workgroups per XCD; ids past the last tile exit at once
        void (*whole_tiles)(const GemmParams) = bfaintb_prefill_kernel<BITS, GROUPED, 4, PACKED, REF>;
        // whole tiles: the form that keeps the weights in registers, where it serves the launch
        hipError_t e = (wreg && !REF && prefill_wreg_serves(p)) ? launch_prefill_wreg(p, BITS, PACKED, stream)
                                                                           : launch_kernel(whole_tiles, dim3(grid, 1, 1), dim3(512, 1, 1), 0, stream, p);
        if (e != hipSuccess) return e;
    }
    if (halves) {
        p.tile_first = whole;
        p.tile_count = halves;
        // ... as left and right halves on the kernel of 256x128 tiles that keeps the weights in registers, where that serves
        if (wreg && !REF && prefill_wreg_serves(p)) {
            p.splits = 1;
            return launch_prefill256x128_wreg(p, BITS, PACKED, stream);
        }
        const uint32_t grid = (2u * halves + 7u) / 8u * 8u;
        void (*half_tiles)(const GemmParams) = bfaintb_prefill_kernel<BITS, GROUPED, 2, PACKED, REF>;
        return launch_kernel(half_tiles, dim3(grid, 1, 1), dim3(512, 1, 1), 0, stream, p);
    }
    return hipSuccess;
}

hipError_t launch_prefill(const GemmParams& p, int bits, hipStream_t stream, bool wreg)
{
    const bool grouped = p.group_size != 0;
    if (p.reference_arith) return (bits == 8 && !grouped) ? launch_prefill_t<8, false, false, true>(p, stream) : hipErrorInvalidValue;
    if (bits == 8) return grouped ? launch_prefill_t<8, true, false>(p, stream, wreg) : launch_prefill_t<8, false, false>(p, stream, wreg);
    return grouped ? launch_prefill_t<4, true, false>(p, stream, wreg) : launch_prefill_t<4, false, false>(p, stream, wreg);
}

// The same kernel over weights in the packed order (p.b is the packed buffer; p.ldb_bytes is unused).
hipError_t launch_prefill_packed(const GemmParams& p, int bits, hipStream_t stream, bool wreg)
{
    const bool grouped = p.group_size != 0;
    if (bits == 8) return grouped ? launch_prefill_t<8, true, true>(p, stream, wreg) : launch_prefill_t<8, false, true>(p, stream, wreg);
    return grouped ? launch_prefill_t<4, true, true>(p, stream, wreg) : launch_prefill_t<4, false, true>(p, stream, wreg);
}

}  // namespace bfaintb
