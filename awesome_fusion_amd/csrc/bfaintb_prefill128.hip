// Tiled variant with 128x128 tiles, for shapes whose 256x256 tiles would leave most of the machine idle
// (a few hundred to a few thousand rows of A against n of a few thousand).
//
// Same job and the same reference kernel replaced as bfaintb_prefill_kernel
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630).  A quarter of that kernel's tile: four times the
// workgroups for the same C, each with a quarter of the matrix instructions, half of the weight conversion and half
// of the LDS traffic per K-step; 64 KiB of LDS and at most 128 registers, so two workgroups share a CU and hide each
// other's waits.  Per flop it converts and moves twice as much as the large tile, so it only pays where the large
// tile cannot fill the CUs.
//
// Shape of the computation
//   512 threads = 8 waves, 2 along m x 4 along n; a wave owns 64 rows x 32 columns = 2 accumulators of
//   v_mfma_f32_32x32x16_bf16.  K advances 64 per step.  LDS: two stages of {A tile, converted W tile}, each 128 rows
//   x 64 k of bf16 = 16 KiB, rows of 128 bytes in 8 chunks of 16, chunk c of row r at position c ^ ((r >> 1) & 7)
//   (as in the large kernel).  A goes global -> LDS directly.
//   W, row-major B: wave w loads rows 8w .. 8w+7 of the step, two codes per lane and row (columns 2*lane, 2*lane+1),
//     converts them and writes one 16-byte chunk per column; column 2*lane + j lives in LDS row 64 j + lane
//     (consecutive lanes write consecutive rows), so wave wn's MFMA column jl is tile column
//     2 * (32 (wn & 1) + jl) + (wn >> 1).
//   W, packed order: wave w converts column block w of the tile's eight: lane (nl, kg) holds column nl, rows 8 kg ..
//     +7 of both K-blocks of the step (16 bytes for 8-bit codes, 8 for 4-bit) and writes chunks kg and 4 + kg of LDS
//     row 16 w + nl; wave wn's MFMA column jl is tile column 32 wn + jl.
//   Per step a wave fetches the fragments of all four K-blocks at once, starts the next A tile's copy, converts its
//   share of the next W tile into the other stage, issues the loads of the codes after those, runs its 8 MFMAs back
//   to back and meets the others at one barrier.  (Tried and slower: A and W through registers two steps ahead,
//   57 instead of 47 us at m = 256, n = k = 4096.)
// Epilogue: the fp32 sums are staged in LDS in true [m][n] order (128 x 128 x 4 bytes = the four tile arrays); then
//   each thread finishes 8 neighbouring columns of a row — bias, SiLU gate, residual, the one rounding — and stores
//   them with one 16-byte (gated: 8-byte) write.
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

namespace {
constexpr uint32_t kT128 = 128;                 // tile edge
constexpr uint32_t kStage128 = 128 * 128;       // bytes of one A or W stage

__device__ __forceinline__ uint32_t swz128(uint32_t row, uint32_t chunk)
{
    return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4);
}
}  // namespace

// REF: the reference kernel's arithmetic (p.reference_arith): one fp32 scale per column, W and C narrowed by truncation.
template <int BITS, bool GROUPED, bool PACKED, bool REF>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
bfaintb_prefill128_kernel(const GemmParams p)
{
    static_assert(!REF || (BITS == 8 && !GROUPED && !PACKED), "the reference's arithmetic: 8-bit codes, row-major, one scale per column");
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a0[kStage128];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a1[kStage128];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w0[kStage128];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w1[kStage128];
    auto a_tile = [&](auto stage_c) -> uint8_t* { return decltype(stage_c)::value == 0 ? lds_a0 : lds_a1; };
    auto w_tile = [&](auto stage_c) -> uint8_t* { return decltype(stage_c)::value == 0 ? lds_w0 : lds_w1; };

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 2, wn = wave & 3u;

    // ---- tile of this workgroup: the ids an XCD receives (id mod 8) cover consecutive logical ids, which walk groups
    //      of 8 tile-rows column by column (each XCD's L2 then serves a compact block of tiles)
    const uint32_t tiles_m = (p.m + kT128 - 1) / kT128, tiles_n = (p.n + kT128 - 1) / kT128;
    const uint32_t wgs = tiles_m * tiles_n;
    const uint32_t per_xcd = (wgs + 7u) / 8u;
    const uint32_t logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (logical >= wgs) return;
    const uint32_t group = logical / (8u * tiles_n);
    const uint32_t first_m = group * 8u;
    const uint32_t group_rows = tiles_m - first_m < 8u ? tiles_m - first_m : 8u;
    const uint32_t in_group = logical - group * 8u * tiles_n;
    const uint32_t tm = first_m + in_group % group_rows;
    const uint32_t tn = in_group / group_rows;
    const uint32_t m0 = tm * kT128, n0 = tn * kT128;

    const uint32_t rows_valid = p.m - m0 < kT128 ? p.m - m0 : kT128;
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.a + (size_t)m0 * p.lda), 0, (int)(((rows_valid - 1u) * p.lda + p.k) * 2u), kBufferFlags);
    const uint32_t cols_valid = p.n - n0 < kT128 ? p.n - n0 : kT128;
    const uint32_t slab_bytes = p.k * 16u * BITS / 8u;
    const __amdgpu_buffer_rsrc_t rsrc_b =
        PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (size_t)(n0 / 16u) * slab_bytes), 0,
                                                   (int)((cols_valid / 16u) * slab_bytes), kBufferFlags)
               : __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (BITS == 8 ? n0 : n0 / 2u)), 0,
                                                   (int)((p.k - 1u) * p.ldb_bytes + (BITS == 8 ? cols_valid : cols_valid / 2u)),
                                                   kBufferFlags);

    // A: instruction j of wave w fills rows 16w + 8j .. +7; lane l fetches the chunk the swizzle places at its position
    // (a partial last K-step — k a multiple of 8, not of 64 — fetches its chunks past the end of k from beyond the
    // buffer's extent, which reads as zero; B's rows past k read as zero codes, finite weights, and the products vanish)
    const uint32_t ksteps = (p.k + 63u) / 64u;
    const uint32_t last_chunks = (p.k - (ksteps - 1u) * 64u) / 8u;
    const uint32_t a_extent = ((rows_valid - 1u) * p.lda + p.k) * 2u;
    uint32_t a_voff[2], a_voff_last[2];
#pragma unroll
    for (uint32_t j = 0; j < 2; ++j) {
        const uint32_t row = 16u * wave + 8u * j + (lane >> 3);
        const uint32_t chunk = (lane & 7u) ^ ((row >> 1) & 7u);
        a_voff[j] = (row * p.lda + chunk * 8u) * 2u;
        a_voff_last[j] = chunk < last_chunks ? a_voff[j] : a_extent;
    }
    // W addressing (see the header)
    const uint32_t b_voff = PACKED ? wave * slab_bytes + lane * 16u : (BITS == 8 ? 2u * lane : lane);
    // LDS destination of this lane's first chunk: row-major column 2*lane (+ 8192 bytes = 64 rows for column 2*lane+1),
    // chunk = wave; packed column nl of block `wave`, chunk kg (chunk 4 + kg is this address ^ 64)
    const uint32_t w_dst = PACKED ? swz128(16u * wave + (lane & 15u), lane >> 4) : swz128(lane, wave);
    // fragment reads: row (lane & 31) of a 32-row block, chunk 2 kk + lane / 32
    uint32_t a_rd[4], w_rd[4];
#pragma unroll
    for (uint32_t kk = 0; kk < 4; ++kk) {
        const uint32_t x = swz128(lane & 31u, 2u * kk + (lane >> 5));
        a_rd[kk] = wm * 8192u + x;   // + mt * 4096
        w_rd[kk] = wn * 4096u + x;
    }

    // ---- scales.  Row-major: cs[j] scales column 2*lane + j.  Packed: cs[h] scales column nl of block `wave` in
    //      K-block h of the step (they differ only for groups of 32 rows).
    const uint32_t ncol = n0 + (PACKED ? 16u * wave + (lane & 15u) : 2u * lane);
    const bool w_ok = ncol < p.n;
    float cs[2];
    uint32_t cur_group = 0xffffffffu, cur_group1 = 0xffffffffu;
    auto fetch_scales = [&](uint32_t g, uint32_t g1) {
        if constexpr (REF) {
            float2 sf = make_float2(0.f, 0.f);
            if (w_ok) sf = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(p.scale) + ncol);
            cs[0] = sf.x;
            cs[1] = sf.y;
            return;
        }
        uint32_t s0 = 0, s1 = 0;
        if (w_ok) {
            if constexpr (PACKED) {
                s0 = p.scale[(size_t)g * p.lds + ncol];
                s1 = p.scale[(size_t)g1 * p.lds + ncol];  // the step's second K-block may lie in the next group
            } else {
                const uint32_t sr = *reinterpret_cast<const uint32_t*>(p.scale + (size_t)g * p.lds + ncol);
                s0 = sr & 0xffffu;
                s1 = sr >> 16;
            }
        }
        cs[0] = make_col_scale<BITS>(s0);
        cs[1] = make_col_scale<BITS>(s1);
    };
    if constexpr (!GROUPED) fetch_scales(0, 0);
    auto update_scales = [&](uint32_t kt) {
        if constexpr (GROUPED) {
            uint32_t g = group_of_row(p, kt * 64u + (PACKED ? 0u : 8u * wave));
            uint32_t g1 = PACKED ? group_of_row(p, kt * 64u + 32u) : g;  // packed: a wave converts both K-blocks of the step
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

    uint32_t b_reg[8];  // row-major: one (16-bit or 8-bit) load per row; packed: 4 (8-bit codes) or 2 dwords

    auto dma_a = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = a_tile(stage_c) + wave * 2048u;
#pragma unroll
        for (uint32_t j = 0; j < 2; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16,
                                                     kt + 1u == ksteps ? a_voff_last[j] : a_voff[j], kt * 128u, 0, 0);
    };
    auto gload = [&](uint32_t kt) {
        if constexpr (PACKED) {
            if constexpr (BITS == 8) {
                const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, b_voff, kt * 1024u, 0);
                b_reg[0] = v[0]; b_reg[1] = v[1]; b_reg[2] = v[2]; b_reg[3] = v[3];
            } else {
                const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(rsrc_b, b_voff, (kt >> 1) * 1024u + (kt & 1u) * 8u, 0);
                b_reg[0] = v[0]; b_reg[1] = v[1];
            }
        } else {
            const uint32_t row0 = (kt * 64u + 8u * wave) * p.ldb_bytes;
#pragma unroll
            for (uint32_t r = 0; r < 8; ++r) {
                if constexpr (BITS == 8) b_reg[r] = __builtin_amdgcn_raw_buffer_load_b16(rsrc_b, b_voff, row0 + r * p.ldb_bytes, 0);
                else b_reg[r] = __builtin_amdgcn_raw_buffer_load_b8(rsrc_b, b_voff, row0 + r * p.ldb_bytes, 0);
            }
        }
    };
    // the raw codes in b_reg -> two chunks of 8 bf16 -> LDS stage
    auto convert_store = [&](auto stage_c) {
        uint4 w[2];
        if constexpr (PACKED) {
            // chunk h = K-block h of column nl: rows 0-3 and 4-7 in two dwords (8-bit), 8 nibbles in one (4-bit)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float s = cs[h];
                if constexpr (BITS == 8) {
                    const uint32_t lo = codes8_to_s8(b_reg[2 * h]), hi = codes8_to_s8(b_reg[2 * h + 1]);
                    w[h].x = pack_bf16<REF>(sbyte_to_f32<0>(lo) * s, sbyte_to_f32<1>(lo) * s);
                    w[h].y = pack_bf16<REF>(sbyte_to_f32<2>(lo) * s, sbyte_to_f32<3>(lo) * s);
                    w[h].z = pack_bf16<REF>(sbyte_to_f32<0>(hi) * s, sbyte_to_f32<1>(hi) * s);
                    w[h].w = pack_bf16<REF>(sbyte_to_f32<2>(hi) * s, sbyte_to_f32<3>(hi) * s);
                } else {
                    uint32_t ev, od;
                    codes4_to_s8x16(b_reg[h], ev, od);
                    w[h].x = pack_bf16<REF>(sbyte_to_f32<0>(ev) * s, sbyte_to_f32<0>(od) * s);
                    w[h].y = pack_bf16<REF>(sbyte_to_f32<1>(ev) * s, sbyte_to_f32<1>(od) * s);
                    w[h].z = pack_bf16<REF>(sbyte_to_f32<2>(ev) * s, sbyte_to_f32<2>(od) * s);
                    w[h].w = pack_bf16<REF>(sbyte_to_f32<3>(ev) * s, sbyte_to_f32<3>(od) * s);
                }
            }
            *reinterpret_cast<uint4*>(w_tile(stage_c) + w_dst) = w[0];
            *reinterpret_cast<uint4*>(w_tile(stage_c) + (w_dst ^ 64u)) = w[1];
        } else {
            // chunk j = column 2*lane + j, the step's rows 8 wave .. +7: byte j of each row's load
            uint32_t s8[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) s8[r] = BITS == 8 ? codes8_to_s8(b_reg[r]) : codes4_quad_to_s8x16(b_reg[r]);
            w[0].x = pack_bf16<REF>(sbyte_to_f32<0>(s8[0]) * cs[0], sbyte_to_f32<0>(s8[1]) * cs[0]);
            w[0].y = pack_bf16<REF>(sbyte_to_f32<0>(s8[2]) * cs[0], sbyte_to_f32<0>(s8[3]) * cs[0]);
            w[0].z = pack_bf16<REF>(sbyte_to_f32<0>(s8[4]) * cs[0], sbyte_to_f32<0>(s8[5]) * cs[0]);
            w[0].w = pack_bf16<REF>(sbyte_to_f32<0>(s8[6]) * cs[0], sbyte_to_f32<0>(s8[7]) * cs[0]);
            w[1].x = pack_bf16<REF>(sbyte_to_f32<1>(s8[0]) * cs[1], sbyte_to_f32<1>(s8[1]) * cs[1]);
            w[1].y = pack_bf16<REF>(sbyte_to_f32<1>(s8[2]) * cs[1], sbyte_to_f32<1>(s8[3]) * cs[1]);
            w[1].z = pack_bf16<REF>(sbyte_to_f32<1>(s8[4]) * cs[1], sbyte_to_f32<1>(s8[5]) * cs[1]);
            w[1].w = pack_bf16<REF>(sbyte_to_f32<1>(s8[6]) * cs[1], sbyte_to_f32<1>(s8[7]) * cs[1]);
            *reinterpret_cast<uint4*>(w_tile(stage_c) + w_dst) = w[0];
            *reinterpret_cast<uint4*>(w_tile(stage_c) + w_dst + 8192u) = w[1];
        }
    };

    f32x16_t acc[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][i] = 0.f;

    using C0 = std::integral_constant<uint32_t, 0>;
    using C1 = std::integral_constant<uint32_t, 1>;

    // One K-step: the fragments of all four K-blocks of the current stage are fetched at once, right behind the barrier
    // that completed it (12 LDS reads in flight: with only two matrix instructions per fragment pair, fetching one K-block
    // ahead left every pair waiting for its reads); behind them the wave starts the next tile on its way — the
    // asynchronous A copy, conversion of the raw W codes it holds into the other stage, the loads of the codes after
    // those — and then runs its eight matrix instructions back to back.
    auto step = [&](auto stage_c, uint32_t kt) {
        constexpr uint32_t S = decltype(stage_c)::value;
        using Other = std::integral_constant<uint32_t, S ^ 1u>;
        auto clamp = [&](uint32_t t) { return t < ksteps ? t : ksteps - 1u; };
        bf16x8_t af[4][2], wf[4];
#pragma unroll
        for (uint32_t kk = 0; kk < 4; ++kk) {
#pragma unroll
            for (uint32_t mt = 0; mt < 2; ++mt) af[kk][mt] = *reinterpret_cast<const bf16x8_t*>(a_tile(stage_c) + a_rd[kk] + mt * 4096u);
            wf[kk] = *reinterpret_cast<const bf16x8_t*>(w_tile(stage_c) + w_rd[kk]);
        }
        dma_a(Other{}, clamp(kt + 1));
        update_scales(clamp(kt + 1));
        convert_store(Other{});
        gload(clamp(kt + 2));
#pragma unroll
        for (uint32_t kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk][mt], wf[kk], acc[mt], 0, 0, 0);
        // this wave's part of the next A tile has landed in LDS (the W loads issued after it may still fly)
        if constexpr (PACKED) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        __syncthreads();
    };

    // ---- prologue: tile 0 -> stage 0, raw codes of tile 1 -> registers
    dma_a(C0{}, 0);
    gload(0);
    update_scales(0);
    convert_store(C0{});
    gload(ksteps > 1 ? 1 : 0);
    if constexpr (PACKED) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __syncthreads();

    uint32_t kt = 0;
    for (; kt + 1 < ksteps; kt += 2) {
        step(C0{}, kt);
        step(C1{}, kt + 1);
    }
    if (kt < ksteps) step(C0{}, kt);

    // ---- epilogue: fp32 sums -> LDS in [m][n] order (rows 32q .. 32q+31 in the q-th array), then finish row-wise
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing asynchronous may still be writing LDS
    auto c_rows = [&](uint32_t q) -> float* {
        return reinterpret_cast<float*>(q == 0 ? lds_a0 : q == 1 ? lds_a1 : q == 2 ? lds_w0 : lds_w1);
    };
    {
        const uint32_t jl = lane & 31u, half = lane >> 5;
        const uint32_t col = PACKED ? 32u * wn + jl : 2u * (32u * (wn & 1u) + jl) + (wn >> 1);
#pragma unroll
        for (uint32_t mt = 0; mt < 2; ++mt) {
            float* base = c_rows(2u * wm + mt);  // the 32-row block of this accumulator
#pragma unroll
            for (uint32_t i = 0; i < 16; ++i) base[(8u * (i >> 2) + 4u * half + (i & 3u)) * kT128 + col] = acc[mt][i];
        }
    }
    __syncthreads();
    const bool gated = p.activation == kActSiluGate;
    const uint32_t ch = tid & 15u;                 // 8 columns: 8 ch .. 8 ch + 7 of the tile
    const uint32_t gn = n0 + 8u * ch;
    float bias[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) bias[i] = 0.f;
    if (p.bias != nullptr && gn < p.n) {
        const uint4 raw = *reinterpret_cast<const uint4*>(p.bias + gn);
        const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            bias[2 * i] = bf16_bits_to_f32(d[i] & 0xffffu);
            bias[2 * i + 1] = bf16_bits_to_f32(d[i] >> 16);
        }
    }
    const bool plain = p.bias == nullptr && p.residual == nullptr && !gated;  // the bare sums keep a -0 as it is
#pragma unroll
    for (uint32_t pass = 0; pass < 4; ++pass) {
        const uint32_t row = 32u * pass + (tid >> 4);
        const uint32_t gm = m0 + row;
        if (gm >= p.m || gn >= p.n) continue;
        const float* src = c_rows(pass) + (row & 31u) * kT128 + 8u * ch;
        const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
        float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        if (!plain) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] += bias[i];
        }
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
            *reinterpret_cast<uint2*>(p.c + (size_t)gm * p.ldc + gn / 2u) = make_uint2(pack_bf16<REF>(o[0], o[1]), pack_bf16<REF>(o[2], o[3]));
        } else {
            if (p.residual != nullptr) {
                const uint4 r = *reinterpret_cast<const uint4*>(p.residual + (size_t)gm * p.ldr + gn);
                const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    v[2 * i] += bf16_bits_to_f32(d[i] & 0xffffu);
                    v[2 * i + 1] += bf16_bits_to_f32(d[i] >> 16);
                }
            }
            *reinterpret_cast<uint4*>(p.c + (size_t)gm * p.ldc + gn) =
                make_uint4(pack_bf16<REF>(v[0], v[1]), pack_bf16<REF>(v[2], v[3]), pack_bf16<REF>(v[4], v[5]), pack_bf16<REF>(v[6], v[7]));
        }
    }
}

template <int BITS, bool GROUPED, bool PACKED, bool REF = false>
static hipError_t launch_prefill128_t(const GemmParams& p, hipStream_t stream)
{
    const uint32_t tiles = ((p.m + kT128 - 1) / kT128) * ((p.n + kT128 - 1) / kT128);
    const uint32_t grid = (tiles + 7u) / 8u * 8u;  // a whole number of workgroups per XCD; ids past the last tile exit at once
    void (*kernel)(const GemmParams) = bfaintb_prefill128_kernel<BITS, GROUPED, PACKED, REF>;
    return launch_kernel(kernel, dim3(grid, 1, 1), dim3(512, 1, 1), 0, stream, p);
}

hipError_t launch_prefill128(const GemmParams& p, int bits, bool packed, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    if (p.reference_arith) return (bits == 8 && !grouped && !packed) ? launch_prefill128_t<8, false, false, true>(p, stream) : hipErrorInvalidValue;
    if (packed) {
        if (bits == 8) return grouped ? launch_prefill128_t<8, true, true>(p, stream) : launch_prefill128_t<8, false, true>(p, stream);
        return grouped ? launch_prefill128_t<4, true, true>(p, stream) : launch_prefill128_t<4, false, true>(p, stream);
    }
    if (bits == 8) return grouped ? launch_prefill128_t<8, true, false>(p, stream) : launch_prefill128_t<8, false, false>(p, stream);
    return grouped ? launch_prefill128_t<4, true, false>(p, stream) : launch_prefill128_t<4, false, false>(p, stream);
}

}  // namespace bfaintb
