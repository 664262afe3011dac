// Prefill variant (m > 32): 256x256x64 LDS-tiled bf16 MFMA kernel for gfx950.
//
// Replaces the reference kernel's 32x64x64 tile, two waves, v_mfma_f32_32x32x8bf16_1k,
// single-buffered LDS with two barriers per K-step
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:410-489, tile origin :222-223,
// LDS layouts :346-393, epilogue :594-630).
//
// Shape of the computation
//   grid = ceil(m/256) * ceil(n/256) workgroups of 512 threads (8 waves, 2 along m x 4 along n);
//   each wave owns a 128 x 64 block of the tile = 4 x 2 accumulators of v_mfma_f32_32x32x16_bf16.
//   K advances 64 per step.  LDS holds two stages of {A tile, dequantised W tile}, each tile
//   256 rows x 64 k of bf16 (row = 128 bytes = 8 chunks of 16 bytes), so a step needs one barrier.
//   Chunk c of row r lives at chunk position c ^ ((r >> 1) & 7): with 64 LDS banks, 16 lanes that
//   read or write the same chunk of 16 consecutive rows then touch 16 different 16-byte bank
//   groups (no conflicts).
// A path: 16-byte global loads (8 lanes per row) -> registers -> ds_write_b128.
// W path: wave w loads rows 8w..8w+7 of the step, one dword (4 codes) per lane per row, so that a
//   lane ends up with 8 consecutive k of 4 columns; it dequantises them (cvt_ubyte, fma, cvt_pk)
//   and writes one 16-byte chunk per column: column (4*lane + j) goes to LDS row
//   rho = (j>>1)*128 + (j&1)*32 + (lane&31) + (lane>>5)*64, which makes consecutive lanes write
//   consecutive rows.  The MFMA "column" index is the LDS row, so wave wn / accumulator t / lane
//   column jl hold tile column 4*(32*(wn&1) + jl) + 2*(wn>>1) + t.
// Epilogue: accumulators are rounded to bf16 (v_cvt_pk_bf16_f32; t = 0,1 are neighbouring
//   columns and share a dword), staged in LDS in true [m][n] order and stored with 16-byte
//   row-contiguous writes.
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr int kTileBytes = 256 * 128;             // one A or W tile in LDS
constexpr int kStageBytes = 2 * kTileBytes;       // A + W
constexpr int kCRowBytes = 256 * 2 + 16;          // epilogue staging row (padded)
constexpr int kLdsBytes = 256 * kCRowBytes;       // 135168 >= 2 stages (131072)

__device__ __forceinline__ uint32_t tile_off(uint32_t row, uint32_t chunk)
{
    return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4);
}

template <int BITS, bool GROUPED>
__global__ void __launch_bounds__(512) bfaintb_prefill_kernel(const GemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave >> 2;   // 0..1
    const uint32_t wn = wave & 3u;   // 0..3

    const uint32_t tiles_n = (p.n + kBN - 1) / kBN;
    const uint32_t tm = blockIdx.x / tiles_n;
    const uint32_t tn = blockIdx.x % tiles_n;
    const uint32_t m0 = tm * kBM;
    const uint32_t n0 = tn * kBN;

    // ---- A global -> LDS mapping: 4 chunks per thread, chunk id q = tid + 512*i
    const uint16_t* a_src[4];
    bool a_ok[4];
    uint32_t a_dst[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t q = tid + 512u * i;
        const uint32_t row = q >> 3, ch = q & 7u;
        a_ok[i] = (m0 + row) < p.m;
        a_src[i] = p.a + (size_t)(a_ok[i] ? (m0 + row) : 0) * p.lda + ch * 8u;
        a_dst[i] = tile_off(row, ch);
    }

    // ---- W mapping: k-group = wave (rows 8*wave..+7 of the step), 4 columns per lane
    const uint32_t ncol = n0 + 4u * lane;
    const bool w_ok = ncol < p.n;
    const uint8_t* b_src = p.b + (size_t)(8u * wave) * p.ldb_bytes + (BITS == 8 ? ncol : ncol / 2);
    uint32_t w_dst[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t rho = (j >> 1) * 128u + (j & 1u) * 32u + (lane & 31u) + (lane >> 5) * 64u;
        w_dst[j] = kTileBytes + tile_off(rho, wave);
    }

    float cs[4];
    uint32_t cur_group = 0xffffffffu;
    auto fetch_scales = [&](uint32_t g) {
        uint2 sr = make_uint2(0, 0);
        if (w_ok) sr = *reinterpret_cast<const uint2*>(p.scale + (size_t)g * p.lds + ncol);
        cs[0] = make_col_scale<BITS>(sr.x & 0xffffu);
        cs[1] = make_col_scale<BITS>(sr.x >> 16);
        cs[2] = make_col_scale<BITS>(sr.y & 0xffffu);
        cs[3] = make_col_scale<BITS>(sr.y >> 16);
    };
    if constexpr (!GROUPED) fetch_scales(0);

    uint4 a_reg[4];
    uint32_t b_reg[8];

    auto gload = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a_reg[i] = make_uint4(0, 0, 0, 0);
            if (a_ok[i]) a_reg[i] = *reinterpret_cast<const uint4*>(a_src[i] + k0);
        }
        const uint8_t* bp = b_src + (size_t)k0 * p.ldb_bytes;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if constexpr (BITS == 8) {
                b_reg[r] = 0x80808080u;
                if (w_ok) b_reg[r] = *reinterpret_cast<const uint32_t*>(bp + (size_t)r * p.ldb_bytes);
            } else {
                b_reg[r] = 0x8888u;
                if (w_ok) b_reg[r] = *reinterpret_cast<const uint16_t*>(bp + (size_t)r * p.ldb_bytes);
            }
        }
    };

    // signed value of column J (0..3) of a prepared row register (x16 for 4-bit codes)
    auto value = [&](uint32_t x, auto jc) -> float {
        constexpr int J = decltype(jc)::value;
        return sbyte_to_f32<J>(x);
    };
    // stored codes of one row (4 columns) -> 4 two's-complement bytes, byte J = column J
    auto prepare = [&](uint32_t x) -> uint32_t {
        if constexpr (BITS == 8) {
            return codes8_to_s8(x);
        } else {
            return codes4_quad_to_s8x16(x);
        }
    };

    auto lds_store = [&](uint32_t stage, uint32_t k0) {
        uint8_t* base = lds + stage * kStageBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4*>(base + a_dst[i]) = a_reg[i];
        if constexpr (GROUPED) {
            const uint32_t g = (k0 + 8u * wave) / p.group_size;
            if (g != cur_group) {
                cur_group = g;
                fetch_scales(g);
            }
        }
        uint32_t b_s8[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) b_s8[r] = prepare(b_reg[r]);
        auto put = [&](auto jc) {
            constexpr int J = decltype(jc)::value;
            uint4 w;
            w.x = pack_bf16_rne(value(b_s8[0], jc) * cs[J], value(b_s8[1], jc) * cs[J]);
            w.y = pack_bf16_rne(value(b_s8[2], jc) * cs[J], value(b_s8[3], jc) * cs[J]);
            w.z = pack_bf16_rne(value(b_s8[4], jc) * cs[J], value(b_s8[5], jc) * cs[J]);
            w.w = pack_bf16_rne(value(b_s8[6], jc) * cs[J], value(b_s8[7], jc) * cs[J]);
            *reinterpret_cast<uint4*>(base + w_dst[J]) = w;
        };
        put(std::integral_constant<int, 0>{});
        put(std::integral_constant<int, 1>{});
        put(std::integral_constant<int, 2>{});
        put(std::integral_constant<int, 3>{});
    };

    f32x16_t acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

    // fragment read offsets (chunk part added per kk)
    const uint32_t frag_row_a = wm * 128u + (lane & 31u);
    const uint32_t frag_row_w = wn * 64u + (lane & 31u);
    const uint32_t frag_half = lane >> 5;

    auto compute = [&](uint32_t stage) {
        const uint8_t* base = lds + stage * kStageBytes;
#pragma unroll
        for (uint32_t kk = 0; kk < 4; ++kk) {
            bf16x8_t af[4], wf[2];
#pragma unroll
            for (uint32_t mt = 0; mt < 4; ++mt)
                af[mt] = *reinterpret_cast<const bf16x8_t*>(base + tile_off(frag_row_a + 32u * mt, 2u * kk + frag_half));
#pragma unroll
            for (uint32_t t = 0; t < 2; ++t)
                wf[t] = *reinterpret_cast<const bf16x8_t*>(base + kTileBytes + tile_off(frag_row_w + 32u * t, 2u * kk + frag_half));
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mt], wf[t], acc[mt][t], 0, 0, 0);
        }
    };

    const uint32_t ksteps = p.k / kBK;
    gload(0);
    lds_store(0, 0);
    __syncthreads();
    for (uint32_t kt = 0; kt < ksteps; ++kt) {
        const uint32_t stage = kt & 1u;
        const bool more = kt + 1 < ksteps;
        if (more) gload((kt + 1) * kBK);
        compute(stage);
        if (more) lds_store(stage ^ 1u, (kt + 1) * kBK);
        __syncthreads();
    }

    // ---- epilogue: bf16 tile through LDS, then 16-byte row-contiguous stores
    {
        const uint32_t jl = lane & 31u;
        const uint32_t colbyte = 8u * (32u * (wn & 1u) + jl) + 4u * (wn >> 1);
#pragma unroll
        for (uint32_t mt = 0; mt < 4; ++mt)
#pragma unroll
            for (uint32_t i = 0; i < 16; ++i) {
                const uint32_t row = wm * 128u + 32u * mt + 8u * (i >> 2) + 4u * frag_half + (i & 3u);
                *reinterpret_cast<uint32_t*>(lds + row * kCRowBytes + colbyte) = pack_bf16_rne(acc[mt][0][i], acc[mt][1][i]);
            }
    }
    __syncthreads();
#pragma unroll 4
    for (uint32_t pass = 0; pass < 16; ++pass) {
        const uint32_t row = pass * 16u + (tid >> 5);
        const uint32_t ch = tid & 31u;
        const uint32_t gm = m0 + row, gn = n0 + ch * 8u;
        if (gm < p.m && gn < p.n) {
            const uint4 v = *reinterpret_cast<const uint4*>(lds + row * kCRowBytes + ch * 16u);
            *reinterpret_cast<uint4*>(p.c + (size_t)gm * p.ldc + gn) = v;
        }
    }
}

template <int BITS, bool GROUPED>
static hipError_t launch_prefill_t(const GemmParams& p, hipStream_t stream)
{
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&bfaintb_prefill_kernel<BITS, GROUPED>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const uint32_t tiles = ((p.m + kBM - 1) / kBM) * ((p.n + kBN - 1) / kBN);
    return launch_kernel(bfaintb_prefill_kernel<BITS, GROUPED>, dim3(tiles, 1, 1), dim3(512, 1, 1), kLdsBytes, stream, p);
}

hipError_t launch_prefill(const GemmParams& p, int bits, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    if (bits == 8) return grouped ? launch_prefill_t<8, true>(p, stream) : launch_prefill_t<8, false>(p, stream);
    return grouped ? launch_prefill_t<4, true>(p, stream) : launch_prefill_t<4, false>(p, stream);
}

}  // namespace bfaintb
