// Decode variant (m <= 32): split-K weight streaming for gfx950.
//
// Replaces, for small m, the reference kernel bf16gemm_rrr_wg1x1_w1x2_32x32x8bf16_1k_pregld2
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630), whose 32x64 tile wastes 31/32 of
// each MFMA at m = 1 and launches only n/64 workgroups with no split along k.
//
// Work decomposition
//   grid  = (ceil(n/256), splits); block = 256 threads = 4 waves.
//   A workgroup owns 256 consecutive columns and k_per_wg rows of B; each wave owns a quarter of
//   those rows and walks them in steps of 32 rows.
//   Within a wave, lane = (kg, nl) with nl = lane%16, kg = lane/16.  Per step the lane loads, from
//   each of the 8 rows k0 + 8*kg + r, the 16 consecutive weights of columns n0 + 16*nl .. +15
//   (one 128-bit load per row for 8-bit codes, one 64-bit load for 4-bit codes): a wave request
//   covers 4 rows x 256 contiguous bytes (8-bit).  Nothing of B goes through LDS.
//   The products run on v_mfma_f32_16x16x32_bf16 with the operands swapped (C^T = W^T A^T): for
//   c = 0..15 the dequantised weights of column 16*nl + c, rows 8*kg..8*kg+7, are exactly the
//   8-element operand of lane (nl, kg); the activations A[mi][k0 + 8*kg .. +7] of row mi = lane%16
//   are the other operand, so one instruction multiplies 16 columns x 32 rows by up to 16 rows of A.
//   Rows of A beyond m are zero operands.
//   The 4 waves' partial sums are added through LDS; with splits > 1 each workgroup stores its
//   fp32 partial tile to the workspace and the LAST workgroup to arrive at a column block (an
//   arrival counter, no spinning) adds the partials in split order and writes bf16 C — the
//   summation order is fixed, so results are reproducible run to run.
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

template <int BITS>
struct RawStep {
    static constexpr int kDwords = BITS == 8 ? 4 : 2;
    uint32_t d[8][kDwords];  // 8 rows x 16 codes
};

// Signed value of column C (0..15) of one prepared row, as fp32 (x16 for 4-bit codes).
template <int BITS, int C>
__device__ __forceinline__ float value_f32(const uint32_t (&row)[4])
{
    if constexpr (BITS == 8) {
        return sbyte_to_f32<C % 4>(row[C / 4]);
    } else {
        // prepared 4-bit row: dwords {even columns of raw dword 0, odd of 0, even of 1, odd of 1};
        // column C sits in raw dword C/8, byte (C%8)/2
        return sbyte_to_f32<(C % 8) / 2>(row[2 * (C / 8) + (C % 2)]);
    }
}

template <int BITS>
__device__ __forceinline__ void load_raw(RawStep<BITS>& raw, const uint8_t* rowptr, uint32_t ldb_bytes, bool ok)
{
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if constexpr (BITS == 8) {
            uint4 v = make_uint4(0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u);
            if (ok) v = *reinterpret_cast<const uint4*>(rowptr + (size_t)r * ldb_bytes);
            raw.d[r][0] = v.x; raw.d[r][1] = v.y; raw.d[r][2] = v.z; raw.d[r][3] = v.w;
        } else {
            uint2 v = make_uint2(0x88888888u, 0x88888888u);
            if (ok) v = *reinterpret_cast<const uint2*>(rowptr + (size_t)r * ldb_bytes);
            raw.d[r][0] = v.x; raw.d[r][1] = v.y;
        }
    }
}

// Stored codes of one row -> four dwords of two's-complement bytes.
template <int BITS>
__device__ __forceinline__ void prepare_row(uint32_t (&out)[4], const uint32_t (&in)[RawStep<BITS>::kDwords])
{
    if constexpr (BITS == 8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = codes8_to_s8(in[i]);
    } else {
        out[0] = codes4_even_to_s8x16(in[0]);
        out[1] = codes4_odd_to_s8x16(in[0]);
        out[2] = codes4_even_to_s8x16(in[1]);
        out[3] = codes4_odd_to_s8x16(in[1]);
    }
}

template <int BITS, int MB, int C>
__device__ __forceinline__ void mac_column(const uint32_t (&rows)[8][4], const float (&cs)[16], const uint4 (&afrag)[MB],
                                           f32x4_t (&acc)[MB][16])
{
    uint4 w;
    w.x = pack_bf16_rne(value_f32<BITS, C>(rows[0]) * cs[C], value_f32<BITS, C>(rows[1]) * cs[C]);
    w.y = pack_bf16_rne(value_f32<BITS, C>(rows[2]) * cs[C], value_f32<BITS, C>(rows[3]) * cs[C]);
    w.z = pack_bf16_rne(value_f32<BITS, C>(rows[4]) * cs[C], value_f32<BITS, C>(rows[5]) * cs[C]);
    w.w = pack_bf16_rne(value_f32<BITS, C>(rows[6]) * cs[C], value_f32<BITS, C>(rows[7]) * cs[C]);
    const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, w);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        acc[mb][C] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, __builtin_bit_cast(bf16x8_t, afrag[mb]), acc[mb][C], 0, 0, 0);
    }
}

template <int BITS, int MB, int... Cs>
__device__ __forceinline__ void mac_step(const RawStep<BITS>& raw, const float (&cs)[16], const uint4 (&afrag)[MB],
                                         f32x4_t (&acc)[MB][16], std::integer_sequence<int, Cs...>)
{
    uint32_t rows[8][4];
#pragma unroll
    for (int r = 0; r < 8; ++r) prepare_row<BITS>(rows[r], raw.d[r]);
    (mac_column<BITS, MB, Cs>(rows, cs, afrag, acc), ...);
}

template <int BITS>
__device__ __forceinline__ void load_scales(uint4 (&sraw)[2], const uint16_t* sptr, bool ok)
{
    sraw[0] = make_uint4(0, 0, 0, 0);
    sraw[1] = make_uint4(0, 0, 0, 0);
    if (ok) {
        sraw[0] = *reinterpret_cast<const uint4*>(sptr);
        sraw[1] = *reinterpret_cast<const uint4*>(sptr + 8);
    }
}

template <int BITS>
__device__ __forceinline__ void apply_scales(float (&cs)[16], const uint4 (&sraw)[2])
{
    const uint32_t d[8] = {sraw[0].x, sraw[0].y, sraw[0].z, sraw[0].w, sraw[1].x, sraw[1].y, sraw[1].z, sraw[1].w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        cs[2 * i] = make_col_scale<BITS>(d[i] & 0xffffu);
        cs[2 * i + 1] = make_col_scale<BITS>(d[i] >> 16);
    }
}

constexpr int kRedStride = 260;  // floats per row of the LDS reduction buffer (256 + 4: spreads rows over banks)

template <int BITS, int MB, bool GROUPED>
__global__ void __launch_bounds__(256) bfaintb_decode_kernel(const GemmParams p)
{
    __shared__ float red[2][MB * 16][kRedStride];
    __shared__ uint32_t s_is_last;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nl = lane & 15;
    const int kg = lane >> 4;
    const uint32_t cb = blockIdx.x;
    const uint32_t ks = blockIdx.y;

    // ---- this lane's 16 weight columns
    const uint32_t n_ld = cb * 256u + (uint32_t)nl * 16u;
    const bool col_ok = n_ld < p.n;

    // ---- this wave's rows of k
    const uint32_t k_per_wave = p.k_per_wg >> 2;
    const uint32_t kb = ks * p.k_per_wg + (uint32_t)wave * k_per_wave;
    uint32_t ke = kb + k_per_wave;
    if (ke > p.k) ke = p.k;
    const int nsteps = kb < ke ? (int)((ke - kb) >> 5) : 0;

    const uint8_t* bptr = p.b + (size_t)(kb + 8u * kg) * p.ldb_bytes + (BITS == 8 ? n_ld : n_ld / 2);
    const size_t bstep = (size_t)32 * p.ldb_bytes;

    // activation operand: row mi = 16*mb + lane%16, 8 consecutive k starting at k0 + 8*kg
    const uint16_t* aptr[MB];
    bool a_ok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const uint32_t mi = 16u * mb + (uint32_t)nl;
        a_ok[mb] = mi < p.m;
        aptr[mb] = p.a + (size_t)(a_ok[mb] ? mi : 0) * p.lda + kb + 8u * kg;
    }

    f32x4_t acc[MB][16];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int c = 0; c < 16; ++c) acc[mb][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    float cs[16];
    uint4 sraw[2];
    uint32_t cur_group = 0;
    {
        if constexpr (GROUPED) cur_group = (kb < p.k ? kb : 0) / p.group_size;
        load_scales<BITS>(sraw, p.scale + (size_t)cur_group * p.lds + n_ld, col_ok);
        apply_scales<BITS>(cs, sraw);
    }

    RawStep<BITS> raw0, raw1;
    uint4 af0[MB], af1[MB];
    auto load_a = [&](uint4(&af)[MB], int step) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            af[mb] = make_uint4(0, 0, 0, 0);
            if (a_ok[mb]) af[mb] = *reinterpret_cast<const uint4*>(aptr[mb] + (size_t)step * 32);
        }
    };
    // Scales for the group a step belongs to are fetched one step ahead, when the group changes.
    auto prefetch_scales = [&](int step) -> bool {
        if constexpr (GROUPED) {
            const uint32_t g = (kb + 32u * step) / p.group_size;
            if (g != cur_group) {
                cur_group = g;
                load_scales<BITS>(sraw, p.scale + (size_t)g * p.lds + n_ld, col_ok);
                return true;
            }
        }
        return false;
    };

    if (nsteps > 0) {
        load_raw<BITS>(raw0, bptr, p.ldb_bytes, col_ok);
        load_a(af0, 0);
    }
    int s = 0;
    bool new_scales = false;
    while (s < nsteps) {
        bool ns_next = false;
        if (s + 1 < nsteps) {
            load_raw<BITS>(raw1, bptr + (size_t)(s + 1) * bstep, p.ldb_bytes, col_ok);
            load_a(af1, s + 1);
        }
        if (new_scales) apply_scales<BITS>(cs, sraw);
        if (s + 1 < nsteps) ns_next = prefetch_scales(s + 1);
        mac_step<BITS, MB>(raw0, cs, af0, acc, std::make_integer_sequence<int, 16>{});
        new_scales = ns_next;
        if (++s >= nsteps) break;

        ns_next = false;
        if (s + 1 < nsteps) {
            load_raw<BITS>(raw0, bptr + (size_t)(s + 1) * bstep, p.ldb_bytes, col_ok);
            load_a(af0, s + 1);
        }
        if (new_scales) apply_scales<BITS>(cs, sraw);
        if (s + 1 < nsteps) ns_next = prefetch_scales(s + 1);
        mac_step<BITS, MB>(raw1, cs, af1, acc, std::make_integer_sequence<int, 16>{});
        new_scales = ns_next;
        ++s;
    }

    // ---- add the 4 waves' partial sums.  acc[mb][c][r] of lane (nl, kg) is
    //      row mi = 16*mb + nl, local column (4*kg + r)*16 + c.
    auto lds_store = [&](int slot) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (!a_ok[mb]) continue;
            float* row = &red[slot][mb * 16 + nl][0];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) {
                    float4 v = make_float4(acc[mb][4 * c4 + 0][r], acc[mb][4 * c4 + 1][r], acc[mb][4 * c4 + 2][r],
                                           acc[mb][4 * c4 + 3][r]);
                    *reinterpret_cast<float4*>(row + (4 * kg + r) * 16 + 4 * c4) = v;
                }
        }
    };
    auto lds_add = [&](int slot) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (!a_ok[mb]) continue;
            const float* row = &red[slot][mb * 16 + nl][0];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) {
                    const float4 v = *reinterpret_cast<const float4*>(row + (4 * kg + r) * 16 + 4 * c4);
                    acc[mb][4 * c4 + 0][r] += v.x;
                    acc[mb][4 * c4 + 1][r] += v.y;
                    acc[mb][4 * c4 + 2][r] += v.z;
                    acc[mb][4 * c4 + 3][r] += v.w;
                }
        }
    };
    if (wave >= 2) lds_store(wave - 2);
    __syncthreads();
    if (wave < 2) lds_add(wave);
    __syncthreads();
    if (wave == 1) lds_store(0);
    __syncthreads();
    if (wave == 0) lds_add(0);

    // ---- output
    if (p.splits == 1) {
        if (wave == 0) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                if (!a_ok[mb]) continue;
                const uint32_t mi = 16u * mb + (uint32_t)nl;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t n_out = cb * 256u + (uint32_t)(4 * kg + r) * 16u;
                    if (n_out >= p.n) continue;
                    uint4 lo, hi;
                    lo.x = pack_bf16_rne(acc[mb][0][r], acc[mb][1][r]);
                    lo.y = pack_bf16_rne(acc[mb][2][r], acc[mb][3][r]);
                    lo.z = pack_bf16_rne(acc[mb][4][r], acc[mb][5][r]);
                    lo.w = pack_bf16_rne(acc[mb][6][r], acc[mb][7][r]);
                    hi.x = pack_bf16_rne(acc[mb][8][r], acc[mb][9][r]);
                    hi.y = pack_bf16_rne(acc[mb][10][r], acc[mb][11][r]);
                    hi.z = pack_bf16_rne(acc[mb][12][r], acc[mb][13][r]);
                    hi.w = pack_bf16_rne(acc[mb][14][r], acc[mb][15][r]);
                    uint16_t* dst = p.c + (size_t)mi * p.ldc + n_out;
                    *reinterpret_cast<uint4*>(dst) = lo;
                    *reinterpret_cast<uint4*>(dst + 8) = hi;
                }
            }
        }
        return;
    }

    // ---- split-K: publish this workgroup's partial tile, last arrival reduces
    if (wave == 0) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            if (!a_ok[mb]) continue;
            const uint32_t mi = 16u * mb + (uint32_t)nl;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t n_out = cb * 256u + (uint32_t)(4 * kg + r) * 16u;
                if (n_out >= p.n) continue;
                float* dst = p.partials + ((size_t)ks * p.m + mi) * p.n + n_out;
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) {
                    *reinterpret_cast<float4*>(dst + 4 * c4) =
                        make_float4(acc[mb][4 * c4 + 0][r], acc[mb][4 * c4 + 1][r], acc[mb][4 * c4 + 2][r], acc[mb][4 * c4 + 3][r]);
                }
            }
        }
        __threadfence();  // release the partial tile at device scope before announcing arrival
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t arrived = atomicAdd(p.counters + cb, 1u);
        s_is_last = (arrived == p.splits - 1u) ? 1u : 0u;
    }
    __syncthreads();
    if (s_is_last == 0u) return;
    __threadfence();  // acquire: the other workgroups' tiles are visible from here on

    const uint32_t col = cb * 256u + threadIdx.x;
    if (col < p.n) {
        for (uint32_t mi = 0; mi < p.m; ++mi) {
            const float* src = p.partials + (size_t)mi * p.n + col;
            float sum = 0.f;
            for (uint32_t sp = 0; sp < p.splits; ++sp) sum += src[(size_t)sp * p.m * p.n];
            p.c[(size_t)mi * p.ldc + col] = (uint16_t)(pack_bf16_rne(sum, 0.f) & 0xffffu);
        }
    }
    if (threadIdx.x == 0) p.counters[cb] = 0u;  // ready for the next launch on this workspace
}

template <int BITS, int MB, bool GROUPED>
static hipError_t launch_decode_t(const GemmParams& p, hipStream_t stream)
{
    const dim3 grid((p.n + 255u) / 256u, p.splits, 1);
    return launch_kernel(bfaintb_decode_kernel<BITS, MB, GROUPED>, grid, dim3(256, 1, 1), 0, stream, p);
}

hipError_t launch_decode(const GemmParams& p, int bits, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    const int mb = p.m <= 16 ? 1 : 2;
    if (bits == 8) {
        if (mb == 1) return grouped ? launch_decode_t<8, 1, true>(p, stream) : launch_decode_t<8, 1, false>(p, stream);
        return grouped ? launch_decode_t<8, 2, true>(p, stream) : launch_decode_t<8, 2, false>(p, stream);
    }
    if (mb == 1) return grouped ? launch_decode_t<4, 1, true>(p, stream) : launch_decode_t<4, 1, false>(p, stream);
    return grouped ? launch_decode_t<4, 2, true>(p, stream) : launch_decode_t<4, 2, false>(p, stream);
}

}  // namespace bfaintb
