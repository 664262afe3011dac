// Decode variant (m <= 32): split-K weight streaming for gfx950.
//
// Replaces, for small m, the reference kernel bf16gemm_rrr_wg1x1_w1x2_32x32x8bf16_1k_pregld2
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630), whose 32x64 tile wastes 31/32 of
// each MFMA at m = 1 and launches only n/64 workgroups with no split along k.
//
// Work decomposition
//   grid  = (ceil(n/256), splits); block = 4 waves (the kernel itself accepts 4 or 8).
//   A workgroup owns 256 consecutive columns and k_per_wg rows of B; each wave owns an equal share of
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
//   The waves' partial sums are added through LDS; with splits > 1 each workgroup stores its
//   fp32 partial tile to the workspace and the LAST workgroup to arrive at a column block (an
//   arrival counter; nobody waits for another workgroup) adds the partials in split order and writes
//   bf16 C — the summation order is fixed, so results are reproducible run to run.
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
__device__ __forceinline__ void load_raw(RawStep<BITS>& raw, const uint8_t* rowptr, uint32_t ldb_bytes)
{
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if constexpr (BITS == 8) {
            const uint4 v = *reinterpret_cast<const uint4*>(rowptr + (size_t)r * ldb_bytes);
            raw.d[r][0] = v.x; raw.d[r][1] = v.y; raw.d[r][2] = v.z; raw.d[r][3] = v.w;
        } else {
            const uint2 v = *reinterpret_cast<const uint2*>(rowptr + (size_t)r * ldb_bytes);
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
#if defined(BFAINTB_EXPERIMENT) && (BFAINTB_EXPERIMENT == 1 || BFAINTB_EXPERIMENT == 2)
    // timing experiment: consume the loaded data without the dequantisation and MFMA work
    uint32_t x = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r) x ^= rows[r][0] ^ rows[r][1] ^ rows[r][2] ^ rows[r][3];
    acc[0][0][0] += __uint_as_float(x & 0x3fffffffu) * cs[0] + __uint_as_float(afrag[0].x);
#else
    (mac_column<BITS, MB, Cs>(rows, cs, afrag, acc), ...);
#endif
}

template <int BITS>
__device__ __forceinline__ void load_scales(uint4 (&sraw)[2], const uint16_t* sptr)
{
    sraw[0] = *reinterpret_cast<const uint4*>(sptr);
    sraw[1] = *reinterpret_cast<const uint4*>(sptr + 8);
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

#ifdef BFAINTB_TRACE
#define TRACE_MARK(i) do { if ((threadIdx.x & 63) == 0) p.partials[((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * 4 + (threadIdx.x >> 6)) * 8 + (i)] = wall_clock64(); } while (0)
#else
#define TRACE_MARK(i) do { } while (0)
#endif

constexpr uint32_t kTaggedMaxM = 4;         // up to this m split-K partial sums travel in tagged slots
constexpr uint32_t kMaxSlotRetries = 1u << 16;  // re-reads of a split-K slot before giving up (each is a memory round trip)
constexpr int kRedStride = 260;  // floats per row of the LDS reduction buffer (256 + 4: spreads rows over banks)

template <int BITS, int MB, bool GROUPED>
__global__ void __launch_bounds__(MB == 1 ? 512 : 256) bfaintb_decode_kernel(const GemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) float red[];  // [waves][m rows][kRedStride], at least waves*1024 floats
    __shared__ uint32_t s_is_last;

    TRACE_MARK(0);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nl = lane & 15;
    const int kg = lane >> 4;
    const uint32_t cb = blockIdx.x;
    const uint32_t ks = blockIdx.y;

    // tag of this launch's split-K slots: one more than the column block's stored epoch, which the
    // last workgroup of the previous launch on this workspace left behind (read early, used late)
    const bool tagged = p.m <= kTaggedMaxM;
    // The tag carries the column block too, so that no two (column block, launch) pairs on one
    // workspace share a tag, whatever shapes the launches had.
    uint32_t epoch = 0, tag = 0;
    if (p.splits > 1) {
        epoch = __hip_atomic_load(p.epochs + cb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
        tag = ((epoch & 0xfffffu) << 12) | cb;  // cb < 4096
    }

    // ---- this lane's 16 weight columns.  A lane past the last column reads the last 16 columns
    //      instead (no predicated loads in the hot loop); what it computes is never stored.
    uint32_t n_ld = cb * 256u + (uint32_t)nl * 16u;
    if (n_ld >= p.n) n_ld = p.n - 16u;

    // ---- this wave's rows of k
    const uint32_t nwaves = blockDim.x >> 6;  // 4 or 8
    const uint32_t k_per_wave = p.k_per_wg / nwaves;
    const uint32_t kb = ks * p.k_per_wg + (uint32_t)wave * k_per_wave;
    uint32_t ke = kb + k_per_wave;
    if (ke > p.k) ke = p.k;
    const int nsteps = kb < ke ? (int)((ke - kb) >> 5) : 0;

    const uint8_t* bptr = p.b + (size_t)(kb + 8u * kg) * p.ldb_bytes + (BITS == 8 ? n_ld : n_ld / 2);
    const size_t bstep = (size_t)32 * p.ldb_bytes;

    // activation operand: row mi = 16*mb + lane%16, 8 consecutive k starting at k0 + 8*kg.
    // Lanes whose row is past m re-read row m-1; their accumulator columns are never stored.
    const uint16_t* aptr[MB];
    bool row_ok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const uint32_t mi = 16u * mb + (uint32_t)nl;
        row_ok[mb] = mi < p.m;
        aptr[mb] = p.a + (size_t)(row_ok[mb] ? mi : p.m - 1u) * p.lda + kb + 8u * kg;
    }

    f32x4_t acc[MB][16];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int c = 0; c < 16; ++c) acc[mb][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    if (nsteps > 0) {
        // Two register stages, used alternately: the loads of step s+1 are issued before step s is
        // computed.  Every load is unconditional and sits in straight-line code (the tail of one
        // or two steps is peeled off behind the loop), so the wait counts the compiler derives are
        // exact; a load behind a branch, or a stage copied into another, makes it wait for the
        // prefetch as well.
        struct Stage {
            RawStep<BITS> raw;
            uint4 af[MB];
            uint4 sraw[2];
        };
        float cs[16];
        const uint16_t* sptr = p.scale + n_ld;
        auto load_stage = [&](Stage& st, int step) {
            load_raw<BITS>(st.raw, bptr + (size_t)step * bstep, p.ldb_bytes);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) st.af[mb] = *reinterpret_cast<const uint4*>(aptr[mb] + (size_t)step * 32);
            if constexpr (GROUPED) load_scales<BITS>(st.sraw, sptr + (size_t)((kb + 32u * (uint32_t)step) / p.group_size) * p.lds);
            __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic that follows
        };
        auto compute_stage = [&](Stage& st) {
            if constexpr (GROUPED) apply_scales<BITS>(cs, st.sraw);
            mac_step<BITS, MB>(st.raw, cs, st.af, acc, std::make_integer_sequence<int, 16>{});
        };
        Stage s0, s1;
        if constexpr (!GROUPED) {
            load_scales<BITS>(s0.sraw, sptr);
        }
        load_stage(s0, 0);
        if constexpr (!GROUPED) apply_scales<BITS>(cs, s0.sraw);
        int s = 0;
        for (; s + 2 < nsteps; s += 2) {
            load_stage(s1, s + 1);
            compute_stage(s0);
            load_stage(s0, s + 2);
            compute_stage(s1);
        }
        if (nsteps - s == 2) {
            load_stage(s1, s + 1);
            compute_stage(s0);
            compute_stage(s1);
        } else {
            compute_stage(s0);
        }
    }
    TRACE_MARK(2);
#if defined(BFAINTB_EXPERIMENT) && BFAINTB_EXPERIMENT == 2
    // timing experiment: streaming phase only
    if (acc[0][0][0] == 123.456f) p.c[threadIdx.x] = 1;
    return;
#endif

    // ---- add the 4 waves' partial sums through LDS: one barrier, then thread t finishes two
    //      neighbouring columns.  acc[mb][c][r] of lane (nl, kg) is row mi = 16*mb + nl,
    //      local column (4*kg + r)*16 + c.
    const uint32_t rows_out = p.m;  // <= 16*MB
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        if (!row_ok[mb]) continue;
        float* row = red + ((size_t)wave * rows_out + (mb * 16 + nl)) * kRedStride;
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                float4 v = make_float4(acc[mb][4 * c4 + 0][r], acc[mb][4 * c4 + 1][r], acc[mb][4 * c4 + 2][r],
                                       acc[mb][4 * c4 + 3][r]);
                *reinterpret_cast<float4*>(row + (4 * kg + r) * 16 + 4 * c4) = v;
            }
    }
    __syncthreads();
    TRACE_MARK(3);
    {
        const uint32_t cp = threadIdx.x & 127u, rsel = threadIdx.x >> 7;
        const uint32_t col = cb * 256u + 2u * cp;
        if (col < p.n) {
            for (uint32_t row = rsel; row < rows_out; row += (blockDim.x >> 7)) {
                const float* src = red + (size_t)row * kRedStride + 2u * cp;
                float sx = 0.f, sy = 0.f;
                for (uint32_t w = 0; w < nwaves; ++w) {  // fixed order: wave 0 first
                    const float2 v = *reinterpret_cast<const float2*>(src + (size_t)w * rows_out * kRedStride);
                    sx += v.x;
                    sy += v.y;
                }
                if (p.splits == 1) {
                    *reinterpret_cast<uint32_t*>(p.c + (size_t)row * p.ldc + col) = pack_bf16_rne(sx, sy);
                } else {
                    // split-K partial sums go to 8-byte slots {value, tag}, written whole with device-scope
                    // (write-through) stores that nobody waits for: the reader recognises a slot of this
                    // launch by its tag
                    if (tagged) {
                        unsigned long long* slot = p.partials + ((size_t)ks * p.m + row) * p.n + col;
                        __hip_atomic_store(slot, (unsigned long long)__float_as_uint(sx) | ((unsigned long long)tag << 32), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(slot + 1, (unsigned long long)__float_as_uint(sy) | ((unsigned long long)tag << 32), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                    } else {
                        // larger m: plain fp32 partials (half the bytes, 16-byte loads for the reader); the
                        // arrival count then has to wait for the stores' acknowledgement
                        __hip_atomic_store(reinterpret_cast<unsigned long long*>(reinterpret_cast<float*>(p.partials) + ((size_t)ks * p.m + row) * p.n + col),
                                           (unsigned long long)__float_as_uint(sx) | ((unsigned long long)__float_as_uint(sy) << 32), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
        }
    }
    if (p.splits == 1) return;
    // ---- split-K: the last workgroup to arrive at this column block adds all partial tiles in a
    // fixed order and writes C.  The arrival count is bumped as soon as this workgroup's stores have
    // been ISSUED (the barrier), not acknowledged: a slot whose store is still in flight shows an old
    // tag and is simply read again.  That wait is on memory operations already under way, never on
    // another workgroup being scheduled, so it cannot deadlock.  (For m > kTaggedMaxM the partials are
    // untagged and the count waits for the acknowledgements instead.)
    if (!tagged) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // s_waitcnt vmcnt(0)
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t arrived = __hip_atomic_fetch_add(p.counters + cb, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_is_last = (arrived == p.splits - 1u) ? 1u : 0u;
    }
    __syncthreads();
    if (s_is_last == 0u) return;
#if defined(BFAINTB_EXPERIMENT) && BFAINTB_EXPERIMENT == 3
    if (threadIdx.x == 0) __hip_atomic_store(p.counters + cb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;  // timing experiment: no final reduction
#endif

    if (!tagged) {
    // acquire at device scope: drops lines of the partial tiles this XCD's L2 may still hold from an
    // earlier launch, so the plain (vectorisable, pipelined) loads below see the other workgroups' stores
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

    // thread t: 4 consecutive columns (cg = t%64), splits sp = sub, sub+waves, ... (sub = t/64), rows
    // in chunks of 4; the per-wave sub-sums are combined through LDS in a fixed order
    {
        const uint32_t cg = threadIdx.x & 63u, sub = threadIdx.x >> 6;
        const uint32_t col = cb * 256u + 4u * cg;
        const bool col_ok = col < p.n;
        __syncthreads();               // every wave is done reading its sums out of red
        float* stage = red;            // [waves][4 rows][256 cols]
        for (uint32_t m0 = 0; m0 < p.m; m0 += 4u) {
            const uint32_t rows = p.m - m0 < 4u ? p.m - m0 : 4u;
            for (uint32_t ri = 0; ri < rows; ++ri) {
                float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
                if (col_ok) {
                    const float* src = reinterpret_cast<const float*>(p.partials) + (size_t)(m0 + ri) * p.n + col;
                    for (uint32_t sp = sub; sp < p.splits; sp += nwaves) {
                        const float4 v = *reinterpret_cast<const float4*>(src + (size_t)sp * p.m * p.n);
                        sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
                    }
                }
                *reinterpret_cast<float4*>(stage + (sub * 4u + ri) * 256u + 4u * cg) = sum;
            }
            __syncthreads();
            {
                const uint32_t ri = sub;  // thread t finishes row t/64 of the chunk
                if (ri < rows && col_ok) {
                    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                    for (uint32_t w = 0; w < nwaves; ++w) {
                        const float4 v = *reinterpret_cast<const float4*>(stage + (w * 4u + ri) * 256u + 4u * cg);
                        t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
                    }
                    uint2 o;
                    o.x = pack_bf16_rne(t.x, t.y);
                    o.y = pack_bf16_rne(t.z, t.w);
                    *reinterpret_cast<uint2*>(p.c + (size_t)(m0 + ri) * p.ldc + col) = o;
                }
            }
            __syncthreads();
        }
    }
    } else {
    // thread t owns column cb*256 + t: all splits of a row are fetched together (device-scope loads,
    // which bypass whatever this XCD's L2 holds from an earlier launch), then added in split order
        const uint32_t col = cb * 256u + threadIdx.x;
        constexpr uint32_t kBatch = 16;
        if (threadIdx.x < 256u && col < p.n) {
            for (uint32_t mi = 0; mi < p.m; ++mi) {
                const unsigned long long* src = p.partials + (size_t)mi * p.n + col;
                const size_t stride = (size_t)p.m * p.n;
                float sum = 0.f;
                for (uint32_t sp0 = 0; sp0 < p.splits; sp0 += kBatch) {
                    unsigned long long v[kBatch];
#pragma unroll
                    for (uint32_t i = 0; i < kBatch; ++i) {
                        const uint32_t sp = sp0 + i < p.splits ? sp0 + i : p.splits - 1u;
                        v[i] = __hip_atomic_load(src + (size_t)sp * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (uint32_t i = 0; i < kBatch; ++i) {
                        if (sp0 + i < p.splits) {
                            // store still in flight: read the slot again (bounded, so the kernel ends whatever happens;
                            // a slot that never shows its tag poisons the output with a NaN instead of hanging)
                            for (uint32_t tries = 0; (uint32_t)(v[i] >> 32) != tag && tries < kMaxSlotRetries; ++tries)
                                v[i] = __hip_atomic_load(src + (size_t)(sp0 + i) * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            sum += (uint32_t)(v[i] >> 32) == tag ? __uint_as_float((uint32_t)v[i]) : __uint_as_float(0x7fc00000u);
                        }
                    }
                }
                p.c[(size_t)mi * p.ldc + col] = (uint16_t)(pack_bf16_rne(sum, 0.f) & 0xffffu);
            }
        }
    }
    if (threadIdx.x == 0) {  // ready for the next launch: new tag, counter back to zero
        __hip_atomic_store(p.epochs + cb, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(p.counters + cb, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <int BITS, int MB, bool GROUPED>
static hipError_t launch_decode_t(const GemmParams& p, hipStream_t stream)
{
    const dim3 grid((p.n + 255u) / 256u, p.splits, 1);
    const uint32_t waves = p.decode_waves;
    size_t lds = (size_t)waves * p.m * kRedStride * sizeof(float);
    if (lds < (size_t)waves * 1024 * sizeof(float)) lds = (size_t)waves * 1024 * sizeof(float);
    if (lds > 64 * 1024) {
        static bool attr_set = false;
        if (!attr_set) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&bfaintb_decode_kernel<BITS, MB, GROUPED>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 4 * 32 * kRedStride * (int)sizeof(float));
            if (e != hipSuccess) return e;
            attr_set = true;
        }
    }
    return launch_kernel(bfaintb_decode_kernel<BITS, MB, GROUPED>, grid, dim3(64 * waves, 1, 1), lds, stream, p);
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
