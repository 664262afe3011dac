// Decode variant (m <= 32): split-K weight streaming for gfx950.
//
// Replaces, for small m, the reference kernel bf16gemm_rrr_wg1x1_w1x2_32x32x8bf16_1k_pregld2
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630), whose 32x64 tile wastes 31/32 of
// each MFMA at m = 1 and launches only n/64 workgroups with no split along k.
//
// Work decomposition
//   grid  = (ceil(n/COLS), splits); block = 4 or 8 waves.  CPL = weights per lane and row (16 or 8),
//   COLS = 16*CPL columns per workgroup (256 or 128).
//   A workgroup owns COLS consecutive columns and k_per_wg rows of B; each wave owns an equal share of
//   those rows and walks them in steps of 32 rows.
//   Within a wave, lane = (kg, nl) with nl = lane%16, kg = lane/16.  Per step the lane loads, from
//   each of the 8 rows k0 + 8*kg + r, the CPL consecutive weights of columns n0 + CPL*nl .. +CPL-1
//   (128-bit or 64-bit loads): a wave request covers 4 rows x 16 lanes of contiguous bytes, whole
//   128-byte lines or more — except 4-bit codes in the 128-column shape (32-bit loads, half a line per row), which the
//   host picks where the weights are few and workgroups count for more than whole lines.  Nothing of B goes through LDS.
//   The products run on v_mfma_f32_16x16x32_bf16 with the operands swapped (C^T = W^T A^T): for
//   c = 0..CPL-1 the dequantised weights of column CPL*nl + c, rows 8*kg..8*kg+7, are exactly the
//   8-element operand of lane (nl, kg); the activations A[mi][k0 + 8*kg .. +7] of row mi = lane%16
//   are the other operand, so one instruction multiplies 16 columns x 32 rows by up to 16 rows of A.
//   Rows of A beyond m re-read row m-1; their results are never stored.
//   The waves' partial sums are added through LDS; with splits > 1 the partial tiles of a column
//   block meet in the workspace and the workgroup of the last split adds them in split order and
//   writes bf16 C — the summation order is fixed, so results are reproducible run to run.  The narrower block (CPL = 8)
//   needs half the splits for the same number of workgroups, i.e. half the partial-sum traffic.
#include <type_traits>
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

template <int BITS, int CPL>
struct RawStep {
    static constexpr int kDwords = CPL * BITS / 32;  // 4, 2 or 1
    uint32_t d[8][kDwords];  // 8 rows x CPL codes
};

// Signed value of column C (0..CPL-1) of one prepared row, as fp32 (divided by 16 for 4-bit codes).
template <int BITS, int C, int PD>
__device__ __forceinline__ float value_f32(const uint32_t (&row)[PD])
{
    if constexpr (BITS == 8) {
        return sbyte_to_f32<C % 4>(row[C / 4]);
    } else {
        // prepared 4-bit row: dwords {even columns of raw dword 0, odd of 0, even of 1, odd of 1};
        // column C sits in raw dword C/8, byte (C%8)/2
        return nibble_to_f32_sixteenth<(C % 8) / 2>(row[2 * (C / 8) + (C % 2)]);
    }
}

// Non-temporal loads: the weights are read once, and marked so they stream through the caches without displacing the
// activations, the scales, the workspace and the kernel's own code (measured on the fetch alone: 16 MiB in 3.9 us
// against 4.3 us with plain loads; 43 MiB in 7.9 against 8.7 us).
// `rows` is the same for every lane of the wave (it stays in scalar registers and advances there); `lane_off` is the
// lane's place within the 8 x CPL block, 32 bits wide.
template <int BITS, int CPL>
__device__ __forceinline__ void load_raw(RawStep<BITS, CPL>& raw, const uint8_t* rows, uint32_t lane_off, uint32_t ldb_bytes)
{
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const uint8_t* src = rows + (size_t)r * ldb_bytes + lane_off;
        if constexpr (RawStep<BITS, CPL>::kDwords == 4) {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
            raw.d[r][0] = v[0]; raw.d[r][1] = v[1]; raw.d[r][2] = v[2]; raw.d[r][3] = v[3];
        } else if constexpr (RawStep<BITS, CPL>::kDwords == 2) {
            const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(src));
            raw.d[r][0] = v[0]; raw.d[r][1] = v[1];
        } else {
            raw.d[r][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(src));
        }
    }
}

// Stored codes of one row -> CPL/4 dwords of two's-complement bytes.
template <int BITS, int CPL>
__device__ __forceinline__ void prepare_row(uint32_t (&out)[CPL / 4], const uint32_t (&in)[RawStep<BITS, CPL>::kDwords])
{
    if constexpr (BITS == 8) {
#pragma unroll
        for (int i = 0; i < CPL / 4; ++i) out[i] = codes8_to_s8(in[i]);
    } else {
        codes4_to_nibbles(in[0], out[0], out[1]);
        if constexpr (CPL == 16) codes4_to_nibbles(in[1], out[2], out[3]);
    }
}

template <int BITS, int CPL, int MB, bool REF, int C>
__device__ __forceinline__ void mac_column(const uint32_t (&rows)[8][CPL / 4], const float (&cs)[CPL], const uint4 (&afrag)[MB],
                                           f32x4_t (&acc)[MB][CPL])
{
    constexpr int PD = CPL / 4;
    uint4 w;
    w.x = pack_bf16<REF>(value_f32<BITS, C, PD>(rows[0]) * cs[C], value_f32<BITS, C, PD>(rows[1]) * cs[C]);
    w.y = pack_bf16<REF>(value_f32<BITS, C, PD>(rows[2]) * cs[C], value_f32<BITS, C, PD>(rows[3]) * cs[C]);
    w.z = pack_bf16<REF>(value_f32<BITS, C, PD>(rows[4]) * cs[C], value_f32<BITS, C, PD>(rows[5]) * cs[C]);
    w.w = pack_bf16<REF>(value_f32<BITS, C, PD>(rows[6]) * cs[C], value_f32<BITS, C, PD>(rows[7]) * cs[C]);
    const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, w);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        acc[mb][C] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, __builtin_bit_cast(bf16x8_t, afrag[mb]), acc[mb][C], 0, 0, 0);
    }
}

template <int BITS, int CPL, int MB, bool REF, int... Cs>
__device__ __forceinline__ void mac_step(const RawStep<BITS, CPL>& raw, const float (&cs)[CPL], const uint4 (&afrag)[MB],
                                         f32x4_t (&acc)[MB][CPL], std::integer_sequence<int, Cs...>)
{
    uint32_t rows[8][CPL / 4];
#pragma unroll
    for (int r = 0; r < 8; ++r) prepare_row<BITS, CPL>(rows[r], raw.d[r]);
    (mac_column<BITS, CPL, MB, REF, Cs>(rows, cs, afrag, acc), ...);
}

// ---- the same step over weights in the packed order (bfaintb_packed.hip): the workgroup's CPL column blocks of 16 take
//      the place of a lane's CPL consecutive columns.  For column block c the lane holds the 8 codes of column nl, rows
//      8 kg .. 8 kg + 7 of the K-block: two dwords (rows 0-3, 4-7) for 8-bit codes, one dword of 8 nibbles for 4-bit.
template <int BITS, int CPL>
struct PackedStep {
    static constexpr int kDwords = BITS == 8 ? 2 : 1;
    uint32_t d[CPL][kDwords];
};

// lane_off: where this lane's codes of the K-block sit inside a column block's slab; slab[c]: the slab of column block c
template <int BITS, int CPL>
__device__ __forceinline__ void load_packed(PackedStep<BITS, CPL>& raw, const uint8_t* const (&slab)[CPL], uint32_t lane_off)
{
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        if constexpr (BITS == 8) {
            const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(slab[c] + lane_off));
            raw.d[c][0] = v[0]; raw.d[c][1] = v[1];
        } else {
            raw.d[c][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(slab[c] + lane_off));
        }
    }
}

// Two neighbouring K-blocks (the first one even) with one load per column block: 16 bytes (8-bit codes) or 8 (4-bit)
template <int BITS, int CPL>
__device__ __forceinline__ void load_packed_pair(PackedStep<BITS, CPL>& first, PackedStep<BITS, CPL>& second, const uint8_t* const (&slab)[CPL],
                                                 uint32_t lane_off)
{
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        if constexpr (BITS == 8) {
            const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(slab[c] + lane_off));
            first.d[c][0] = v[0]; first.d[c][1] = v[1];
            second.d[c][0] = v[2]; second.d[c][1] = v[3];
        } else {
            const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(slab[c] + lane_off));
            first.d[c][0] = v[0];
            second.d[c][0] = v[1];
        }
    }
}

// 4-bit codes: a lane's whole share of a K-chunk of 128 rows (its four K-blocks) with one 16-byte load per column block
template <int CPL>
__device__ __forceinline__ void load_packed_chunk4(PackedStep<4, CPL> (&blocks)[4], const uint8_t* const (&slab)[CPL], uint32_t lane_off)
{
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(slab[c] + lane_off));
        blocks[0].d[c][0] = v[0];
        blocks[1].d[c][0] = v[1];
        blocks[2].d[c][0] = v[2];
        blocks[3].d[c][0] = v[3];
    }
}

template <int BITS, int CPL, int MB>
__device__ __forceinline__ void mac_step_packed(const PackedStep<BITS, CPL>& raw, const float (&cs)[CPL], const uint4 (&afrag)[MB],
                                                f32x4_t (&acc)[MB][CPL])
{
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const float s = cs[c];
        uint4 w;
        if constexpr (BITS == 8) {
            const uint32_t lo = codes8_to_s8(raw.d[c][0]), hi = codes8_to_s8(raw.d[c][1]);
            w.x = pack_bf16_rne(sbyte_to_f32<0>(lo) * s, sbyte_to_f32<1>(lo) * s);
            w.y = pack_bf16_rne(sbyte_to_f32<2>(lo) * s, sbyte_to_f32<3>(lo) * s);
            w.z = pack_bf16_rne(sbyte_to_f32<0>(hi) * s, sbyte_to_f32<1>(hi) * s);
            w.w = pack_bf16_rne(sbyte_to_f32<2>(hi) * s, sbyte_to_f32<3>(hi) * s);
        } else {
            uint32_t ev, od;
            codes4_to_nibbles(raw.d[c][0], ev, od);
            w.x = pack_bf16_rne(nibble_to_f32_sixteenth<0>(ev) * s, nibble_to_f32_sixteenth<0>(od) * s);
            w.y = pack_bf16_rne(nibble_to_f32_sixteenth<1>(ev) * s, nibble_to_f32_sixteenth<1>(od) * s);
            w.z = pack_bf16_rne(nibble_to_f32_sixteenth<2>(ev) * s, nibble_to_f32_sixteenth<2>(od) * s);
            w.w = pack_bf16_rne(nibble_to_f32_sixteenth<3>(ev) * s, nibble_to_f32_sixteenth<3>(od) * s);
        }
        const bf16x8_t wf = __builtin_bit_cast(bf16x8_t, w);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            acc[mb][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, __builtin_bit_cast(bf16x8_t, afrag[mb]), acc[mb][c], 0, 0, 0);
    }
}

// the lane's CPL scales in packed mode: column col[c] of a scale row, as raw bf16 pairs in the layout load_scales
// produces (scale c in half c % 2 of dword c / 2)
template <int CPL>
__device__ __forceinline__ void load_scales_packed(uint4 (&sraw)[CPL / 8], const uint16_t* srow, const uint32_t (&col)[CPL])
{
    uint32_t d[CPL / 2];
#pragma unroll
    for (int i = 0; i < CPL / 2; ++i) d[i] = (uint32_t)srow[col[2 * i]] | ((uint32_t)srow[col[2 * i + 1]] << 16);
#pragma unroll
    for (int i = 0; i < CPL / 8; ++i) sraw[i] = make_uint4(d[4 * i], d[4 * i + 1], d[4 * i + 2], d[4 * i + 3]);
}

// `srow`: a row of scales, the same for every lane; `first_col`: the lane's first column
template <int CPL>
__device__ __forceinline__ void load_scales(uint4 (&sraw)[CPL / 8], const uint16_t* srow, uint32_t first_col)
{
    const uint8_t* src = reinterpret_cast<const uint8_t*>(srow) + first_col * 2u;
#pragma unroll
    for (int i = 0; i < CPL / 8; ++i) sraw[i] = *reinterpret_cast<const uint4*>(src + 16 * i);
}

template <int BITS, int CPL>
__device__ __forceinline__ void apply_scales(float (&cs)[CPL], const uint4 (&sraw)[CPL / 8])
{
    uint32_t d[CPL / 2];
#pragma unroll
    for (int i = 0; i < CPL / 8; ++i) {
        d[4 * i] = sraw[i].x; d[4 * i + 1] = sraw[i].y; d[4 * i + 2] = sraw[i].z; d[4 * i + 3] = sraw[i].w;
    }
#pragma unroll
    for (int i = 0; i < CPL / 2; ++i) {
        cs[2 * i] = make_col_scale_nibble<BITS>(d[i] & 0xffffu);
        cs[2 * i + 1] = make_col_scale_nibble<BITS>(d[i] >> 16);
    }
}

#ifdef BFAINTB_TRACE
#define TRACE_MARK(i) do { if ((threadIdx.x & 63) == 0) p.trace[((size_t)((blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 8 + (i)] = wall_clock64(); } while (0)
#else
#define TRACE_MARK(i) do { } while (0)
#endif

// Blocks of 16 rows whose per-wave tiles fit in LDS together (4 waves; 8 waves run MB <= 2).
__host__ __device__ constexpr int decode_rows16_per_pass(int cpl, int mb)
{
    const int fit = cpl == 8 ? 4 : 2;  // 4 waves x 64 rows x 132 floats, or 4 waves x 32 rows x 260 floats: 133 KiB
    return mb < fit ? mb : fit;
}

// Dynamic LDS of one workgroup, in floats: the waves' tiles [waves][rows of one pass][COLS + 4].
__host__ __device__ inline uint32_t decode_red_floats(uint32_t waves, uint32_t rows, uint32_t cols)
{
    return waves * rows * (cols + 4u);
}

// Finishes four neighbouring columns of one row: t += bias[col .. col+3]; then either += residual[row][col .. col+3] and
// four bf16 outputs at C[row][col ..], or (gated) the two outputs silu(t.x) * t.y and silu(t.z) * t.w, += residual[row]
// [col/2 ..], at C[row][col/2 ..].  All additions in fp32, one rounding (a truncation with the reference's arithmetic).
__device__ __forceinline__ void finish_row4(const GemmParams& p, float4 t, uint32_t row, uint32_t col)
{
    if (p.bias != nullptr) {
        const uint2 raw = *reinterpret_cast<const uint2*>(p.bias + col);
        t.x += bf16_bits_to_f32(raw.x & 0xffffu);
        t.y += bf16_bits_to_f32(raw.x >> 16);
        t.z += bf16_bits_to_f32(raw.y & 0xffffu);
        t.w += bf16_bits_to_f32(raw.y >> 16);
    }
    if (p.activation == kActSiluGate) {
        float o0 = silu_gate(t.x, t.y), o1 = silu_gate(t.z, t.w);
        if (p.residual != nullptr) {
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(p.residual + (size_t)row * p.ldr + col / 2u);
            o0 += bf16_bits_to_f32(raw & 0xffffu);
            o1 += bf16_bits_to_f32(raw >> 16);
        }
        *reinterpret_cast<uint32_t*>(p.c + (size_t)row * p.ldc + col / 2u) = p.reference_arith ? pack_bf16_rtz(o0, o1) : pack_bf16_rne(o0, o1);
        return;
    }
    if (p.residual != nullptr) {
        const uint2 raw = *reinterpret_cast<const uint2*>(p.residual + (size_t)row * p.ldr + col);
        t.x += bf16_bits_to_f32(raw.x & 0xffffu);
        t.y += bf16_bits_to_f32(raw.x >> 16);
        t.z += bf16_bits_to_f32(raw.y & 0xffffu);
        t.w += bf16_bits_to_f32(raw.y >> 16);
    }
    uint2 o;
    o.x = p.reference_arith ? pack_bf16_rtz(t.x, t.y) : pack_bf16_rne(t.x, t.y);
    o.y = p.reference_arith ? pack_bf16_rtz(t.z, t.w) : pack_bf16_rne(t.z, t.w);
    *reinterpret_cast<uint2*>(p.c + (size_t)row * p.ldc + col) = o;
}

// Split-K, the reducing workgroup's part for one thread: R rows (first_row + rs, + nrs, ...; `rows` of
// them exist from first_row on) of 4 columns.  Fetches the other splits' partial sums, adds them in
// split order with the thread's own sums last, writes bf16 C and leaves the workspace words empty
// again.  sum[] may hold more than R rows; the rest is not this launch's.
template <uint32_t R, uint32_t NSUM>
__device__ __forceinline__ void reduce_splits(const GemmParams& p, const float4 (&sum)[NSUM], uint32_t first_row, uint32_t rows, uint32_t rs,
                                              uint32_t nrs, uint32_t col, bool col_ok)
{
    static_assert(R <= NSUM, "rows per thread");
    constexpr uint32_t kSplitBatch = 16u / R;  // splits whose partial sums a thread fetches together
    // Only threads that own an output of this pass take part: every fetch is a trip past the L1 cache, and the ones
    // a thread without outputs would make (there are many when m is small) only queue up in front of the others.
    if (!col_ok || rs >= rows) return;
    const uint32_t others = p.splits - 1u;
    const uint32_t split_bytes = p.m * p.n * 4u;
    // 16-byte device-scope accesses through a buffer resource over the workspace: four words of one row per
    // access, each word judged on its own (a 32-bit word is never torn)
    const __amdgpu_buffer_rsrc_t ws = __builtin_amdgcn_make_buffer_rsrc(p.partials, 0, (int)p.partial_bytes, kBufferFlags);
    const uint32_t base = (first_row * p.n + col) * 4u;
    const u32x4_t empty4 = {kEmptyWord, kEmptyWord, kEmptyWord, kEmptyWord};
    float4 total[R];
#pragma unroll
    for (uint32_t i = 0; i < R; ++i) total[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t sp0 = 0; sp0 < others; sp0 += kSplitBatch) {
        u32x4_t v[kSplitBatch][R];
        // All words of the batch are fetched together, and fetched again together while any of them is
        // still empty: one memory round trip per attempt, however many words were late.
        // Rows past the last one re-read a word that exists; what they fetch is not used.
        bool complete = false;
        uint32_t tries = 0;
        for (; !complete && tries < p.split_wait_limit; ++tries) {
#ifdef BFAINTB_TRACE
            if (tries == 1) TRACE_MARK(6);
#endif
            if (tries) __builtin_amdgcn_s_sleep(2);
            asm volatile("" ::: "memory");  // other workgroups write these words: every attempt really loads
#pragma unroll
            for (uint32_t j = 0; j < kSplitBatch; ++j) {
                if (sp0 + j < others) {  // the same for every thread
#pragma unroll
                    for (uint32_t i = 0; i < R; ++i) {
                        uint32_t row = rs + i * nrs;
                        if (row >= rows) row = rows - 1u;
                        v[j][i] = __builtin_amdgcn_raw_buffer_load_b128(ws, (int)(base + row * p.n * 4u), (int)((sp0 + j) * split_bytes), kAuxDeviceScope);
                    }
                }
            }
            complete = true;
#pragma unroll
            for (uint32_t j = 0; j < kSplitBatch; ++j)
                if (sp0 + j < others)
#pragma unroll
                    for (uint32_t i = 0; i < R; ++i)
                        if (rs + i * nrs < rows)
#pragma unroll
                            for (int h = 0; h < 4; ++h)
                                if (v[j][i][h] == kEmptyWord) complete = false;
        }
#ifdef BFAINTB_TRACE
        if ((threadIdx.x & 63) == 0) p.trace[((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 8 + 7] = tries;
        TRACE_MARK(1);
#endif
        // a word that never arrived is still the empty pattern, a NaN, and turns its sum into one; the workspace's
        // header remembers that it happened
        if (!complete) __hip_atomic_store(p.ws_header, kWorkspaceGaveUp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (uint32_t j = 0; j < kSplitBatch; ++j) {
#pragma unroll
            for (uint32_t i = 0; i < R; ++i) {
                const uint32_t row = rs + i * nrs;
                if (sp0 + j < others && row < rows) {
                    __builtin_amdgcn_raw_buffer_store_b128(empty4, ws, (int)(base + row * p.n * 4u), (int)((sp0 + j) * split_bytes), kAuxDeviceScope);
                    total[i].x += __uint_as_float(v[j][i][0]);
                    total[i].y += __uint_as_float(v[j][i][1]);
                    total[i].z += __uint_as_float(v[j][i][2]);
                    total[i].w += __uint_as_float(v[j][i][3]);
                }
            }
        }
    }
#pragma unroll
    for (uint32_t i = 0; i < R; ++i) {
        const uint32_t row = rs + i * nrs;
        if (row < rows) {
            finish_row4(p, make_float4(total[i].x + sum[i].x, total[i].y + sum[i].y, total[i].z + sum[i].z, total[i].w + sum[i].w),
                        first_row + row, col);
        }
    }
}

// The reducing workgroup's part where a thread has one row and the launch at most 8 splits (the 128-column kernels up to
// 16 rows of A): the same hand-over as reduce_splits — same words, same order of addition, same bits — with TWO fetch
// attempts in flight, the second issued kPollGap x 64 cycles after the first and each issued again as soon as it has come
// back incomplete.  A fetch is a round trip of about a microsecond past the L2, and whether the first one samples the
// workspace before or after the last producer's store has landed varies from launch to launch; with one attempt at a
// time a miss costs a whole further round trip, with two the workspace is sampled about twice per round trip.  Measured
// on one box (us, one attempt / two): 4096 x 4096, m = 1 / 4 / 16: 7.43 / 7.32, 7.71 / 7.86, 8.69 / 8.44;
// 11008 x 4096, m = 8 / 16: 12.79 / 12.42, 13.74 / 13.33; 1024 x 8192, m = 4: 7.83 / 7.50; 2048 x 4096, m = 12: 7.84 / 7.51.
// The 256-column kernels keep the single attempt: with two they were 1.5 to 6 % slower (11008 x 4096, m = 1: 11.88 / 12.59;
// 4-bit 28672 x 8192: 29.7 / 30.2).
// The selection of the winning attempt is written as copies under uniform branches: indexing the two register sets by a
// run-time flag sent both through scratch memory (0.8 us at m = 1, 5 us at m = 16).
constexpr int kPollGap = 8;
template <uint32_t NL, uint32_t NSUM>
__device__ __forceinline__ void reduce_splits_two_in_flight(const GemmParams& p, const float4 (&sum)[NSUM], uint32_t first_row, uint32_t rows,
                                                            uint32_t rs, uint32_t col, bool col_ok)
{
    if (!col_ok || rs >= rows) return;
    const uint32_t others = p.splits - 1u;  // 1 .. NL
    const uint32_t split_bytes = p.m * p.n * 4u;
    const __amdgpu_buffer_rsrc_t ws = __builtin_amdgcn_make_buffer_rsrc(p.partials, 0, (int)p.partial_bytes, kBufferFlags);
    const uint32_t off = ((first_row + rs) * p.n + col) * 4u;
    // (always NL loads, so that the wait counts are compile-time numbers: splits that do not exist re-read split 0)
    auto fetch = [&](u32x4_t (&v)[NL]) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (uint32_t j = 0; j < NL; ++j)
            v[j] = __builtin_amdgcn_raw_buffer_load_b128(ws, (int)off, (int)((j < others ? j : 0u) * split_bytes), kAuxDeviceScope);
    };
    auto whole = [&](const u32x4_t (&v)[NL]) -> bool {
        bool ok = true;
#pragma unroll
        for (uint32_t j = 0; j < NL; ++j)
#pragma unroll
            for (int h = 0; h < 4; ++h)
                if (j < others && v[j][h] == kEmptyWord) ok = false;
        return ok;
    };
    u32x4_t a[NL], b[NL];
    fetch(a);
    __builtin_amdgcn_s_sleep(kPollGap);
    fetch(b);
    uint32_t tries = 2;
    bool complete = false;
    u32x4_t win[NL];
    auto take = [&](const u32x4_t (&v)[NL]) {
#pragma unroll
        for (uint32_t j = 0; j < NL; ++j) win[j] = v[j];
    };
    for (;;) {
        if (whole(a)) { take(a); complete = true; break; }
#ifdef BFAINTB_TRACE
        if (tries == 2) TRACE_MARK(6);  // the first attempt has come back incomplete
#endif
        if (tries >= p.split_wait_limit) { take(a); break; }
        fetch(a);
        ++tries;
        if (whole(b)) { take(b); complete = true; break; }
        if (tries >= p.split_wait_limit) { take(b); break; }
        fetch(b);
        ++tries;
    }
#ifdef BFAINTB_TRACE
    // (attempts issued, the two up front included: 2 = the first one was whole)
    if ((threadIdx.x & 63) == 0) p.trace[((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) * 8 + 7] = tries;
    TRACE_MARK(1);
#endif
    if (!complete) __hip_atomic_store(p.ws_header, kWorkspaceGaveUp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const u32x4_t empty4 = {kEmptyWord, kEmptyWord, kEmptyWord, kEmptyWord};
    float4 total = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (uint32_t j = 0; j < NL; ++j) {
        if (j < others) {
            __builtin_amdgcn_raw_buffer_store_b128(empty4, ws, (int)off, (int)(j * split_bytes), kAuxDeviceScope);
            const u32x4_t v = win[j];
            total.x += __uint_as_float(v[0]);
            total.y += __uint_as_float(v[1]);
            total.z += __uint_as_float(v[2]);
            total.w += __uint_as_float(v[3]);
        }
    }
    finish_row4(p, make_float4(total.x + sum[0].x, total.y + sum[0].y, total.z + sum[0].z, total.w + sum[0].w), first_row + rs, col);
    // The attempt that did not win may still be in flight.  Its destination registers stay this function's until it has
    // come back: with nothing holding them, the compiler handed them to the constants of the emptying stores above while
    // the loads were still due to write them (a workspace word of the second split left holding a partial sum: found
    // by the at-rest check of the test suite).  The wait is behind every store this thread issues, where it costs nothing.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (uint32_t j = 0; j < NL; ++j) asm volatile("" ::"v"(a[j]), "v"(b[j]));
}

// PACKED: p.b holds the weights in the packed order; the workgroup's kCols columns are CPL column blocks of 16, and
// accumulator c of a lane belongs to column block c (local column 16 c + 4 kg + r instead of (4 kg + r) CPL + c).
// REF: the reference kernel's arithmetic (p.reference_arith): p.scale holds one fp32 scale per column, W is narrowed by
// truncation.
template <int BITS, int CPL, int MB, bool GROUPED, bool PACKED, bool REF>
// (packed 4-bit codes always run 4 waves: with 8 — their registers would allow it for one block of 16 rows — the 256-column
// kernel over packed weights is slower, 28672 x 8192, m = 16: 55 against 42 us)
__global__ void __launch_bounds__((MB <= 2 && (CPL == 8 || MB == 1) && !(PACKED && BITS == 4 && CPL == 16)) ? 512 : 256)
bfaintb_decode_kernel(const GemmParams p)
{
    static_assert(!REF || (BITS == 8 && !GROUPED && !PACKED), "the reference's arithmetic: 8-bit codes, row-major, one scale per column");
    constexpr int KB = decode_blocks_per_step(BITS, CPL, PACKED, MB);  // blocks of 32 rows per pipeline step
    constexpr uint32_t kCols = 16u * CPL;             // columns per workgroup
    constexpr uint32_t kRedStride = kCols + 4u;       // floats per row of a wave's tile in LDS (+4: spreads rows over banks)
    constexpr uint32_t kLaneBytes = CPL * BITS / 8;   // bytes of one row a lane loads
    extern __shared__ __attribute__((aligned(16))) float red[];

    TRACE_MARK(0);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same for the wave's lanes: what follows from it stays scalar
    const int nl = lane & 15;
    const int kg = lane >> 4;
    // 4-bit codes in rows, 128 columns per workgroup: a workgroup reads half of every 128-byte line and its neighbour the
    // other half.  Workgroups go to the XCDs (each with its own L2) in turn, so neighbours i and i + 1 would fetch every
    // line once each; within a run of 16 column blocks the two halves of a line are given to workgroups 8 apart instead,
    // which share an L2.
    uint32_t cb = blockIdx.x;
    if constexpr (BITS == 4 && CPL == 8 && !PACKED) {
        const uint32_t run = cb & ~15u;
        if (run + 16u <= gridDim.x) cb = run + 2u * (cb & 7u) + ((cb >> 3) & 1u);
    }
    const uint32_t ks = blockIdx.y;
    // rows of A and C this workgroup covers: block blockIdx.z of 16*MB rows
    const uint32_t row0 = blockIdx.z * (16u * MB);
    const uint32_t rows_here = p.m - row0 < 16u * MB ? p.m - row0 : 16u * MB;

    // ---- this lane's CPL weight columns.  A lane past the last column reads the last CPL columns
    //      instead (no predicated loads in the hot loop); what it computes is never stored.
    uint32_t n_ld = cb * kCols + (uint32_t)nl * CPL;
    if (n_ld >= p.n) n_ld = p.n - CPL;

    // ---- this wave's rows of k
    const uint32_t nwaves = blockDim.x >> 6;  // 4 or 8
    const uint32_t k_per_wave = p.k_per_wg / nwaves;
    const uint32_t kb = ks * p.k_per_wg + (uint32_t)wave * k_per_wave;
    uint32_t ke = kb + k_per_wave;
    if (ke > p.k) ke = p.k;
    const int nsteps = kb < ke ? (int)((ke - kb) / (32u * KB)) : 0;
    // Row-major weights, k not a multiple of 32 (it is one of 8): the wave that holds the end of k runs one more, partial
    // step.  (Packed weights come in whole K-chunks; scale groups are multiples of 32 rows that divide k.)
    const uint32_t tail_rows = (PACKED || GROUPED || kb >= ke) ? 0u : (ke - kb) % 32u;

    // the wave's first row of B (scalar) and this lane's place in a block of 32 rows (the host has checked that 32 rows'
    // worth of bytes fit 32 bits)
    const uint8_t* bptr = p.b + (size_t)kb * p.ldb_bytes;
    const uint32_t b_lane = 8u * (uint32_t)kg * p.ldb_bytes + n_ld * BITS / 8u;
    const size_t bstep = (size_t)32 * p.ldb_bytes;
    // packed: K-chunks of 64 (8-bit) or 128 (4-bit) rows, 1024 bytes each, hold 2 or 4 K-blocks of 32 rows; a lane's 16
    // bytes of a chunk are its K-blocks in order
    constexpr uint32_t kBlocksPerChunk = BITS == 8 ? 2u : 4u;
    constexpr uint32_t kBlockBytes = 16u / kBlocksPerChunk;
    // column block c of the workgroup (blocks past the last one re-read it; what they compute is never stored)
    constexpr bool kUniformSlabs = BITS == 8 || (CPL == 8 && MB == 2);
    const uint8_t* slab[CPL];
    uint32_t pk_col[CPL];
    if constexpr (PACKED) {
        const size_t slab_bytes = (size_t)p.k * 16u * BITS / 8u;
        const uint32_t nblocks = p.n / 16u;
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            uint32_t gb = cb * CPL + (uint32_t)c;
            if (gb >= nblocks) gb = nblocks - 1u;
            // 8-bit codes, and 4-bit codes with two row blocks in the 128-column form: the same for every lane (scalar registers;
            // the lane's share is in the load's offset): those 8-wave kernels have no vector registers to spare.  Other 4-bit
            // kernels: 16 bases do not fit the scalar file, and there is room for per-lane pointers (measured 4-19 % faster
            // that way).
            slab[c] = p.b + (size_t)gb * slab_bytes + (kUniformSlabs ? 0u : (size_t)lane * 16u);
            pk_col[c] = 16u * gb + (uint32_t)nl;
        }
    }
    const uint32_t kblock0 = kb / 32u;  // first K-block of this wave
    static_assert(kLaneBytes == 16 || kLaneBytes == 8 || kLaneBytes == 4, "row-major weights: a lane loads 16, 8 or (4-bit codes, 128 columns) 4 bytes of a row");

    // activation operand: row mi = 16*mb + lane%16, 8 consecutive k starting at k0 + 8*kg.
    // Lanes whose row is past the last one re-read the last one; their accumulator columns are never stored.
    const uint16_t* aptr[MB];
    bool row_ok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const uint32_t mi = 16u * mb + (uint32_t)nl;
        row_ok[mb] = mi < rows_here;
        aptr[mb] = p.a + (size_t)(row0 + (row_ok[mb] ? mi : rows_here - 1u)) * p.lda + kb + 8u * kg;
    }

    f32x4_t acc[MB][CPL];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int c = 0; c < CPL; ++c) acc[mb][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    if (nsteps > 0 || tail_rows != 0u) {
        // Two register stages, used alternately: the loads of step s+1 are issued before step s is
        // computed.  A step is KB blocks of 32 rows, so that a lane has 128 bytes of B in flight per
        // stage whatever CPL is.  Every load is unconditional and sits in straight-line code (the
        // tail of one or two steps is peeled off behind the loop), so the wait counts the compiler
        // derives are exact; a load behind a branch, or a stage copied into another, makes it wait
        // for the prefetch as well.
        struct Stage {
            std::conditional_t<PACKED, PackedStep<BITS, CPL>, RawStep<BITS, CPL>> raw[KB];
            uint4 af[KB][MB];
            uint4 sraw[KB][CPL / 8];
        };
        float cs[CPL];
        const uint16_t* sptr = p.scale;
        // packed weights with grouped scales: the wave's transposition table in LDS, behind the reduction area, and
        // the columns whose scales this lane fetches (kept inside the scale row)
        uint16_t* sc_table = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(red) + p.decode_scale_lds) + (uint32_t)wave * 16u * CPL;
        uint32_t sc_col = cb * kCols + 4u * (uint32_t)lane;
        if (sc_col + 4u > p.n) sc_col = p.n - 4u;
        // Packed 8-bit codes: a workgroup starts its walk along k at a step of its own (and wraps round).  Slabs lie k x 16 bytes apart; when that is a large power of two, every workgroup's loads of a step
        // differ only in address bits that do not choose the memory channel, and the launch crowds onto a few of them
        // (8192 x 8192, m = 16: 20.7 us, 16.6 with k = 8064 — same plan, fewer bytes by 1.6 %).  The order in which a
        // wave adds its steps differs from workgroup to workgroup, so it is fixed by the launch shape, as before.
        constexpr bool kRotateSteps = PACKED && BITS == 8;
        int first_step = 0;
        if constexpr (kRotateSteps) {
            if (nsteps > 1) first_step = (int)((cb + ks) % (uint32_t)nsteps);
        }
        auto load_stage = [&](Stage& st, int step) {
            if constexpr (kRotateSteps) {
                step += first_step;
                if (step >= nsteps) step -= nsteps;
            }
#pragma unroll
            for (int q = 0; q < KB; ++q) {
                const size_t blk = (size_t)step * KB + q;
                if constexpr (PACKED && KB == 4) {
                    // the step is one K-chunk of 4-bit codes: the lane's 16 bytes of it
                    if constexpr (BITS == 4) {
                        if (q == 0) {
                            const uint32_t kblock = kblock0 + (uint32_t)blk;
                            load_packed_chunk4<CPL>(st.raw, slab, (kUniformSlabs ? (uint32_t)lane * 16u : 0u) + (kblock / kBlocksPerChunk) * 1024u);
                        }
                    }
                } else if constexpr (PACKED && KB == 2) {
                    // the step's two K-blocks (an even one and its successor) lie side by side in a lane's share of the chunk
                    if (q == 0) {
                        const uint32_t kblock = kblock0 + (uint32_t)blk;
                        load_packed_pair<BITS, CPL>(st.raw[0], st.raw[1], slab,
                                                    (kUniformSlabs ? (uint32_t)lane * 16u : 0u) + (kblock / kBlocksPerChunk) * 1024u + (kblock % kBlocksPerChunk) * kBlockBytes);
                    }
                } else if constexpr (PACKED) {
                    const uint32_t kblock = kblock0 + (uint32_t)blk;
                    load_packed<BITS, CPL>(st.raw[q], slab,
                                           (kUniformSlabs ? (uint32_t)lane * 16u : 0u) + (kblock / kBlocksPerChunk) * 1024u + (kblock % kBlocksPerChunk) * kBlockBytes);
                } else {
                    load_raw<BITS, CPL>(st.raw[q], bptr + blk * bstep, b_lane, p.ldb_bytes);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) st.af[q][mb] = *reinterpret_cast<const uint4*>(aptr[mb] + blk * 32);
                if constexpr (GROUPED) {
                    const uint16_t* srow = sptr + (size_t)group_of_row(p, kb + 32u * (uint32_t)blk) * p.lds;
                    if constexpr (PACKED) {
                        // lane j fetches the scales of the workgroup's columns 4j .. 4j+3 (one 8-byte load instead of CPL
                        // 2-byte gathers); compute_stage turns them, through LDS, into this lane's CPL scales
                        const uint2 v = *reinterpret_cast<const uint2*>(srow + sc_col);
                        st.sraw[q][0].x = v.x;
                        st.sraw[q][0].y = v.y;
                    } else {
                        load_scales<CPL>(st.sraw[q], srow, n_ld);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic that follows
        };
        // grouped scales: blocks of 32 rows until the next group begins (0: the block at hand opens one — so does the wave's
        // first, wherever in a group it lies), and how many the group after that spans
        uint32_t blocks_to_group = 0u;
        uint32_t next_group_blocks = 0u;
        // (a walk that starts at step first_step wraps round to the wave's first row after nsteps - first_step steps, and
        // the count starts again there)
        uint32_t steps_to_wrap = 0u;
        if constexpr (GROUPED) {
            const uint32_t kb_uniform = __builtin_amdgcn_readfirstlane(kb) + 32u * (uint32_t)KB * (uint32_t)first_step;
            next_group_blocks = (p.group_size - kb_uniform % p.group_size) / 32u;
            steps_to_wrap = (uint32_t)(nsteps - first_step);
        }
        auto compute_stage = [&](Stage& st) {
            if constexpr (GROUPED && kRotateSteps) {
                if (steps_to_wrap == 0u) {
                    blocks_to_group = 0u;
                    next_group_blocks = (p.group_size - __builtin_amdgcn_readfirstlane(kb) % p.group_size) / 32u;
                }
                --steps_to_wrap;
            }
#pragma unroll
            for (int q = 0; q < KB; ++q) {
                if constexpr (GROUPED) {
                    // the scales change only where a group of rows begins: widen them there, not for every block
                    if (blocks_to_group == 0u) {
                        if constexpr (PACKED) {
                            // scale of column 4j + e goes to T[(4j + e) % 16][(4j + e) / 16]; lane (nl, kg) then reads row nl: its
                            // CPL scales, in column-block order.  The table is this wave's own; LDS serves a wave's requests in order.
                            if ((uint32_t)lane < kCols / 4u) {
                                const uint32_t d[2] = {st.sraw[q][0].x, st.sraw[q][0].y};
#pragma unroll
                                for (uint32_t e = 0; e < 4; ++e) {
                                    const uint32_t cix = 4u * (uint32_t)lane + e;
                                    sc_table[(cix & 15u) * CPL + (cix >> 4)] = (uint16_t)(e & 1u ? d[e >> 1] >> 16 : d[e >> 1] & 0xffffu);
                                }
                            }
                            uint4 mine[CPL / 8];
#pragma unroll
                            for (int i = 0; i < CPL / 8; ++i) mine[i] = *reinterpret_cast<const uint4*>(sc_table + (uint32_t)nl * CPL + 8u * i);
                            apply_scales<BITS, CPL>(cs, mine);
                        } else {
                            apply_scales<BITS, CPL>(cs, st.sraw[q]);
                        }
                        blocks_to_group = next_group_blocks;
                        next_group_blocks = p.group_size / 32u;
                    }
                    --blocks_to_group;
                }
                if constexpr (PACKED) mac_step_packed<BITS, CPL, MB>(st.raw[q], cs, st.af[q], acc);
                else mac_step<BITS, CPL, MB, REF>(st.raw[q], cs, st.af[q], acc, std::make_integer_sequence<int, CPL>{});
            }
        };
        auto request_scales = [&](Stage& st) {  // one scale per column: requested once, before the first weights
            if constexpr (REF) {
                const float4* sf = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.scale) + n_ld);
#pragma unroll
                for (int i = 0; i < CPL / 4; ++i) {
                    const float4 v = sf[i];
                    cs[4 * i] = v.x; cs[4 * i + 1] = v.y; cs[4 * i + 2] = v.z; cs[4 * i + 3] = v.w;
                }
            } else if constexpr (!GROUPED) {
                if constexpr (PACKED) load_scales_packed<CPL>(st.sraw[0], sptr, pk_col);
                else load_scales<CPL>(st.sraw[0], sptr, n_ld);
            }
        };
        if (nsteps > 0) {
            Stage s0, s1;
            request_scales(s0);
            load_stage(s0, 0);
            if constexpr (!GROUPED && !REF) apply_scales<BITS, CPL>(cs, s0.sraw[0]);
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
        if constexpr (!PACKED && !GROUPED) {
            if (tail_rows != 0u) {
                // the partial step: groups of 8 rows past the end of k get zero activations (and re-read the last 8 rows
                // of B, whose products with zero vanish)
                Stage st;
                if (nsteps == 0) {
                    request_scales(st);
                    if constexpr (!REF) apply_scales<BITS, CPL>(cs, st.sraw[0]);
                }
                const uint32_t krow = kb + 32u * (uint32_t)nsteps + 8u * (uint32_t)kg;
                const bool live = krow < p.k;
                load_raw<BITS, CPL>(st.raw[0], p.b + (size_t)(live ? krow : p.k - 8u) * p.ldb_bytes, n_ld * BITS / 8u, p.ldb_bytes);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    st.af[0][mb] = make_uint4(0u, 0u, 0u, 0u);
                    if (live) st.af[0][mb] = *reinterpret_cast<const uint4*>(aptr[mb] + (size_t)nsteps * 32);
                }
                compute_stage(st);
            }
        }
    }
    TRACE_MARK(2);

    // ---- add the waves' partial sums through LDS, kMBC blocks of 16 rows at a time (what fits): one barrier,
    //      then each thread finishes 4 neighbouring columns of some rows.  acc[mb][c][r] of lane (nl, kg) is
    //      row 16*mb + nl, local column (4*kg + r)*CPL + c.
    constexpr int kMBC = decode_rows16_per_pass(CPL, MB);
    constexpr uint32_t kQuads = kCols / 4u;
    constexpr uint32_t kMaxR = 16u * kMBC * kQuads / 256u;      // rows per thread and pass with 4 waves (half that with 8)
    // thread t: 4 consecutive columns (cg = t % (kCols/4)) of rows t / (kCols/4), + threads/(kCols/4), ...
    const uint32_t cg = threadIdx.x % kQuads, rs = threadIdx.x / kQuads, nrs = blockDim.x / kQuads;
    const uint32_t col = cb * kCols + 4u * cg;
    const bool col_ok = col < p.n;

#pragma unroll
    for (int mb0 = 0; mb0 < MB; mb0 += kMBC) {
        const uint32_t pass_row0 = 16u * mb0;  // within the row block
        if (pass_row0 >= rows_here) break;     // uniform over the workgroup
        const uint32_t rows_out = rows_here - pass_row0 < 16u * kMBC ? rows_here - pass_row0 : 16u * kMBC;
        if (mb0 > 0) __syncthreads();          // the previous pass's tiles have been read
#pragma unroll
        for (int mbi = 0; mbi < kMBC; ++mbi) {
            const int mb = mb0 + mbi;
            if (mb >= MB || !row_ok[mb]) continue;
            float* row = red + ((size_t)wave * rows_out + (mbi * 16 + nl)) * kRedStride;
            if constexpr (PACKED) {
#pragma unroll
                for (int c = 0; c < CPL; ++c)  // column block c, columns 4 kg .. 4 kg + 3 of it
                    *reinterpret_cast<float4*>(row + 16 * c + 4 * kg) = make_float4(acc[mb][c][0], acc[mb][c][1], acc[mb][c][2], acc[mb][c][3]);
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int c4 = 0; c4 < CPL / 4; ++c4) {
                        float4 v = make_float4(acc[mb][4 * c4 + 0][r], acc[mb][4 * c4 + 1][r], acc[mb][4 * c4 + 2][r],
                                               acc[mb][4 * c4 + 3][r]);
                        *reinterpret_cast<float4*>(row + (4 * kg + r) * CPL + 4 * c4) = v;
                    }
            }
        }
        __syncthreads();
        TRACE_MARK(3);

        float4 sum[kMaxR];
        // The waves' tiles are read with every load of a row in flight at once and added in wave order (wave 0 first:
        // the order is fixed).  Written for the two workgroup sizes there are, so that the loop over the waves is
        // unrolled: as a loop with a run-time bound it was a chain of 4 or 8 dependent LDS round trips, and this sum
        // sits between the end of the weight stream and the hand-over of the partial sums, where nothing hides it.
        auto add_waves = [&](auto waves_c) {
            constexpr uint32_t W = decltype(waves_c)::value;
#pragma unroll
            for (uint32_t i = 0; i < kMaxR; ++i) {
                const uint32_t row = rs + i * nrs;
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (row < rows_out) {
                    const float* src = red + (size_t)row * kRedStride + 4u * cg;
                    float4 v[W];
#pragma unroll
                    for (uint32_t w = 0; w < W; ++w) v[w] = *reinterpret_cast<const float4*>(src + (size_t)w * rows_out * kRedStride);
#pragma unroll
                    for (uint32_t w = 0; w < W; ++w) { t.x += v[w].x; t.y += v[w].y; t.z += v[w].z; t.w += v[w].w; }
                }
                sum[i] = t;
            }
        };
        if (nwaves == 8u) add_waves(std::integral_constant<uint32_t, 8>{});
        else add_waves(std::integral_constant<uint32_t, 4>{});
        const uint32_t first_row = row0 + pass_row0;  // global row of this pass's row 0
        if (p.splits == 1) {
#pragma unroll
            for (uint32_t i = 0; i < kMaxR; ++i) {
                const uint32_t row = rs + i * nrs;
                if (row < rows_out && col_ok) {
                    finish_row4(p, sum[i], first_row + row, col);
                }
            }
        } else if (ks != p.splits - 1u) {
            // ---- split-K.  The workspace holds one fp32 word per (split, row, column); at rest every word is
            // kEmptyWord, a NaN pattern no sum of products of bf16 numbers takes.  The workgroups of all splits
            // but the last write their sums there with device-scope (write-through) stores and are done: they
            // wait for nothing, not even the stores' acknowledgement.
            const __amdgpu_buffer_rsrc_t ws = __builtin_amdgcn_make_buffer_rsrc(p.partials, 0, (int)p.partial_bytes, kBufferFlags);
            const bool withhold = (p.debug_flags & kDebugWithholdPartials) != 0;  // test hook: lets the reducer's wait run out
#pragma unroll
            for (uint32_t i = 0; i < kMaxR; ++i) {
                const uint32_t row = rs + i * nrs;
                if (row < rows_out && col_ok && !withhold) {
                    const u32x4_t w4 = {__float_as_uint(sum[i].x), __float_as_uint(sum[i].y), __float_as_uint(sum[i].z), __float_as_uint(sum[i].w)};
                    __builtin_amdgcn_raw_buffer_store_b128(w4, ws, (int)(((first_row + row) * p.n + col) * 4u), (int)(ks * p.m * p.n * 4u), kAuxDeviceScope);
                }
            }
            TRACE_MARK(4);
        } else {
            // The workgroup of the LAST split (dispatched after the others) fetches the words with device-scope
            // loads, reads again whichever still shows kEmptyWord (a store in flight), adds them in split order
            // with its own sums last, writes C and puts kEmptyWord back for the next launch.  No counter, no
            // flag, no read-modify-write; only this workgroup ever waits, and only on workgroups that wait for
            // nothing, so the wait ends whatever order they run in.  It is bounded all the same: a word that
            // never arrives leaves a NaN in the output instead of hanging the kernel.
            // Rows a thread has in this pass: a power of two up to kMaxR; the fewer, the more splits are fetched at once.
            const uint32_t rows_per_thread = (rows_out + nrs - 1u) / nrs;
            constexpr bool kTwoAttempts = CPL == 8;  // (see reduce_splits_two_in_flight)
            if (kTwoAttempts && rows_per_thread <= 1u && p.splits <= 2u) reduce_splits_two_in_flight<1>(p, sum, first_row, rows_out, rs, col, col_ok);
            else if (kTwoAttempts && rows_per_thread <= 1u && p.splits <= 3u) reduce_splits_two_in_flight<2>(p, sum, first_row, rows_out, rs, col, col_ok);
            else if (kTwoAttempts && rows_per_thread <= 1u && p.splits <= 5u) reduce_splits_two_in_flight<4>(p, sum, first_row, rows_out, rs, col, col_ok);
            else if (kTwoAttempts && rows_per_thread <= 1u && p.splits <= 8u) reduce_splits_two_in_flight<7>(p, sum, first_row, rows_out, rs, col, col_ok);
            else if (rows_per_thread <= 1u) reduce_splits<1>(p, sum, first_row, rows_out, rs, nrs, col, col_ok);
            else if (rows_per_thread <= 2u) reduce_splits<(kMaxR < 2u ? kMaxR : 2u)>(p, sum, first_row, rows_out, rs, nrs, col, col_ok);
            else if (rows_per_thread <= 4u) reduce_splits<(kMaxR < 4u ? kMaxR : 4u)>(p, sum, first_row, rows_out, rs, nrs, col, col_ok);
            else reduce_splits<kMaxR>(p, sum, first_row, rows_out, rs, nrs, col, col_ok);
            TRACE_MARK(5);
        }
    }
}

template <int BITS, int CPL, int MB, bool GROUPED, bool PACKED, bool REF = false>
static hipError_t launch_decode_t(const GemmParams& p, hipStream_t stream)
{
    constexpr uint32_t kCols = 16u * CPL;
    constexpr uint32_t kRows = 16u * MB;
    const uint32_t waves = p.decode_waves;
    if ((MB > 2 || (PACKED && BITS == 4 && CPL == 16)) && waves != 4u) return hipErrorInvalidValue;  // kernels compiled for 256 threads
    const dim3 grid((p.n + kCols - 1u) / kCols, p.splits, (p.m + kRows - 1u) / kRows);
    if (grid.z > 65535u) return hipErrorInvalidValue;
    const uint32_t pass_rows = 16u * (uint32_t)decode_rows16_per_pass(CPL, MB);
    size_t lds = (size_t)decode_red_floats(waves, p.m < pass_rows ? p.m : pass_rows, kCols) * sizeof(float);
    GemmParams q = p;
    if (PACKED && GROUPED) {
        q.decode_scale_lds = (uint32_t)lds;     // each wave's 16 x CPL table of bf16 scales sits behind the reduction area
        lds += (size_t)waves * 16u * CPL * 2u;
    }
    if (lds > 160 * 1024 - 64) return hipErrorInvalidValue;
    void (*kernel)(const GemmParams) = bfaintb_decode_kernel<BITS, CPL, MB, GROUPED, PACKED, REF>;
    return launch_kernel(kernel, grid, dim3(64 * waves, 1, 1), lds, stream, q);
}

template <int BITS, int CPL, bool PACKED>
static hipError_t launch_decode_b(const GemmParams& p, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    switch (p.decode_mb) {
        case 1: return grouped ? launch_decode_t<BITS, CPL, 1, true, PACKED>(p, stream) : launch_decode_t<BITS, CPL, 1, false, PACKED>(p, stream);
        case 2: return grouped ? launch_decode_t<BITS, CPL, 2, true, PACKED>(p, stream) : launch_decode_t<BITS, CPL, 2, false, PACKED>(p, stream);
        case 4:  // 16 accumulators x 4 blocks x 8 columns = 128 registers: only the 128-column shape has room
            if constexpr (CPL == 8) return grouped ? launch_decode_t<BITS, CPL, 4, true, PACKED>(p, stream) : launch_decode_t<BITS, CPL, 4, false, PACKED>(p, stream);
            break;
        default: break;
    }
    return hipErrorInvalidValue;
}

// The reference's arithmetic: 8-bit codes, one fp32 scale per column.
template <int CPL>
static hipError_t launch_decode_ref(const GemmParams& p, hipStream_t stream)
{
    switch (p.decode_mb) {
        case 1: return launch_decode_t<8, CPL, 1, false, false, true>(p, stream);
        case 2: return launch_decode_t<8, CPL, 2, false, false, true>(p, stream);
        case 4:
            if constexpr (CPL == 8) return launch_decode_t<8, CPL, 4, false, false, true>(p, stream);
            break;
        default: break;
    }
    return hipErrorInvalidValue;
}

hipError_t launch_decode(const GemmParams& p, int bits, hipStream_t stream)
{
    if (p.reference_arith) {
        if (bits != 8 || p.group_size != 0) return hipErrorInvalidValue;
        return p.decode_cols == 128u ? launch_decode_ref<8>(p, stream) : launch_decode_ref<16>(p, stream);
    }
    if (bits == 8) return p.decode_cols == 128u ? launch_decode_b<8, 8, false>(p, stream) : launch_decode_b<8, 16, false>(p, stream);
    return p.decode_cols == 128u ? launch_decode_b<4, 8, false>(p, stream) : launch_decode_b<4, 16, false>(p, stream);
}

// The same family over weights in the packed order (p.b = the packed buffer): the shapes the plan uses beyond 32 rows of A,
// 128 columns for 8-bit and 256 for 4-bit codes.  n must hold at least one such group of column blocks.
hipError_t launch_decode_family_packed(const GemmParams& p, int bits, hipStream_t stream)
{
    if (bits == 8) return p.decode_cols == 128u ? launch_decode_b<8, 8, true>(p, stream) : hipErrorInvalidValue;
    return p.decode_cols == 128u ? launch_decode_b<4, 8, true>(p, stream) : launch_decode_b<4, 16, true>(p, stream);
}

// Allows every kernel of the family its largest dynamic LDS size on the current device.  Runs once per device, from the
// library's set-up (never from a launch: it is not a stream operation, and a launch may be under stream capture).
template <int BITS, int CPL, int MB, bool GROUPED, bool PACKED, bool REF = false>
static hipError_t allow_lds()
{
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&bfaintb_decode_kernel<BITS, CPL, MB, GROUPED, PACKED, REF>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
}

template <int BITS, int CPL, bool PACKED>
static hipError_t allow_lds_b()
{
    hipError_t e = allow_lds<BITS, CPL, 1, false, PACKED>();
    if (e == hipSuccess) e = allow_lds<BITS, CPL, 1, true, PACKED>();
    if (e == hipSuccess) e = allow_lds<BITS, CPL, 2, false, PACKED>();
    if (e == hipSuccess) e = allow_lds<BITS, CPL, 2, true, PACKED>();
    if constexpr (CPL == 8) {
        if (e == hipSuccess) e = allow_lds<BITS, CPL, 4, false, PACKED>();
        if (e == hipSuccess) e = allow_lds<BITS, CPL, 4, true, PACKED>();
    }
    return e;
}

hipError_t decode_prepare_device()
{
    hipError_t e = allow_lds_b<8, 8, false>();
    if (e == hipSuccess) e = allow_lds_b<8, 16, false>();
    if (e == hipSuccess) e = allow_lds_b<4, 16, false>();
    if (e == hipSuccess) e = allow_lds_b<8, 8, true>();
    if (e == hipSuccess) e = allow_lds_b<4, 16, true>();
    if (e == hipSuccess) e = allow_lds<8, 8, 1, false, false, true>();
    if (e == hipSuccess) e = allow_lds<8, 8, 2, false, false, true>();
    if (e == hipSuccess) e = allow_lds<8, 8, 4, false, false, true>();
    if (e == hipSuccess) e = allow_lds<8, 16, 1, false, false, true>();
    if (e == hipSuccess) e = allow_lds<8, 16, 2, false, false, true>();
    return e;
}

}  // namespace bfaintb
