// Device-side building blocks shared by every bfAintBGemm kernel for gfx950.
//
// The arithmetic restated here is the reference kernel's dequantisation
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:18-55): integer code -> fp32, times the
// column's scale, narrowed to bf16.  Differences by contract: scales are bf16 (so the product is
// exact in fp32), the narrowing rounds to nearest even (v_cvt_pk_bf16_f32) instead of truncating,
// and 4-bit codes exist.  GemmParams.reference_arith selects the reference's own arithmetic instead
// (fp32 scales, truncation) in the kernels that read row-major 8-bit weights with one scale per column.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <tuple>
#include <utility>

namespace bfaintb {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kBufferFlags = 0x00027000;  // buffer resource word 3: raw buffer, 32-bit data format
// Cache-policy operand of the raw buffer load/store builtins: device scope (sc1: the store writes through to
// where every XCD sees it, the load does not settle for a stale local copy).
constexpr int kAuxDeviceScope = 16;

// Epilogue activations (values of bfaintb_epilogue.activation).
constexpr uint32_t kActNone = 0, kActSiluGate = 1;

// silu(g) * u in fp32: g / (1 + exp(-g)) * u.  exp through the hardware's base-2 exponential, the quotient through its
// reciprocal: a few units in the last place of fp32, far below the bf16 rounding that follows.  g -> -inf gives -0 * u.
__device__ __forceinline__ float silu_gate(float g, float u)
{
    return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}

// A split-K workspace word that holds no partial sum: an all-ones NaN.  Sums of products of bf16 numbers
// are never this pattern (NaNs born in the arithmetic are the default quiet NaN; NaNs carried over from
// bf16 inputs have zero low bits).
constexpr uint32_t kEmptyWord = 0xffffffffu;

// The first 256 bytes of a split-K workspace are its header; the partial sums follow.
//   word 0  sticky failure mark: kEmptyWord while all is well, kWorkspaceGaveUp once a reducing workgroup has given up
//           waiting for a partial sum (the workspace may then hold words at rest that are not empty: initialise it again)
//   word 1  kWorkspaceMagic, written by the initialisation: tells an initialised workspace from arbitrary memory
// The GEMM kernels never read the header; bfaintb_workspace_status does, on the host.
constexpr uint32_t kWorkspaceHeaderBytes = 256;
constexpr uint32_t kWorkspaceGaveUp = 0x0bad0badu;
constexpr uint32_t kWorkspaceMagic = 0x42464157u;  // "BFAW"
constexpr uint32_t kDefaultSplitWaitLimit = 1u << 18;  // re-reads of a split-K word before giving up (each a memory round trip)
constexpr uint32_t kDebugWithholdPartials = 1u;        // GemmParams.debug_flags: producers keep their sums to themselves

template <typename Tuple, size_t... I>
inline void fill_argv(void** argv, Tuple& t, std::index_sequence<I...>)
{
    ((argv[I] = const_cast<void*>(static_cast<const void*>(&std::get<I>(t)))), ...);
}

// Decode variant: blocks of 32 rows of k a wave loads per pipeline step (cpl = weights per lane and
// row).  Row-major weights: one; two blocks for the 8-byte-per-row layouts measured no faster (more bytes in
// flight per wave, fewer waves per CU).  Packed weights: a lane's whole 16-byte share of a K-chunk with one load where the
// registers allow it — two blocks (a 64-row chunk) for 8-bit codes, four (a 128-row chunk) for 4-bit codes in the
// 128-column form with one or two blocks of 16 rows of A.  Half a share per load (8 bytes at a stride of 16) touches
// every line of the chunk twice, a step apart, and the second touch misses in cache: 40 % more bytes fetched than the
// matrix holds (32000 x 4096, m = 16, counted) and 30 - 60 % longer launches where it was tried for 8-bit codes.  Packed
// 4-bit codes with four row blocks, or in the 256-column form, have no registers for four blocks per stage and stay at
// two (two row blocks fit with the slab bases in scalar registers: 7 registers spilled with grouped scales, and still
// 9 - 14 % faster on matrices from 32 MiB).
__host__ __device__ constexpr int decode_blocks_per_step(int bits, int cpl, bool packed, int mb)
{
    return packed ? (bits == 4 && cpl == 8 && mb <= 2 ? 4 : 2) : 1;
}

struct GemmParams {
    uint16_t* c;
    const uint16_t* a;
    const uint8_t* b;
    const uint16_t* scale;  // bf16 scales; with reference_arith: fp32 scales, one per column
    const uint16_t* bias;  // bf16 [n] added to the fp32 sums before the one rounding to bf16, or null
    const uint16_t* residual;  // bf16 [m, ldr] added after the bias, before the rounding, or null
    uint32_t ldr;              // elements per row of residual
    uint32_t reference_arith;  // non-zero: the reference kernel's arithmetic — fp32 per-column scales, W and C narrowed by
                               // truncation (8-bit codes, row-major B, no groups); zero: bf16 scales, round to nearest even
    uint32_t activation;       // kActNone, or kActSiluGate: columns (2j, 2j+1) of the sums are (gate, up) of output column j
    uint32_t m, n, k;
    uint32_t lda;        // elements
    uint32_t ldb_bytes;  // bytes per row of packed weights
    uint32_t ldc;        // elements
    uint32_t lds;        // elements per scale row (= n)
    uint32_t group_size; // rows of k per scale group; 0 = one group
    // the division of a block index (row / 32) by group_size / 32 as a multiplication: see set_group_division()
    uint32_t group_div_magic, group_div_shift1, group_div_shift2;
    // prefill variant: the logical 256x256 tiles one launch covers
    uint32_t tile_first, tile_count;
    uint32_t cus;        // compute units the launch plan is made for (host side only)
    // split-K (decode variant only)
    uint32_t k_per_wg;   // rows of k one workgroup covers (multiple of 32 * decode_blocks_per_step * decode_waves)
    uint32_t decode_waves; // waves per workgroup of the decode variant (4 or 8)
    uint32_t decode_cols;  // columns per workgroup of the decode variant (256, or 128 for 8-bit codes)
    uint32_t decode_mb;    // blocks of 16 rows of A per workgroup of the decode variant (1, 2 or 4)
    uint32_t decode_scale_lds;  // byte offset, in dynamic LDS, of the waves' scale tables (packed weights, grouped scales)
    uint32_t splits;     // workgroups along k
    unsigned long long* partials;  // [splits - 1][m][n] fp32 partial sums; kEmptyWord wherever none is waiting
    uint32_t partial_bytes;        // size of that area (below 2^31)
    uint32_t* ws_header;           // the workspace's header (see kWorkspaceHeaderBytes), or null without split-K
    uint32_t split_wait_limit;     // fetch attempts of the reducing workgroup before it gives up
    uint32_t debug_flags;          // kDebug* (test hooks; zero in normal operation)
#ifdef BFAINTB_TRACE
    unsigned long long* trace;  // timestamp sink (instrumented builds only)
#endif
};

// The scale group of a row of B.  The kernels ask for it per block of 32 rows inside their inner loops, where a division
// by the run-time group size (some 25 dependent scalar instructions) stalls the one wave of a SIMD for longer than a
// matrix instruction runs: 128x128 tiles, groups of 128 rows, 640 x 4096 x 4096: 41.5 us with the division, 36.8 without.
// So the host turns the divisor d = group_size / 32 into a multiplier (Granlund and Montgomery's round-up method, exact
// for every 32-bit dividend): l = ceil(log2 d), magic = floor(2^32 (2^l - d) / d) + 1, and then
// n / d = (t + ((n - t) >> min(l, 1))) >> max(l - 1, 0) with t = the high half of magic x n.
inline void set_group_division(GemmParams& p)
{
    const uint32_t d = p.group_size / 32u;
    if (d == 0u) {
        p.group_div_magic = 1u, p.group_div_shift1 = 0u, p.group_div_shift2 = 0u;  // (no groups: never asked)
        return;
    }
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    p.group_div_magic = (uint32_t)((((1ull << l) - d) << 32) / d) + 1u;
    p.group_div_shift1 = l < 1u ? l : 1u;
    p.group_div_shift2 = l > 1u ? l - 1u : 0u;
}
__device__ __forceinline__ uint32_t group_of_row(const GemmParams& p, uint32_t row)
{
    const uint32_t n = row >> 5;
    const uint32_t t = __umulhi(p.group_div_magic, n);
    return (t + ((n - t) >> p.group_div_shift1)) >> p.group_div_shift2;
}

// 256x256 tiles: how many of them, at the end, run as a second launch of half tiles.  Tiles beyond whole rounds of one
// workgroup per CU, when they would fill at most half of the CUs (and every launch with fewer tiles than that), run as
// twice as many workgroups of half the size.
inline uint32_t thin_round_tiles(uint32_t tiles, uint32_t m, uint32_t cus)
{
    const uint32_t rest = tiles % cus;
    return (rest != 0u && rest <= cus / 2u && m > 128u) ? rest : 0u;
}

// Launch through hipLaunchKernel so that the error returned belongs to THIS launch:
// hipGetLastError() would also hand back whatever an earlier, unrelated runtime call left behind.
template <typename... Params, typename... Args>
inline hipError_t launch_kernel(void (*kernel)(Params...), dim3 grid, dim3 block, size_t dyn_lds, hipStream_t stream, Args... args)
{
    static_assert(sizeof...(Params) == sizeof...(Args), "argument count");
    std::tuple<Params...> pack{static_cast<Params>(args)...};
    void* argv[sizeof...(Params)];
    fill_argv(argv, pack, std::index_sequence_for<Params...>{});
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, argv, dyn_lds, stream);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// Two fp32 -> one dword of two bf16 (lo in bits 15:0), round to nearest even.
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi)
{
    bf16x2_t v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}

// Two fp32 -> one dword of two bf16 by truncation (the high halves of the two words): how the reference kernel narrows,
// both where it forms W (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:29-35, v_pack_b32_f16 with op_sel:[1,1])
// and where it stores C (.s:597-611, ds_write_b16_d16_hi).
__device__ __forceinline__ uint32_t pack_bf16_rtz(float lo, float hi)
{
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);  // bytes {lo.2, lo.3, hi.2, hi.3}
}

// RTZ = the reference kernel's arithmetic (fp32 scales, truncation), else this library's contract (round to nearest even).
template <bool RTZ>
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    if constexpr (RTZ) return pack_bf16_rtz(lo, hi);
    else return pack_bf16_rne(lo, hi);
}

// Signed byte `I` of a dword as fp32: one v_cvt_f32_i32 with an SDWA sign-extending byte select.
template <int I>
__device__ __forceinline__ float sbyte_to_f32(uint32_t x)
{
    if constexpr (I == 3) return (float)((int32_t)x >> 24);
    return (float)(int32_t)(int8_t)((x >> (8 * I)) & 0xffu);
}

// Stored codes -> two's complement bytes the conversion above can read.
//   8-bit: excess-128 byte u = q + 128; u ^ 0x80 is q as int8.
//   4-bit: excess-8 nibble c = q + 8; c ^ 8 is q as int4; moved to the HIGH nibble of a byte it reads
//          as the int8 value 16*q, and the column's scale is pre-divided by 16 (exact: a power of two).
__device__ __forceinline__ uint32_t codes8_to_s8(uint32_t x) { return x ^ 0x80808080u; }
// Both halves of a dword of eight codes: the even codes move up into their bytes' high nibbles; each half is then one
// three-input bit operation (mask the high nibbles, flip every code's top bit): 3 operations for the dword.
__device__ __forceinline__ void codes4_to_s8x16(uint32_t x, uint32_t& even, uint32_t& odd)
{
    even = ((x << 4) & 0xf0f0f0f0u) ^ 0x80808080u;
    odd = (x & 0xf0f0f0f0u) ^ 0x80808080u;
}

// The same eight codes for the conversion instruction that reads a nibble directly (v_cvt_off_f32_i4: bits 3:0 of its
// source as a two's-complement value, divided by 16 — exact): flip every code's top bit, and shift the odd codes down to
// the low nibbles of their bytes.  2 operations for the dword; the bits above a nibble are ignored by the instruction.
__device__ __forceinline__ void codes4_to_nibbles(uint32_t x, uint32_t& even, uint32_t& odd)
{
    even = x ^ 0x88888888u;
    odd = even >> 4;
    asm("" : "+v"(odd));  // keep the shifted dword: its bytes are then picked by the conversion's own byte select
}
// q / 16 of the code in the low nibble of byte I
template <int I>
__device__ __forceinline__ float nibble_to_f32_sixteenth(uint32_t x)
{
    if constexpr (I == 0) return __builtin_amdgcn_cvt_off_f32_i4((int)x);
    return __builtin_amdgcn_cvt_off_f32_i4((int)((x >> (8 * I)) & 0xffu));
}
// The multiplier that goes with it: 16 x scale (exact; a scale of 2^124 or more would overflow here, one that small
// that scale / 16 is not exact would lose bits in make_col_scale below: neither occurs in quantised weights).
template <int BITS>
__device__ __forceinline__ float make_col_scale_nibble(uint32_t scale_bf16_bits)
{
    const float s = bf16_bits_to_f32(scale_bf16_bits);
    return BITS == 8 ? s : s * 16.0f;
}

// 16 bits holding four consecutive 4-bit codes (column j in nibble j) -> dword whose byte j reads as int8(16*q_j).
// Byte 0 of (x << 4) is code 0 in the high nibble over zeros; byte 0 of x has code 1 in its high nibble, byte 1 of
// (x << 4) code 2, byte 1 of x code 3: one byte permute gathers them, one three-input bit operation clears the low
// nibbles and flips each code's top bit (excess-8 -> two's complement).
__device__ __forceinline__ uint32_t codes4_quad_to_s8x16(uint32_t x)
{
    const uint32_t mixed = __builtin_amdgcn_perm(x << 4, x, 0x01050004u);  // bytes {(x<<4).0, x.0, (x<<4).1, x.1}
    return (mixed & 0xf0f0f0f0u) ^ 0x80808080u;
}

// A column's multiplier: the bf16 scale widened to fp32 (times 1/16 for 4-bit codes, see above).
// w = value * multiplier is one IEEE fp32 multiply of float(q) (or float(16 q)) by it — exact for a
// bf16 scale (8 x 8 significant bits), with the sign of zero of a true product — and is then
// rounded once to bf16.
template <int BITS>
__device__ __forceinline__ float make_col_scale(uint32_t scale_bf16_bits)
{
    const float s = bf16_bits_to_f32(scale_bf16_bits);
    return BITS == 8 ? s : s * 0.0625f;
}

// A workgroup barrier without the memory fence that __syncthreads() carries.  That fence makes the compiler wait, before
// the barrier, for EVERY asynchronous global -> LDS copy issued so far — also the ones meant to land steps later — which
// turns a pipeline of several stages into one of a single stage.  The caller states what must have completed with
// explicit wait counts (its own part of the stage the others are about to read: s_waitcnt vmcnt; its LDS reads of the
// stage about to be overwritten were consumed by matrix instructions it has already issued); the empty assembly
// statements keep the compiler from moving memory operations across the barrier.
__device__ __forceinline__ void barrier_no_fence()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

}  // namespace bfaintb
