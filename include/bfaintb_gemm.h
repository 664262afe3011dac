/*
 * bfaintb_gemm.h — C ABI of the MI355X (gfx950) bf16-activation x integer-weight GEMM.
 *
 *     C[m,n] = sum_k A[m,k] * W[k,n],      W[k,n] = bf16( float(q[k,n]) * float(scale[g(k),n]) )
 *
 * A, C: bf16, row-major.  B: packed integer codes q, row-major K x N.  fp32 accumulation, one
 * rounding (to nearest even) when W is formed and one when C is stored.
 *
 * The entry points replace the raw module launch of the reference driver
 * (/root/reference/bfAintBGemm/bfAintBGemm.cc:65-66 hipModuleLoad/hipModuleGetFunction and
 * :119-152 packed kernarg + hipModuleLaunchKernel).  The argument order of bfaintb_gemm is that
 * kernarg block — {c, a, b, scale, m, n, k, lda, ldb, ldc} (bfAintBGemm.cc:119-133, kernel side
 * bf16gemm_kernel_gfx90a.s:97-108) — followed by what the reference did not have.
 *
 * All pointers are DEVICE pointers owned by the caller.  Calls are asynchronous and ordered on
 * `stream` (a hipStream_t passed as void*; NULL is the default stream, which is what the reference
 * launches on).  No call allocates or frees; only bfaintb_init and bfaintb_workspace_status wait for the
 * device.  Return value: 0 on success, a negative BFAINTB_ERR_* for a rejected argument (nothing was
 * launched), or a positive hipError_t.
 *
 * The first GEMM call on a device prepares the library's kernels there (a few runtime calls that are not
 * stream operations).  A caller whose first call would come under stream capture runs bfaintb_init before.
 */
#ifndef BFAINTB_GEMM_H
#define BFAINTB_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define BFAINTB_API __attribute__((visibility("default")))
#else
#define BFAINTB_API
#endif

#define BFAINTB_VERSION 200 /* major*10000 + minor*100 + patch */

enum {
    BFAINTB_OK = 0,
    BFAINTB_ERR_NULL_POINTER = -1,  /* c, a, b or scale is NULL (with m,n,k all non-zero) */
    BFAINTB_ERR_BAD_SHAPE = -2,     /* n not a multiple of 8 (16 for 4-bit codes), k not a multiple of 8, or sizes overflow 2^31 */
    BFAINTB_ERR_BAD_LD = -3,        /* lda < k, ldb < n, ldb >= 2^27, ldc < n, or a leading dimension that breaks 16-byte rows */
    BFAINTB_ERR_ALIGNMENT = -4,     /* a pointer is not 16-byte aligned */
    BFAINTB_ERR_UNSUPPORTED = -5,   /* weight_bits not 8 or 4; group_size not 0 or a multiple of 32 dividing k */
    BFAINTB_ERR_WORKSPACE = -6,     /* workspace NULL/too small for this shape (see bfaintb_gemm_workspace_bytes) */
    BFAINTB_ERR_BAD_VARIANT = -7,   /* unknown variant, or a variant that cannot run this shape */
    BFAINTB_ERR_NOT_INITIALISED = -8,     /* the first call on a device came under stream capture: call bfaintb_init before */
    BFAINTB_ERR_WORKSPACE_POISONED = -9,  /* bfaintb_workspace_status: a split-K wait gave up on this workspace */
    BFAINTB_ERR_STATIC_SCRATCH = -10      /* bfaintb_gemm_static: the shape needs more scratch than the library holds */
};

/* Which kernel family runs a shape. */
enum {
    BFAINTB_VARIANT_AUTO = 0,   /* decode up to m = 32; beyond, whichever the library estimates faster for (m, n, k) */
    BFAINTB_VARIANT_DECODE = 1, /* split-K weight-streaming kernel (HBM-bound); m > 32 in row blocks; accepts m <= 32768 */
    BFAINTB_VARIANT_PREFILL = 2, /* LDS-tiled MFMA kernels (MFMA-bound): 256x256 tiles, or 128x128 tiles while m x n
                                  * holds at most 256 of those (the large tiles would leave most CUs idle); while even
                                  * the small tiles leave CUs idle, their kernel splits k between workgroups (same
                                  * workspace and hand-over as the decode family's split-K) */
    BFAINTB_VARIANT_PREFILL_256 = 3, /* the tiled kernel with 256x256 tiles, whatever the shape (tests, tuning) */
    BFAINTB_VARIANT_PREFILL_128 = 4, /* the tiled kernel with 128x128 tiles, whatever the shape (tests, tuning).  Its fp32
                                      * sums are those of two chains of matrix instructions added at the end (even and odd
                                      * blocks of 32 k), so it agrees with the other tiled forms to rounding, not in
                                      * every bit; like every form it gives the same bits on every run */
    BFAINTB_VARIANT_PREFILL_256_LDS = 5, /* 256x256 tiles with both operands staged in LDS — the older form, which the
                                          * reference's arithmetic and the half tiles of a thin last round still use;
                                          * otherwise the form that keeps the weights in registers runs (tests, tuning) */
    BFAINTB_VARIANT_PREFILL_128_LDS = 6, /* 128x128 tiles with both operands staged in LDS — the older form, kept for the
                                          * reference's arithmetic; otherwise the form that keeps the weights in
                                          * registers runs (tests, tuning) */
    BFAINTB_VARIANT_PREFILL_256X128 = 7  /* tiles of 256 rows x 128 columns, weights in registers (this library's
                                          * arithmetic), whatever the shape (tests, tuning): what PREFILL runs
                                          * where 128x128 tiles would need a second round and 256x256 tiles leave CUs idle */
};

/*
 * Data formats.
 *   a      bf16 [m, lda], lda in elements (bfAintBGemm.cc:47,119-133; the kernel doubles it, asm:216).
 *   b      weight_bits == 8: one byte per weight, [k, ldb] bytes, excess-128 code u = q + 128 — the
 *          byte format the reference's host writes (mem_transfer.hpp:30) and its kernel decodes
 *          (bf16gemm_kernel_gfx90a.s:19-27).
 *          weight_bits == 4: two weights per byte along n, row stride ldb/2 bytes; byte j of a row
 *          holds column 2j in its low nibble and column 2j+1 in its high nibble, each excess-8
 *          (q + 8).  ldb is in ELEMENTS in both cases, like the reference's ldb.
 *   scale  bf16 [groups, n] with row stride n, groups = group_size ? k / group_size : 1.
 *          (The reference stores fp32 scales, bfAintBGemm.cc:27; this build's contract is bf16,
 *          which makes q*scale exact in fp32 and the dequantised weight a single rounding.)
 *   c      bf16 [m, ldc].
 * Requirements: n % 8 == 0 (n % 16 == 0 for 4-bit codes), k % 8 == 0 (the reference kernel needs n % 64 == 0 and
 * k % 64 == 0, bf16gemm_kernel_gfx90a.s:341-343, :402-408), lda % 8 == 0, ldb % 16 == 0, ldb < 2^27, ldc % 8 == 0,
 * all four pointers 16-byte aligned, |scale| finite and below 2^120.  Pre-packed weights (below) keep whole chunks:
 * n % 16 == 0 and k % 64 == 0 (k % 128 == 0 for 4-bit codes).
 */

/*
 * The GEMM.  Replaces hipModuleLaunchKernel(kernel_func, ...) at bfAintBGemm.cc:152 and :176.
 *   weight_bits   8 or 4
 *   group_size    0: one scale per output channel (the reference's only mode);
 *                 otherwise rows per scale group along k (multiple of 32, divides k)
 *   workspace     device scratch of at least bfaintb_gemm_workspace_bytes(...) bytes that has been
 *                 passed through bfaintb_workspace_init once.
 *                 The call leaves it in that state again, ready for the next call of any shape.
 *                 Two calls that may run concurrently must not share a workspace.  May be NULL
 *                 when the required size is 0.
 */
BFAINTB_API int bfaintb_gemm(void* c, const void* a, const void* b, const void* scale, uint32_t m, uint32_t n, uint32_t k,
                 uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                 size_t workspace_bytes, void* stream);

/* Same, with the kernel family and the split-K factor forced (0 = choose, 1 = none).  For benchmarks and tests.
 * split_k applies to the decode family and to the 128x128-tile kernel over row-major weights (at most 16 splits there,
 * each of whole 64-row steps of k); the 256x256 tiles, the forms with both operands in LDS and the reference
 * arithmetic run unsplit whatever it says. */
BFAINTB_API int bfaintb_gemm_ex(void* c, const void* a, const void* b, const void* scale, uint32_t m, uint32_t n, uint32_t k,
                    uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                    size_t workspace_bytes, void* stream, int variant, uint32_t split_k);

/*
 * The GEMM with a fused bias: C[m,n] = bf16_rne(sum_k A[m,k]*W[k,n] + bias[n]), the bias (bf16 [n], 16-byte
 * aligned) added to the fp32 sum before the one rounding.  bias == NULL is bfaintb_gemm.  No counterpart in the
 * reference, whose kernel stores the sums as they are (bf16gemm_kernel_gfx90a.s:594-630); it is the first of the
 * epilogues a linear layer wants (the reference's stated purpose, README.md:2).  Same workspace as bfaintb_gemm.
 */
BFAINTB_API int bfaintb_gemm_bias(void* c, const void* a, const void* b, const void* scale, const void* bias, uint32_t m,
                      uint32_t n, uint32_t k, uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * The GEMM with a fused epilogue, described by a struct so that it can grow:
 *     activation == BFAINTB_ACT_NONE:
 *         C[m,n] = bf16_rne( sum_k A[m,k]*W[k,n]  + bias[n]  + residual[m,n] )
 *     activation == BFAINTB_ACT_SILU_GATE (the gated MLP of LLaMA-style models: gate and up projections in one GEMM):
 *         S[m,c] = sum_k A[m,k]*W[k,c] + bias[c]          for the n columns of B, scale and bias, where column 2j is
 *                                                         "gate" and column 2j+1 is "up" of output column j;
 *         C[m,j] = bf16_rne( silu(S[m,2j]) * S[m,2j+1] + residual[m,j] ),   silu(x) = x / (1 + exp(-x)),   j < n/2
 *         (C and residual have n/2 columns: ldc, ldr >= n/2).
 * Each term that is present is added in fp32, in this order, before the one rounding.  bias: bf16 [n]; residual: bf16
 * [m, ldr] (ldr in elements, a multiple of 8); both 16-byte aligned; either may be NULL; epilogue == NULL is
 * bfaintb_gemm.  The reference kernel stores the bare sums (bf16gemm_kernel_gfx90a.s:594-630);
 * these are the first epilogues of the reference's stated purpose, "gemm fusion for llm" (README.md:2): a linear layer's
 * bias and a transformer block's residual connection, without a second pass over C.  The residual may alias c when
 * ldr == ldc (every element is read by the thread that then writes it).
 */
typedef struct bfaintb_epilogue {
    const void* bias;
    const void* residual;
    uint32_t ldr;
    uint32_t activation; /* BFAINTB_ACT_* */
} bfaintb_epilogue;
#define BFAINTB_ACT_NONE 0u
#define BFAINTB_ACT_SILU_GATE 1u
BFAINTB_API int bfaintb_gemm_fused(void* c, const void* a, const void* b, const void* scale, const bfaintb_epilogue* epilogue, uint32_t m,
                       uint32_t n, uint32_t k, uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size,
                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * The reference kernel's launch, argument for argument, with the reference kernel's own arithmetic: for a caller that
 * keeps the reference's buffers exactly as they are.  The arguments are the kernarg block of bfAintBGemm.cc:119-133
 * (c, a, b, scale, m, n, k, lda, ldb, ldc); scale is fp32 [n] (ScaleDataType = float, bfAintBGemm.cc:27), not bf16;
 *     W[k,n] = truncate_to_bf16( float(q[k,n]) * scale[n] )      (bf16gemm_kernel_gfx90a.s:18-55: fp32 product, the
 *                                                                 high halves kept by v_pack_b32_f16 op_sel:[1,1])
 *     C[m,n] = truncate_to_bf16( sum_k A[m,k] * W[k,n] )         (fp32 accumulation; the store keeps the high halves,
 *                                                                 .s:597-611, "rtz mode")
 * 8-bit excess-128 codes with one scale per column: the reference's only format.  Same kernels, variant choice,
 * workspace (bfaintb_gemm_workspace_bytes(m, n, k, 8, 0)) and stream semantics as bfaintb_gemm; the order in which the
 * fp32 sums are formed differs from the reference kernel's (as it does between any two tilings), so results agree with
 * it to the last bit only where the sums are exact — as in the reference's own test data (random_gen.hpp:24,37,50) —
 * and otherwise to one bf16 unit.  scale must be 16-byte aligned.
 */
BFAINTB_API int bfaintb_gemm_reference(void* c, const void* a, const void* b, const float* scale, uint32_t m, uint32_t n, uint32_t k,
                           uint32_t lda, uint32_t ldb, uint32_t ldc, void* workspace, size_t workspace_bytes, void* stream);
/* Same with the variant and split factor forced, as bfaintb_gemm_ex. */
BFAINTB_API int bfaintb_gemm_reference_ex(void* c, const void* a, const void* b, const float* scale, uint32_t m, uint32_t n, uint32_t k,
                              uint32_t lda, uint32_t ldb, uint32_t ldc, void* workspace, size_t workspace_bytes, void* stream,
                              int variant, uint32_t split_k);

/* Scratch the GEMM needs for a shape: a 256-byte header, then one fp32 word per (split but the last, row,
 * column) of the split-K partial sums, rounded up to 256 bytes; 0 when the shape runs without split-K.  Depends only
 * on its arguments.  The reference kernel has no scratch (no split-K, bfAintBGemm.cc:107-109). */
BFAINTB_API size_t bfaintb_gemm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size);
BFAINTB_API size_t bfaintb_gemm_workspace_bytes_ex(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size,
                                       int variant, uint32_t split_k);

/* Prepares a freshly allocated workspace: marks every word "no partial sum here" (all bits set) and writes the
 * 256-byte header the sizes above include.  Stream-ordered, graph-capturable; workspace_bytes a multiple of 4, at least 256. */
BFAINTB_API int bfaintb_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/*
 * Health of a workspace, read back from its header (waits for `stream`): BFAINTB_OK; BFAINTB_ERR_WORKSPACE when the
 * memory was never passed through bfaintb_workspace_init; BFAINTB_ERR_WORKSPACE_POISONED when a reducing workgroup
 * gave up waiting for a partial sum (after 2^18 fetch attempts, about a tenth of a second: the workgroups it waits
 * for wait for nothing themselves, so this means a launch was lost or two overlapping calls shared the workspace).
 * The output of that call holds NaNs where the sums were incomplete, and the workspace may hold stray partial sums:
 * initialise it again before further use.  The mark is sticky until then.  No counterpart in the reference (no
 * split-K there, bfAintBGemm.cc:107-109).
 */
BFAINTB_API int bfaintb_workspace_status(const void* workspace, void* stream);

/*
 * Prepares the library on the current device — kernel attributes, and the scratch of bfaintb_gemm_static filled with
 * its at-rest pattern on `stream` — and waits for that.  Optional: the first GEMM call on a device does the same by
 * itself, except under stream capture, where it returns BFAINTB_ERR_NOT_INITIALISED instead.  Call it outside any
 * capture, once per device (further calls return at once).  Stands where the reference's main() loads its code object
 * (bfAintBGemm.cc:63-66: hipSetDevice, hipModuleLoad, hipModuleGetFunction).
 */
BFAINTB_API int bfaintb_init(void* stream);

/*
 * The GEMM for callers that cannot allocate or carry a workspace — code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  bfaintb_gemm without the workspace arguments: the split-K partial sums go to a
 * scratch array the library holds in device memory, one per GPU, 16 MiB (bfaintb_gemm_static_scratch_bytes), kept
 * until the process ends.  Same kernels, same variant choice and bit-for-bit the results of bfaintb_gemm.  A shape
 * whose bfaintb_gemm_workspace_bytes exceeds the scratch is refused with BFAINTB_ERR_STATIC_SCRATCH (nothing launched).
 * Every call on a GPU shares that GPU's scratch (each call leaves it in its at-rest state for the next): calls that may
 * overlap on one GPU — different streams, different host threads — race on it and must use bfaintb_gemm with
 * workspaces of their own.  Allocates nothing, on any call.  No counterpart in the reference, whose kernel needs no
 * scratch (no split-K).
 */
BFAINTB_API int bfaintb_gemm_static(void* c, const void* a, const void* b, const void* scale, uint32_t m, uint32_t n, uint32_t k,
                        uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* stream);
BFAINTB_API size_t bfaintb_gemm_static_scratch_bytes(void);
/*
 * bfaintb_workspace_status and bfaintb_workspace_init for that scratch, whose address the library keeps to itself.
 * _status (a synchronising query, like bfaintb_workspace_status) answers BFAINTB_OK, or BFAINTB_ERR_WORKSPACE_POISONED
 * once a split-K wait has given up on the current device's scratch — two overlapping bfaintb_gemm_static calls on one
 * GPU are the likely cause — after which later static calls on that GPU may take a stale partial sum for a fresh one.
 * _reset puts the scratch back into its at-rest state on `stream` (a fill kernel, asynchronous; after bfaintb_init it
 * may be recorded into a HIP graph); the caller makes sure that no bfaintb_gemm_static call on that GPU is in flight
 * or follows on another stream before the reset has run.  Both allocate nothing.  No counterpart in the reference.
 */
BFAINTB_API int bfaintb_static_scratch_status(void* stream);
BFAINTB_API int bfaintb_static_scratch_reset(void* stream);

/*
 * Test hooks (no effect on results in normal operation; process-wide, read by each following launch).  The first two
 * change what split-K launches do and are for the library's own tests: they are refused with BFAINTB_ERR_UNSUPPORTED
 * unless the process has BFAINTB_TEST_HOOKS=1 in its environment.
 *   BFAINTB_DEBUG_SPLIT_WAIT_LIMIT   value = fetch attempts a reducing workgroup makes before it gives up (0 restores 2^18)
 *   BFAINTB_DEBUG_WITHHOLD_PARTIALS  value != 0: the workgroups of all splits but the last compute and then keep their
 *                                    sums to themselves, so the reducer's wait runs out — the way to exercise the
 *                                    give-up path with every kernel exiting normally
 *   BFAINTB_DEBUG_FORCE_ROW_BLOCK    value = 1, 2 or 4: beyond 32 rows of A the decode family runs blocks of 16 x value rows
 *                                    whatever its estimates say (tuning; results do not depend on it); 0 restores the choice
 *   BFAINTB_DEBUG_PLAN_COMPUTE_UNITS value = the number of compute units the launch plans are made for instead of the
 *                                    device's own (tuning, partitioned devices; every plan is a correct launch on any
 *                                    device; workspace sizes follow the plan, so set it before asking for them);
 *                                    0 restores the device's count
 */
#define BFAINTB_DEBUG_SPLIT_WAIT_LIMIT 1u
#define BFAINTB_DEBUG_WITHHOLD_PARTIALS 2u
#define BFAINTB_DEBUG_FORCE_ROW_BLOCK 3u
#define BFAINTB_DEBUG_PLAN_COMPUTE_UNITS 4u
BFAINTB_API int bfaintb_debug_control(uint32_t what, uint32_t value);

/*
 * Pre-packed weights.  bfaintb_prepack reorders a row-major B (the layout above) once, offline, into the operand
 * order of the matrix instruction ("mfma16": column blocks of 16, K-chunks of 64 rows, a lane's two 8-row operands
 * adjacent; bfaintb_packed.hip states it byte by byte); bfaintb_gemm_prepacked multiplies by the packed copy.  A
 * block of 16 columns is then one contiguous slab, n / 16 workgroups stream their slabs linearly and own their
 * outputs, and a few rows of A need no split along k, no workspace and no second pass.  Successor of the
 * reference's host-side formatter mem_transfer<int8_t, ...> (mem_transfer.hpp:23-32), which writes the
 * bytes the device will read; the reference itself keeps B row-major (bfAintBGemm.cc:101-103).
 *   packed    device buffer of bfaintb_prepack_bytes(n, k, weight_bits) bytes (= n * k * weight_bits / 8), 16-byte aligned;
 *             4-bit codes need k % 128 == 0 in this format (bfaintb_prepack_bytes returns 0 otherwise)
 *   b, ldb    as for bfaintb_gemm;  scale and bias are used as they are, not reordered
 * bfaintb_unpack is the inverse (packed -> row-major), for tools and tests.
 */
BFAINTB_API size_t bfaintb_prepack_bytes(uint32_t n, uint32_t k, int weight_bits);
BFAINTB_API int bfaintb_prepack(void* packed, const void* b, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream);
BFAINTB_API int bfaintb_unpack(void* b, const void* packed, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream);
/* The same packed buffer from column-major B ("rcr"): n columns stored one after the other, k codes each, ldb elements
 * (>= k, a multiple of 16) from one column to the next — the layout tag the reference declares and never uses
 * (gemm_tensor_layout.hpp:16-19, bfAintBGemm.cc:18), and how a [out_features, in_features] weight lies in memory.
 * 8-bit: byte i of a column is row i's code.  4-bit: byte j of a column holds rows 2j (low nibble) and 2j+1 (high
 * nibble).  The result is byte for byte what bfaintb_prepack makes of the row-major form of the same codes. */
BFAINTB_API int bfaintb_prepack_colmajor(void* packed, const void* b, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream);
BFAINTB_API int bfaintb_gemm_prepacked(void* c, const void* a, const void* packed_b, const void* scale, const void* bias, uint32_t m,
                           uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc, int weight_bits, uint32_t group_size,
                           void* workspace, size_t workspace_bytes, void* stream);
/* The packed-weight GEMM with the epilogue descriptor of bfaintb_gemm_fused. */
BFAINTB_API int bfaintb_gemm_prepacked_fused(void* c, const void* a, const void* packed_b, const void* scale,
                                 const bfaintb_epilogue* epilogue, uint32_t m, uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc,
                                 int weight_bits, uint32_t group_size, void* workspace, size_t workspace_bytes, void* stream);
/* Scratch bfaintb_gemm_prepacked needs: 0 where a kernel that does not split k runs (the slab-streaming kernel for a few
 * rows of A, the large tiles), otherwise what the decode family or the small tiles need when they split along k — always
 * ask, for the shape at hand.  Same workspace protocol as bfaintb_gemm (bfaintb_workspace_init once; one workspace may
 * serve both entry points). */
BFAINTB_API size_t bfaintb_gemm_prepacked_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size);
BFAINTB_API size_t bfaintb_gemm_prepacked_workspace_bytes_ex(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size,
                                                 int variant);
/* Same with the kernel family forced (BFAINTB_VARIANT_*: DECODE = the slab-streaming kernel for a few rows of A and the
 * decode family beyond, m <= 32768; PREFILL[_256|_128|_256X128|_256_LDS|_128_LDS] = the tiled kernels reading packed weights), and which of
 * the two bfaintb_gemm_prepacked would run. */
BFAINTB_API int bfaintb_gemm_prepacked_ex(void* c, const void* a, const void* packed_b, const void* scale, const void* bias, uint32_t m,
                              uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc, int weight_bits, uint32_t group_size,
                              void* workspace, size_t workspace_bytes, void* stream, int variant);
BFAINTB_API int bfaintb_gemm_prepacked_variant(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size);

/*
 * Wire / on-disk form of a pre-packed weight: this 64-byte little-endian header, then payload_bytes of packed codes
 * (what bfaintb_prepack wrote), then scale_bytes of bf16 scales, row-major [groups][n], then, if has_bias, n bf16
 * biases.  Sections follow one another without padding (all sizes are multiples of 32 bytes).  The two functions run
 * on the host and touch no device: _init fills a header for a shape (same shape rules as bfaintb_prepack), _check
 * returns BFAINTB_OK for a header this library can consume (magic, layout, shape rules, section sizes that agree
 * with the shape) and a negative BFAINTB_ERR_* otherwise.
 */
typedef struct bfaintb_packed_header {
    char magic[8];          /* "BFAINTB1" */
    uint32_t header_bytes;  /* 64 */
    uint32_t layout;        /* BFAINTB_LAYOUT_MFMA16 */
    uint32_t weight_bits;   /* 8 or 4 */
    uint32_t group_size;    /* rows of k per scale group; 0 = one scale per output channel */
    uint32_t k, n;
    uint64_t payload_bytes; /* n * k * weight_bits / 8 */
    uint64_t scale_bytes;   /* groups * n * 2 */
    uint32_t has_bias;      /* 0 or 1 */
    uint32_t reserved[3];   /* zero */
} bfaintb_packed_header;
#define BFAINTB_LAYOUT_MFMA16 1u
BFAINTB_API int bfaintb_packed_header_init(bfaintb_packed_header* h, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size,
                               int has_bias);
BFAINTB_API int bfaintb_packed_header_check(const bfaintb_packed_header* h);

/*
 * What a call would launch, without launching anything: the kernel, the shape of a workgroup's share, the split along
 * k and the scratch it needs.  packed != 0 describes bfaintb_gemm_prepacked, else bfaintb_gemm; variant and split_k as
 * for bfaintb_gemm_ex (BFAINTB_VARIANT_AUTO, 0 = the library's own choice).  Host only; returns 0 or a negative error.
 * The plan is made for the compute units of the device that was current when the library first made one (256 when
 * there is none), reported in compute_units.  No counterpart in the reference, whose grid is fixed by the shape
 * (bfAintBGemm.cc:105-109).
 */
enum {
    BFAINTB_KERNEL_DECODE_FAMILY = 1, /* weight streaming with split-K, in row blocks beyond 32 rows of A */
    BFAINTB_KERNEL_DECODE_SLAB = 2,   /* packed weights: one column block of 16 per workgroup, no split */
    BFAINTB_KERNEL_TILES_128 = 3,     /* 128 x 128 tiles, weights in registers, may split k */
    BFAINTB_KERNEL_TILES_128_LDS = 4, /* 128 x 128 tiles, both operands through LDS */
    BFAINTB_KERNEL_TILES_256X128 = 5, /* tiles of 256 rows x 128 columns, weights in registers */
    BFAINTB_KERNEL_TILES_256 = 6,     /* 256 x 256 tiles, weights in registers */
    BFAINTB_KERNEL_TILES_256_LDS = 7  /* 256 x 256 tiles, both operands through LDS */
};
typedef struct bfaintb_plan {
    int32_t variant;           /* BFAINTB_VARIANT_DECODE, or the tiled variant with its tile size resolved */
    uint32_t kernel;           /* BFAINTB_KERNEL_* */
    uint32_t tile_rows;        /* rows of A per workgroup */
    uint32_t tile_cols;        /* columns of B per workgroup */
    uint32_t waves;            /* waves per workgroup */
    uint32_t splits;           /* workgroups along k per tile */
    uint32_t k_per_workgroup;  /* rows of k one workgroup covers */
    uint32_t workgroups;       /* of the launch (the first one, if there are two) */
    uint32_t tail_workgroups;  /* of a second launch over a last, thin round of tiles, or 0 */
    uint32_t launches;         /* 1 or 2 */
    uint32_t compute_units;    /* what the plan was made for */
    uint32_t reserved;
    uint64_t workspace_bytes;  /* what bfaintb_gemm[_prepacked]_workspace_bytes_ex reports for the same arguments */
} bfaintb_plan;
BFAINTB_API int bfaintb_gemm_plan(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size, int packed, int variant,
                                  uint32_t split_k, bfaintb_plan* out);

/* Which variant bfaintb_gemm would run (BFAINTB_VARIANT_*), or a negative error. */
BFAINTB_API int bfaintb_gemm_variant(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size);

/* Rows (bfaintb_prefill_tile) and columns of the tiles BFAINTB_VARIANT_PREFILL runs an m x n output of row-major
 * weights with: 128 x 128 while that makes at most 256 tiles (one per CU); else 256 rows x 128 columns while that
 * makes at most 256; else 256 x 256 (256 = the device's compute units: one tile per unit) — except that up to 512
 * tiles of 128 x 128 run in two rounds where the 256 x 128 ones just miss one round and the 256 x 256 ones would fill
 * at most 60 % of the units (640 x 11008), and that up to 128 rows always run 128 x 128 tiles, in as many rounds as it
 * takes (taller tiles would be half empty).  The two functions answer for 8-bit codes; 4-bit codes keep the 128 x 128
 * tiles up to 345 of them (their 256 x 128 kernel is the weaker one); bfaintb_gemm_plan answers for either.  Pre-packed
 * weights run the same tiles.  (The reference arithmetic has no 256 x 128 form: 256 x 256 there.) */
BFAINTB_API uint32_t bfaintb_prefill_tile(uint32_t m, uint32_t n);
BFAINTB_API uint32_t bfaintb_prefill_tile_cols(uint32_t m, uint32_t n);

/* The split-K factor the decode variant would use for a shape (1 for the prefill variant). */
BFAINTB_API uint32_t bfaintb_gemm_split_k(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size);

/*
 * Writes the dequantised weights W[k,n] as bf16 to w (row stride ldw elements), using the same
 * device dequantisation routine as the GEMM kernels.  Successor of the reference's ASM_PRINT debug
 * channel (bfAintBGemm.cc:113-118,156-169; bf16gemm_kernel_gfx90a.s:2-16), which was its only way
 * to look at in-kernel values.
 */
BFAINTB_API int bfaintb_dequant(void* w, const void* b, const void* scale, uint32_t n, uint32_t k, uint32_t ldb, uint32_t ldw,
                    int weight_bits, uint32_t group_size, void* stream);

/*
 * Measurement aid with no counterpart in the reference: reads `bytes` bytes from src with fully
 * coalesced 16-byte loads and discards them (sink may be NULL).  Timing it on the same buffers as the
 * decode GEMM gives the time this GPU needs just to fetch the weights in one launch.
 */
BFAINTB_API int bfaintb_probe_read(const void* src, size_t bytes, void* sink, void* stream);

/* Name of the __global__ function a variant launches, as it appears in a kernel trace.  Pass what
 * bfaintb_gemm_variant returned; BFAINTB_VARIANT_AUTO is read as decode up to m = 32, else prefill,
 * which for 32 < m <= 4096 need not be what bfaintb_gemm picks for a given n and k. */
BFAINTB_API const char* bfaintb_kernel_name(int variant, int weight_bits, uint32_t group_size, uint32_t m);

/* Text for a return code of this library (negative codes; positive ones are hipError_t values). */
BFAINTB_API const char* bfaintb_error_string(int code);

BFAINTB_API int bfaintb_version(void);

#ifdef __cplusplus
}
#endif
#endif /* BFAINTB_GEMM_H */
