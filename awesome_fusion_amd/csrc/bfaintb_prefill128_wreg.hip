// Tiled variant, 128x128 tiles, weights kept in registers: the small-tile kernel, for row-major B (described first) and
// for B in the packed order (PACKED: what changes is said where the codes are copied and read).
//
// Same job and the same reference kernel replaced as bfaintb_prefill128_kernel
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630; the reference's own tile is 32 x 64,
// /root/reference/bfAintBGemm/bfAintBGemm.cc:105-109).  That kernel converts W into LDS and every wave reads both
// operands back: a K-step takes 0.75 us whatever the load on the machine, three times its matrix-instruction time.
// Here, as in bfaintb_prefill_wreg_kernel, only A goes through LDS:
//   4 column groups side by side along n, KH waves each (the launch uses KH = 2: 512 threads, two waves per SIMD);
//   a wave owns ALL 128 rows x 32 columns of the tile = 8 x 2 accumulators of v_mfma_f32_16x16x32_bf16, converts exactly
//   the weights it multiplies by, straight into the instruction's operand registers, and each weight of the tile is
//   converted once.  With KH = 2 the two waves of a column group share a K-step by its blocks of 32 k (wave kh takes
//   block kh of every step) and the epilogue adds their sums, first blocks + second blocks: an output is the sum of
//   two chains of matrix instructions, not of one as in the other tiled kernels, so it agrees with them to rounding,
//   not bit for bit (it is reproducible run to run: nothing depends on timing).  The second wave per SIMD gives
//   the in-order issue something to run while the other waits for LDS: 2-11 % on every shape measured.
//   The vector-memory path takes about 20 cycles per instruction of a wave whatever it moves (measured: with the codes
//   fetched by 16 two-byte loads per wave and step, 80 instructions per CU and step took 1600 cycles and the kernel was
//   no faster than its predecessor; without them a step took 0.48 us instead of 0.80).  So the codes, too, come in by the
//   asynchronous copy — 16 bytes per lane, 8 KiB (4 for 4-bit codes) per step in 8 (4) instructions of the workgroup — into
//   four LDS stages of their own, kept as stored (rows of the tile's 128 codes), and each lane picks its codes out of
//   LDS: lane (c16 = lane % 16, kq = lane / 16) reads, per block of 32 k and for each of the 8 rows k0 + 8 kq + r, the
//   codes of columns 2 c16, 2 c16 + 1 of the wave's 32 (one ds_read_u16; u8 for 4-bit codes): code j of those 8 reads
//   is the 8-element operand of column 2 c16 + j, rows 8 kq .. 8 kq + 7.  The 16-byte chunks of a row are rotated by
//   twice (once) the row's block of 8, so the four kq groups of a wave read from different banks.
//   A: global -> LDS directly, four stages of 128 rows x 64 k (16 KiB each), same chunk swizzle as the other tiled
//   kernels; the copies of step kt + 3 (A and codes) start at step kt, behind the step's one barrier (which also says
//   every wave is done reading the stages they overwrite).  96 KiB of LDS in all.
//   Per K-step a CU reads 64 KiB of A fragments and 8 KiB of codes from LDS and the copy engine writes 24.
// Each of a wave's 8 (KH = 1: 16) units (block of 32 k, row block) of a step runs two matrix instructions and carries
// one conversion pair of the next step's weights (two weights: five instructions), so conversion and matrix work
// alternate finely.
// Accumulator (mt, j), register r of lane (c16, q = lane / 16): row 16 mt + 4 q + r, column 32 w + 2 c16 + j of the tile.
// Epilogue: as bfaintb_prefill128_kernel — fp32 sums staged in LDS in [m][n] order, each thread finishes 8 neighbouring
// columns of a row (bias, SiLU gate, residual, the one rounding) and stores them with one 16-byte write.
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

namespace {
constexpr uint32_t kTw = 128, kTwK = 64;
constexpr uint32_t kTwStage = 128 * 128;  // bytes of one A stage
constexpr uint32_t kTwCodeStage = 64 * 128;  // bytes of one stage of codes (8-bit; half of it used by 4-bit codes)

__device__ __forceinline__ uint32_t tw_swz(uint32_t row, uint32_t chunk) { return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4); }

// acc += a x b with the accumulator pinned to the accumulation registers and updated in place: written as assembly
// because the compiler gives some of the kernel's matrix instructions a destination other than their source and copies
// the sums back (21 of 224 instructions, 150 accumulator moves).  Behind the assembly its hazard bookkeeping sees
// nothing, so: the operands are written long before (LDS reads and conversions, under wait counts the compiler does
// insert for assembly operands); the accumulators are written by ordinary instructions only at the very start, with the
// whole prologue between that and the first matrix instruction, and read by them only in the epilogue, behind explicit
// idle cycles (tw_settle).
__device__ __forceinline__ void tw_mfma(f32x4_t& acc, const bf16x8_t& a, const bf16x8_t& b)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void tw_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
}  // namespace

// MT: the blocks of 16 rows of the tile that are multiplied (8, or 4 for an m of at most 64: the rows beyond take no
// matrix instructions, no fragment reads and no accumulators; everything about the weights stays as it is).
template <int BITS, bool GROUPED, bool PACKED, int KH, bool COPIER, int MT>
__global__ void __launch_bounds__(256 * KH + (COPIER ? 64 : 0)) __attribute__((amdgpu_waves_per_eu(KH + (COPIER ? 1 : 0), KH + (COPIER ? 1 : 0))))
bfaintb_prefill128_wreg_kernel(const GemmParams p)
{
    static_assert(KH == 1 || KH == 2, "one wave per SIMD, or two that share a K-step by its blocks of 32 k");
    static_assert(MT == 8 || MT == 4, "whole tiles, or their first 64 rows");
    constexpr uint32_t kWaves = 4u * KH;
    constexpr uint32_t NB = 2u / KH;  // blocks of 32 k of a K-step that a wave multiplies
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a0[kTwStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a1[kTwStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a2[kTwStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a3[kTwStage];
    constexpr uint32_t kRowBytes = 128u * BITS / 8u;  // a tile row of codes
    // (the codes of one K-step: 64 rows; the arrays keep the 8-bit extent for both code widths — an extent that depends
    // on a template parameter, in an array the lambdas below capture, makes the host pass drop the kernel's launch
    // stub without a diagnostic)
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w0[kTwCodeStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w1[kTwCodeStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w2[kTwCodeStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w3[kTwCodeStage];
    auto w_tile = [&](auto stage_c) -> uint8_t* {
        constexpr uint32_t St = decltype(stage_c)::value;
        return St == 0 ? lds_w0 : St == 1 ? lds_w1 : St == 2 ? lds_w2 : lds_w3;
    };
    auto a_tile = [&](auto stage_c) -> uint8_t* {
        constexpr uint32_t St = decltype(stage_c)::value;
        return St == 0 ? lds_a0 : St == 1 ? lds_a1 : St == 2 ? lds_a2 : lds_a3;
    };
    using C0 = std::integral_constant<uint32_t, 0>;
    using C1 = std::integral_constant<uint32_t, 1>;
    using C2 = std::integral_constant<uint32_t, 2>;
    using C3 = std::integral_constant<uint32_t, 3>;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wc = wave & 3u;                  // the wave's 32 columns
    const uint32_t kh = KH == 2 ? wave >> 2 : 0u;   // two waves per column group: the block of 32 k this one multiplies
    // local block lb of this wave is block blk_of(lb) of the step
    auto blk_of = [&](uint32_t lb) { return KH == 2 ? kh : lb; };
    const uint32_t c16 = lane & 15u, kq = lane >> 4;

    // ---- tile of this workgroup (the order of bfaintb_prefill128_kernel: the ids an XCD receives cover consecutive
    //      logical ids, which walk groups of 8 tile-rows column by column)
    const uint32_t tiles_m = (p.m + kTw - 1) / kTw, tiles_n = (p.n + kTw - 1) / kTw;
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
    const uint32_t m0 = tm * kTw, n0 = tn * kTw;

    const uint32_t rows_valid = p.m - m0 < kTw ? p.m - m0 : kTw;
    const uint32_t a_extent = ((rows_valid - 1u) * p.lda + p.k) * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.a + (size_t)m0 * p.lda), 0, (int)a_extent, kBufferFlags);
    const uint32_t cols_valid = p.n - n0 < kTw ? p.n - n0 : kTw;
    // packed weights: a block of 16 columns is one run of k x 16 codes in chunks of 1024 bytes (64 rows of 8-bit, 128 rows
    // of 4-bit codes); the tile's 8 column blocks follow one another, and one past n reads as zero through the extent
    const uint32_t slab_bytes = p.k * (BITS == 8 ? 16u : 8u);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        PACKED ? __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (size_t)(n0 / 16u) * slab_bytes), 0,
                                                   (int)(cols_valid / 16u * slab_bytes), kBufferFlags)
               : __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.b + (BITS == 8 ? n0 : n0 / 2u)), 0,
                                                   (int)((p.k - 1u) * p.ldb_bytes + (BITS == 8 ? cols_valid : cols_valid / 2u)), kBufferFlags);

    // K-steps of this workgroup: all of them, or the share of split blockIdx.y (p.k_per_wg rows each; the host makes sure
    // every split has at least one).  kt below counts within the share; kbase + kt is the step of the whole matrix.
    const uint32_t ksteps_all = (p.k + kTwK - 1u) / kTwK;
    const uint32_t ks = blockIdx.y;
    const uint32_t kbase = ks * (p.k_per_wg / kTwK);
    const uint32_t ksteps = p.k_per_wg / kTwK < ksteps_all - kbase ? p.k_per_wg / kTwK : ksteps_all - kbase;
    const uint32_t last_chunks = (p.k - (ksteps_all - 1u) * kTwK) / 8u;  // valid 16-byte chunks per row of A in the last step
    auto clamp = [&](uint32_t t) { return t < ksteps ? t : ksteps - 1u; };

    // A copy: instruction j of wave w fills rows 8 (kACopies w + j) .. + 7; lane l lands at row + l / 8, chunk position l % 8, so
    // it fetches chunk (l % 8) ^ ((row >> 1) & 7) = (l % 8) ^ (l / 16) for even j and that ^ 4 for odd j; the row advance
    // of j and the K advance sit in the scalar offset.  A chunk past the end of k (partial last step) is fetched from
    // beyond the extent and reads as zero; rows of B past k read as zero codes, finite weights, and multiply those zeros.
    constexpr uint32_t kACopies = 4u / KH;  // per wave and step: 8 rows each
    const uint32_t a_row = 8u * kACopies * wave + (lane >> 3);
    const uint32_t chunk_e = (lane & 7u) ^ ((lane >> 4) & 7u), chunk_o = chunk_e ^ 4u;
    const uint32_t a_voff_e = (a_row * p.lda + chunk_e * 8u) * 2u, a_voff_o = (a_row * p.lda + chunk_o * 8u) * 2u;
    const uint32_t a_last_e = chunk_e < last_chunks ? a_voff_e : a_extent, a_last_o = chunk_o < last_chunks ? a_voff_o : a_extent;
    auto dma_a = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = a_tile(stage_c) + wave * (1024u * kACopies);
        const bool last = kbase + kt + 1u == ksteps_all;
        const uint32_t ve = last ? a_last_e : a_voff_e, vo = last ? a_last_o : a_voff_o;
#pragma unroll
        for (uint32_t j = 0; j < kACopies; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16,
                                                     (j & 1u) ? vo : ve, (kbase + kt) * kTwK * 2u + j * 16u * p.lda, 0, 0);
    };

    // W codes.  Copy: a 16-byte-per-lane instruction fills 1024 bytes = kRowsPerCopy rows of the stage; the step's 64
    // rows take kCopies instructions, kCopiesPerWave for each wave.  Lane l lands at row l / kChunks of its block, chunk
    // position l % kChunks, and fetches the chunk the rotation puts there: position = chunk + kRot * (row / 8 % 4).
    //
    // Packed weights: the chunk of a column block that holds the step (1024 bytes: all of it for 8-bit codes; for 4-bit
    // codes it spans two steps and is copied for each) is one instruction; wave w copies column blocks 2 w and 2 w + 1,
    // its own columns.  The chunk's 16-byte pieces are the lanes of the packed order: piece 16 kg + nl = rows 8 kg .. + 7
    // of both K-blocks (4-bit: of four), column nl.  This kernel's lane (c16, kq) wants columns nl = 2 (c16 % 8) and
    // nl + 1 of column block 2 w + c16 / 8, rows of kq: pieces 16 kq + nl and the next.  So that a wave reads each of the
    // two with one conflict-free instruction, piece 16 g + 2 c + h is stored at position 32 h + ((8 g + c) ^ 8 (column
    // block odd)): the 16 lanes of one kq then read 16 neighbouring pieces' worth of banks.
    constexpr uint32_t kChunks = kRowBytes / 16u;        // 8 or 4 chunks per row
    constexpr uint32_t kRowsPerCopy = 1024u / kRowBytes; // 8 or 16
    // (eight waves, 4-bit codes in rows: four instructions for eight waves — waves 4 .. 7 repeat the copies of waves
    // 0 .. 3, same bytes to the same place, so that every wave has the same number of requests in flight for the one
    // wait count at the top of a step)
    constexpr uint32_t kCopies = PACKED ? 8u : 64u / kRowsPerCopy;  // per step: 8, or 4 for 4-bit codes in rows
    constexpr uint32_t kCopiesPerWave = kCopies >= kWaves ? kCopies / kWaves : 1u;
    const uint32_t wcopier = kCopies >= kWaves ? wave : wave & (kCopies - 1u);
    constexpr uint32_t kRot = BITS == 8 ? 2u : 1u;       // a wave's 16 lanes of one kq cover 32 (16) bytes of a row
    uint32_t w_voff[2];  // (fixed extent: see the note on the arrays above)
#pragma unroll
    for (uint32_t j = 0; j < kCopiesPerWave; ++j) {
        if constexpr (PACKED) {
            const uint32_t cblock = kCopiesPerWave * wcopier + j;  // the column block this instruction copies
            const uint32_t at = (lane & 31u) ^ (8u * (cblock & 1u));  // 8 g + c of the piece this lane's position holds
            w_voff[j] = cblock * slab_bytes + (16u * (at >> 3) + 2u * (at & 7u) + (lane >> 5)) * 16u;
        } else {
            const uint32_t row = (kCopiesPerWave * wcopier + j) * kRowsPerCopy + lane / kChunks;  // within the step
            const uint32_t chunk = ((lane % kChunks) - kRot * ((row >> 3) & 3u)) & (kChunks - 1u);
            w_voff[j] = row * p.ldb_bytes + chunk * 16u;
        }
    }
    // where step kt's codes start, beyond the lane's offset: w_step * (kbase + kt >> w_shift)  (spelt out at the two copies:
    // with a lambda for it among the copy's arguments the host pass drops the kernel's launch stub without a diagnostic)
    const uint32_t w_step = PACKED ? 1024u : kTwK * p.ldb_bytes;
    constexpr uint32_t w_shift = (PACKED && BITS == 4) ? 1u : 0u;
    auto dma_w = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = w_tile(stage_c) + kCopiesPerWave * wcopier * 1024u;
#pragma unroll
        for (uint32_t j = 0; j < kCopiesPerWave; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16, w_voff[j], ((kbase + kt) >> w_shift) * w_step, 0, 0);
    };
    // The copying wave (COPIER: one wave more than those that compute): every copy of the K loop is its request, so that
    // the computing waves' only memory requests are their group scales and the wait for those — which the compiler
    // places, and which counts every request of the wave ahead of them — no longer holds a wave until copies of later
    // steps have landed (grouped scales: 9-11 % on the whole kernel; with one scale per column, where the computing
    // waves load nothing in the loop, the copying wave changes -1 .. +4 % and is not used).
    // Instruction j of a step's A fills rows 8 j .. 8 j + 7 (the lane's offsets are those of rows 0 .. 7, the row advance
    // sits in the scalar offset); the codes go as the computing waves would copy them.  The first three steps' copies
    // are shared out over the computing waves (the prologue below): one wave would issue them one after the other.
    if (COPIER && wave == kWaves) {
        const uint32_t pa_e = ((lane >> 3) * p.lda + chunk_e * 8u) * 2u, pa_o = ((lane >> 3) * p.lda + chunk_o * 8u) * 2u;
        const uint32_t pl_e = chunk_e < last_chunks ? pa_e : a_extent, pl_o = chunk_o < last_chunks ? pa_o : a_extent;
        uint32_t pw[8];
#pragma unroll
        for (uint32_t j = 0; j < kCopies; ++j) {
            if constexpr (PACKED) {
                const uint32_t at = (lane & 31u) ^ (8u * (j & 1u));
                pw[j] = j * slab_bytes + (16u * (at >> 3) + 2u * (at & 7u) + (lane >> 5)) * 16u;
            } else {
                const uint32_t row = j * kRowsPerCopy + lane / kChunks;
                const uint32_t chunk = ((lane % kChunks) - kRot * ((row >> 3) & 3u)) & (kChunks - 1u);
                pw[j] = row * p.ldb_bytes + chunk * 16u;
            }
        }
        auto copy_step = [&](uint32_t stage, uint32_t kt) {
            uint8_t* const a_base = stage == 0u ? lds_a0 : stage == 1u ? lds_a1 : stage == 2u ? lds_a2 : lds_a3;
            uint8_t* const w_base = stage == 0u ? lds_w0 : stage == 1u ? lds_w1 : stage == 2u ? lds_w2 : lds_w3;
            const bool last = kbase + kt + 1u == ksteps_all;
            const uint32_t ve = last ? pl_e : pa_e, vo = last ? pl_o : pa_o;
#pragma unroll
            for (uint32_t j = 0; j < 16u; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(a_base + j * 1024u), 16, (j & 1u) ? vo : ve,
                                                         (kbase + kt) * kTwK * 2u + j * 16u * p.lda, 0, 0);
#pragma unroll
            for (uint32_t j = 0; j < kCopies; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)(w_base + j * 1024u), 16, pw[j],
                                                         ((kbase + kt) >> w_shift) * w_step, 0, 0);
        };
        barrier_no_fence();  // (the first three steps' copies are shared out over the computing waves: see the prologue)
        for (uint32_t kt = 0; kt < ksteps; ++kt) {
            // the computing waves start step kt behind this barrier: the copies of steps up to kt + 1 have landed when at
            // most those of step kt + 2 (requested behind the last barrier) are in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(16 + kCopies) : "memory");
            barrier_no_fence();
            copy_step((kt + 3u) & 3u, clamp(kt + 3u));  // into the stage of step kt - 1, which every wave has left
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // the epilogue's first barrier: nothing is writing LDS any more
        return;               // (a wave that has ended no longer counts at the barriers that follow)
    }
    // Pick: this lane's 2 columns (byte offset wbyte of a row), rows 8 kq .. 8 kq + 7 of block blk of 32 k: row
    // 32 blk + 8 kq + r, whose block of 8 is 4 blk + kq, rotation kRot * kq
    const uint32_t wcol = 32u * wc + 2u * c16;  // within the tile
    const uint32_t wbyte = wcol * BITS / 8u;
    // (packed: the piece of the lane's first column; the second one's is 512 bytes on; 4-bit codes: + 8 in odd steps)
    const uint32_t w_rd = PACKED ? (2u * wc + (c16 >> 3)) * 1024u + (((8u * kq + (c16 & 7u)) ^ (8u * (c16 >> 3))) << 4)
                                 : (8u * kq) * kRowBytes + ((((wbyte >> 4) + kRot * kq) & (kChunks - 1u)) << 4) + (wbyte & 15u);  // + 32 blk rows + r rows
    // Packed codes of a step as a lane reads them: [column j][K-block][half]: 8-bit codes: rows 4 half .. + 3 in the bytes
    // of a dword; 4-bit codes: [j][K-block][0] holds the 8 rows in its nibbles.
    // (K-block: the wave's own; with two waves per column group each reads its half of the piece)
    struct PackedCodes {
        uint32_t d[2][NB][2];
    };
    auto read_packed = [&](PackedCodes& pc, const uint8_t* src, uint32_t kt, uint32_t j) {  // src: the stage + w_rd
        if constexpr (BITS == 8 && KH == 1) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + 512u * j);
            pc.d[j][0][0] = v[0], pc.d[j][0][1] = v[1], pc.d[j][1][0] = v[2], pc.d[j][1][1] = v[3];
        } else if constexpr (BITS == 8) {
            const u32x2_t v = *reinterpret_cast<const u32x2_t*>(src + 512u * j + 8u * kh);
            pc.d[j][0][0] = v[0], pc.d[j][0][1] = v[1];
        } else if constexpr (KH == 1) {
            const u32x2_t v = *reinterpret_cast<const u32x2_t*>(src + 512u * j + 8u * ((kbase + kt) & 1u));
            pc.d[j][0][0] = v[0], pc.d[j][1][0] = v[1];
        } else {
            pc.d[j][0][0] = *reinterpret_cast<const uint32_t*>(src + 512u * j + 8u * ((kbase + kt) & 1u) + 4u * kh);
        }
    };
    // 4-bit: the two's-complement nibbles of a dword of 8 rows: even rows in the low nibbles of `ev`'s bytes, odd rows of `od`'s
    struct PackedNibbles {
        uint32_t ev[2][NB], od[2][NB];  // [column j][K-block]
    };
    // rows 2 pr, 2 pr + 1 of column j of K-block blk, as fp32 (8-bit: the stored code; 4-bit: q / 16)
    auto packed_values = [&](const PackedCodes& pc, PackedNibbles& nb, uint32_t blk, uint32_t j, uint32_t pr, float& f0, float& f1) {
        if constexpr (BITS == 8) {
            const uint32_t x = pc.d[j][blk][pr >> 1];
            f0 = (pr & 1u) ? (float)((x >> 16) & 0xffu) : (float)(x & 0xffu);  // v_cvt_f32_ubyte2 / 0
            f1 = (pr & 1u) ? (float)(x >> 24) : (float)((x >> 8) & 0xffu);     // v_cvt_f32_ubyte3 / 1
        } else {
            if (pr == 0) codes4_to_nibbles(pc.d[j][blk][0], nb.ev[j][blk], nb.od[j][blk]);
            const uint32_t e = nb.ev[j][blk], o = nb.od[j][blk];
            f0 = pr == 0 ? nibble_to_f32_sixteenth<0>(e) : pr == 1 ? nibble_to_f32_sixteenth<1>(e) : pr == 2 ? nibble_to_f32_sixteenth<2>(e) : nibble_to_f32_sixteenth<3>(e);
            f1 = pr == 0 ? nibble_to_f32_sixteenth<0>(o) : pr == 1 ? nibble_to_f32_sixteenth<1>(o) : pr == 2 ? nibble_to_f32_sixteenth<2>(o) : nibble_to_f32_sixteenth<3>(o);
        }
    };
    struct Raw {
        uint32_t d[NB][8];  // [the wave's block of 32 k][row]: two codes
    };
    auto pick = [&](Raw& raw, auto stage_c) {
        const uint8_t* tile = w_tile(stage_c) + w_rd;
#pragma unroll
        for (uint32_t lb = 0; lb < NB; ++lb)
#pragma unroll
            for (uint32_t r = 0; r < 8; ++r) {
                if constexpr (BITS == 8) raw.d[lb][r] = *reinterpret_cast<const uint16_t*>(tile + (32u * blk_of(lb) + r) * kRowBytes);
                else raw.d[lb][r] = *(tile + (32u * blk_of(lb) + r) * kRowBytes);
            }
    };
    // Scales go through a buffer resource so that the load is issued whatever the lane's column (the wait counts
    // below count requests): columns past n read other columns' scales, or zero beyond the array; their results are
    // never stored.
    const uint32_t scale_rows = GROUPED ? p.k / p.group_size : 1u;
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.scale), 0, (int)(((scale_rows - 1u) * p.lds + p.n) * 2u), kBufferFlags);
    const uint32_t s_voff = (n0 + wcol) * 2u;
    auto block_group_scales = [&](uint32_t (&sr)[NB], uint32_t kt, uint32_t lb) {
        uint32_t g = group_of_row(p, (kbase + kt) * kTwK + 32u * blk_of(lb));
        if (g >= scale_rows) g = scale_rows - 1u;  // rows past k in a partial last step: any scale will do
        sr[lb] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_s, s_voff, g * p.lds * 2u, 0);
    };
    auto group_scales = [&](uint32_t (&sr)[NB], uint32_t kt) {
#pragma unroll
        for (uint32_t lb = 0; lb < NB; ++lb) block_group_scales(sr, kt, lb);
    };
    float cs[2] = {0.f, 0.f};  // one scale per column: fixed
    if constexpr (!GROUPED) {
        const uint32_t sr = __builtin_amdgcn_raw_buffer_load_b32(rsrc_s, s_voff, 0, 0);
        cs[0] = make_col_scale_nibble<BITS>(sr & 0xffffu);
        cs[1] = make_col_scale_nibble<BITS>(sr >> 16);
    }
    struct Ops {
        uint32_t w[NB][2][4];  // [the wave's block of 32 k][column j][dword]: the 8-element operand as 4 packed pairs
    };
    // the two codes of a load, ready for the conversion: as stored (8-bit codes: the excess of 128 comes off in the
    // multiplication, see scaled()); two's-complement nibbles, the second shifted down to a low nibble (4-bit codes)
    auto prepare = [&](uint32_t x, uint32_t& c0, uint32_t& c1) {
        if constexpr (BITS == 8) {
            c0 = x;
            c1 = x;
        } else {
            c0 = x ^ 0x88u;
            c1 = c0 >> 4;
        }
    };
    auto value = [&](uint32_t c, uint32_t j) -> float {
        if constexpr (BITS == 8) return j == 0 ? (float)(c & 0xffu) : (float)((c >> 8) & 0xffu);  // v_cvt_f32_ubyte0 / 1
        else return nibble_to_f32_sixteenth<0>(c);
    };
    // value x scale.  8-bit codes: u s - 128 s in one fused operation — u s (8 x 8 bits), 128 s and their difference
    // (u - 128) s are all exact in fp32, so this is the product q s of the signed code, bit for bit (a zero code gives +0
    // where q s gives -0 for a negative scale: no sum can tell), and the sign flip of the codes is saved.
    auto scaled = [&](float f, float scale) -> float {
        if constexpr (BITS == 8) return __builtin_fmaf(f, scale, -128.0f * scale);
        else return f * scale;
    };
    // one sixteenth of a step's conversion: rows 2 pr, 2 pr + 1 of column j of the wave's block blk
    auto convert_pair = [&](Ops& ops, const Raw& raw, uint32_t (&pre)[NB][8][2], const float (&sc)[NB][2], uint32_t blk, uint32_t j, uint32_t pr) {
        if (j == 0) {
            prepare(raw.d[blk][2 * pr], pre[blk][2 * pr][0], pre[blk][2 * pr][1]);
            prepare(raw.d[blk][2 * pr + 1], pre[blk][2 * pr + 1][0], pre[blk][2 * pr + 1][1]);
        }
        ops.w[blk][j][pr] = pack_bf16_rne(scaled(value(pre[blk][2 * pr][j], j), sc[blk][j]), scaled(value(pre[blk][2 * pr + 1][j], j), sc[blk][j]));
    };
    auto block_scales = [&](float (&sc)[NB][2], const uint32_t (&sr)[NB]) {
#pragma unroll
        for (uint32_t blk = 0; blk < NB; ++blk) {
            if constexpr (GROUPED) {
                sc[blk][0] = make_col_scale_nibble<BITS>(sr[blk] & 0xffffu);
                sc[blk][1] = make_col_scale_nibble<BITS>(sr[blk] >> 16);
            } else {
                sc[blk][0] = cs[0];
                sc[blk][1] = cs[1];
            }
        }
    };
    auto convert_all = [&](Ops& ops, const Raw& raw, const uint32_t (&sr)[NB]) {
        uint32_t pre[NB][8][2];
        float sc[NB][2];
        block_scales(sc, sr);
#pragma unroll
        for (uint32_t u = 0; u < 8u * NB; ++u) convert_pair(ops, raw, pre, sc, u >> 3, (u >> 2) & 1u, u & 3u);
    };
    // the same from packed codes: step kt, whose codes are in the stage behind src
    auto convert_all_packed = [&](Ops& ops, const uint8_t* src, uint32_t kt, const uint32_t (&sr)[NB]) {
        PackedCodes pc;
        PackedNibbles nb;
        float sc[NB][2];
        block_scales(sc, sr);
        read_packed(pc, src, kt, 0);
        read_packed(pc, src, kt, 1);
#pragma unroll
        for (uint32_t u = 0; u < 8u * NB; ++u) {
            const uint32_t blk = u >> 3, j = (u >> 2) & 1u, pr = u & 3u;
            float f0, f1;
            packed_values(pc, nb, blk, j, pr, f0, f1);
            ops.w[blk][j][pr] = pack_bf16_rne(scaled(f0, sc[blk][j]), scaled(f1, sc[blk][j]));
        }
    };

    f32x4_t acc[8][2];
#pragma unroll
    for (int mt = 0; mt < 8; ++mt)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[mt][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // fragment (mt, blk): row 16 mt + c16 of the tile, chunk 4 blk + kq (the swizzle repeats every 16 rows)
    bf16x8_t af[4];  // the fragments of the next few units, carried from step to step
    uint32_t a_rd[NB];
#pragma unroll
    for (uint32_t lb = 0; lb < NB; ++lb) a_rd[lb] = tw_swz(c16, 4u * blk_of(lb) + kq);

    // One K-step.  `cur`: the operands of this step; `nxt` receives those of step kt + 1, converted from the codes in stage
    // S + 1; stage S holds this step's A; the copies of step kt + 3 go into stage S + 3 = S - 1, which every wave finished
    // reading (A during step kt - 1, the codes during step kt - 2) before the barrier at the top.  `s1`: the group scales
    // of step kt + 1 (requested one step ago), `s2` receives those of step kt + 2.
    // With one wave per SIMD the wave issues in order and the matrix pipe idles whenever something else takes longer to
    // issue than a matrix instruction runs, so the step is written as 32 fenced slots of one matrix instruction plus a
    // few other instructions: unit u = (block of 32 k, row block) has two slots (the wave's two columns groups);
    //   slot 0 of unit u: the A fragment of unit u + kAhead (the last kAhead units fetch the next step's first
    //          fragments: its stage is complete, see the wait below); the two code reads that conversion pair u + 4 needs;
    //          the first half of conversion pair u (two weights: sign flips, two conversions)
    //   slot 1 of unit u: one memory request (with group scales: those first, in unit 0; then the copies); the second
    //          half of pair u (two multiplications, the rounding pack)
    constexpr uint32_t kAhead = 4;
    constexpr uint32_t kUnits = 8u * NB;
    auto step = [&](auto stage_c, uint32_t kt, const Ops& cur, Ops& nxt, const uint32_t (&s1)[NB], uint32_t (&s2)[NB]) {
        constexpr uint32_t S = decltype(stage_c)::value;
        using Next = std::integral_constant<uint32_t, (S + 1u) & 3u>;
        using Target = std::integral_constant<uint32_t, (S + 3u) & 3u>;
        // At most the requests of the step before this one may still be in flight: then this wave's part of this step's
        // AND the next step's A (requested three and two steps ago) and of the next step's codes (two steps ago) has
        // landed.  Behind the barrier every wave's has.
        if constexpr (!COPIER) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kACopies + kCopiesPerWave + (GROUPED ? NB : 0)) : "memory");
        barrier_no_fence();  // (a fenced barrier would also wait for the copies of the steps ahead)
        const uint32_t kt3 = clamp(kt + 3), kt2 = clamp(kt + 2);
        const bool last3 = kbase + kt3 + 1u == ksteps_all;
        const uint32_t ve = last3 ? a_last_e : a_voff_e, vo = last3 ? a_last_o : a_voff_o;
        uint8_t* const a_dst = a_tile(Target{}) + wave * (1024u * kACopies);
        uint8_t* const w_dst = w_tile(Target{}) + kCopiesPerWave * wcopier * 1024u;
        const uint8_t* const a_src = a_tile(stage_c);
        const uint8_t* const a_nxt = a_tile(Next{});
        const uint8_t* const w_src = w_tile(Next{}) + w_rd;
        uint32_t code[NB][8];   // the codes of step kt + 1 as read: [block][row], two codes each
        uint32_t pre[NB][8][2];
        PackedCodes pc;        // ... or, from packed weights, the lane's 2 x 16 (8) bytes
        PackedNibbles nb;
        float sc[NB][2];
        float f0 = 0.f, f1 = 0.f;
        block_scales(sc, s1);
        // pair v = (block v / 8, rows 2 (v / 2 % 4), + 1, column v % 2): its two rows are read by the pair with column 0
        auto read_codes = [&](uint32_t v) {
            const uint32_t blk = v >> 3, pr = (v >> 1) & 3u;
#pragma unroll
            for (uint32_t h = 0; h < 2; ++h) {
                const uint32_t r = 2u * pr + h;
                if constexpr (BITS == 8) code[blk][r] = *reinterpret_cast<const uint16_t*>(w_src + (32u * blk_of(blk) + r) * kRowBytes);
                else code[blk][r] = *(w_src + (32u * blk_of(blk) + r) * kRowBytes);
            }
        };
        if constexpr (PACKED) {
            read_packed(pc, w_src, kt + 1u, 0);
            read_packed(pc, w_src, kt + 1u, 1);
        } else {
            read_codes(0);
            read_codes(2);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t u = 0; u < kUnits; ++u) {
            const uint32_t blk = u >> 3, mt = u & 7u;
            const uint32_t cblk = u >> 3, cpr = (u >> 1) & 3u, cj = u & 1u;  // conversion pair u
            const bf16x8_t a_now = af[u % kAhead];
            const bf16x8_t wf0 = __builtin_bit_cast(bf16x8_t, make_uint4(cur.w[blk][0][0], cur.w[blk][0][1], cur.w[blk][0][2], cur.w[blk][0][3]));
            const bf16x8_t wf1 = __builtin_bit_cast(bf16x8_t, make_uint4(cur.w[blk][1][0], cur.w[blk][1][1], cur.w[blk][1][2], cur.w[blk][1][3]));
            // ---- slot 0
            if (mt < (uint32_t)MT) tw_mfma(acc[mt][0], a_now, wf0);
            if (((u + kAhead) & 7u) < (uint32_t)MT) {  // (the fragment of a row block that is multiplied)
                if (u + kAhead < kUnits) af[u % kAhead] = *reinterpret_cast<const bf16x8_t*>(a_src + a_rd[(u + kAhead) >> 3] + ((u + kAhead) & 7u) * 2048u);
                else af[u % kAhead] = *reinterpret_cast<const bf16x8_t*>(a_nxt + a_rd[0] + (u + kAhead - kUnits) * 2048u);
            }
            if constexpr (PACKED) {
                packed_values(pc, nb, cblk, cj, cpr, f0, f1);
            } else {
                if (cj == 0 && u + 4 < kUnits) read_codes(u + 4);
                if (cj == 0) {
                    if constexpr (BITS == 8) {
                        // (the two reads stay two registers: left to itself the compiler packs them into one and shifts the
                        // pair about before converting — six instructions where four byte-selecting conversions do.  Said here,
                        // where the values are needed, and not at the reads, where it would make the wave wait for them.)
                        asm("" : "+v"(code[cblk][2 * cpr]));
                        asm("" : "+v"(code[cblk][2 * cpr + 1]));
                    }
                    prepare(code[cblk][2 * cpr], pre[cblk][2 * cpr][0], pre[cblk][2 * cpr][1]);
                    prepare(code[cblk][2 * cpr + 1], pre[cblk][2 * cpr + 1][0], pre[cblk][2 * cpr + 1][1]);
                }
                f0 = value(pre[cblk][2 * cpr][cj], cj);
                f1 = value(pre[cblk][2 * cpr + 1][cj], cj);
            }
            __builtin_amdgcn_sched_barrier(0);
            // ---- slot 1
            if (mt < (uint32_t)MT) tw_mfma(acc[mt][1], a_now, wf1);
            // (the group scales first: the next step waits for them at its very start, and that wait then leaves the
            // copies requested behind them in flight — requested last, they made it a wait for everything)
            // (one block's scales per slot: finding a group is a chain of five scalar instructions)
            constexpr uint32_t kFirstCopy = GROUPED ? NB : 0u;
            if (GROUPED && u < NB) {
                block_group_scales(s2, kt2, u);
            } else if (COPIER) {
            } else if (u >= kFirstCopy && u < kFirstCopy + kACopies) {
                const uint32_t q = u - kFirstCopy;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(a_dst + q * 1024u), 16, (q & 1u) ? vo : ve,
                                                         (kbase + kt3) * kTwK * 2u + q * 16u * p.lda, 0, 0);
            } else if (u >= kFirstCopy + kACopies && u < kFirstCopy + kACopies + kCopiesPerWave) {
                const uint32_t q = u - kFirstCopy - kACopies;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)(w_dst + q * 1024u), 16, w_voff[q],
                                                         ((kbase + kt3) >> w_shift) * w_step, 0, 0);
            }
            nxt.w[cblk][cj][cpr] = pack_bf16_rne(scaled(f0, sc[cblk][cj]), scaled(f1, sc[cblk][cj]));
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- prologue: A tiles and codes of steps 0, 1, 2 -> stages 0, 1, 2; operands of step 0
    Ops ops0, ops1;
    uint32_t sa[NB] = {}, sb[NB] = {};  // group scales, alternating: sb = step 0 (then 2, ...), sa = step 1 (then 3, ...)
    dma_w(C0{}, 0);
    dma_a(C0{}, 0);
    dma_w(C1{}, clamp(1));
    dma_a(C1{}, clamp(1));
    dma_w(C2{}, clamp(2));
    dma_a(C2{}, clamp(2));
    if constexpr (GROUPED) {
        group_scales(sb, 0);
        group_scales(sa, clamp(1));
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    barrier_no_fence();
    if constexpr (PACKED) {
        convert_all_packed(ops0, w_tile(C0{}) + w_rd, 0, sb);
    } else {
        Raw raw;
        pick(raw, C0{});
        convert_all(ops0, raw, sb);
    }
#pragma unroll
    for (uint32_t u = 0; u < kAhead; ++u) af[u] = *reinterpret_cast<const bf16x8_t*>(a_tile(C0{}) + a_rd[0] + u * 2048u);

    uint32_t kt = 0;
    for (; kt + 3 < ksteps; kt += 4) {
        step(C0{}, kt, ops0, ops1, sa, sb);
        step(C1{}, kt + 1, ops1, ops0, sb, sa);
        step(C2{}, kt + 2, ops0, ops1, sa, sb);
        step(C3{}, kt + 3, ops1, ops0, sb, sa);
    }
    if (kt < ksteps) step(C0{}, kt, ops0, ops1, sa, sb);
    if (kt + 1 < ksteps) step(C1{}, kt + 1, ops1, ops0, sb, sa);
    if (kt + 2 < ksteps) step(C2{}, kt + 2, ops0, ops1, sa, sb);

    // ---- epilogue: fp32 sums -> LDS in [m][n] order (rows 32 q .. 32 q + 31 in the q-th array), then finish row-wise
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing asynchronous may still be writing LDS
    tw_settle();                                       // the last matrix instructions have written their sums
    __syncthreads();                                   // ... and every wave is done reading the stages
    auto c_rows = [&](uint32_t q) -> float* {
        return reinterpret_cast<float*>(q == 0 ? lds_a0 : q == 1 ? lds_a1 : q == 2 ? lds_a2 : lds_a3);
    };
    // (two waves per column group: the wave of the second blocks stages its sums, the wave of the first blocks adds its
    // own to them — first blocks + second blocks, whatever the timing)
    auto stage_sums = [&](bool add) {
#pragma unroll
        for (uint32_t mt = 0; mt < (uint32_t)MT; ++mt) {
            float* base = c_rows(mt >> 1);
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) {
                const uint32_t row = 16u * (mt & 1u) + 4u * kq + r;  // within the 32 rows of this array
                float2* at = reinterpret_cast<float2*>(base + row * kTw + wcol);
                float2 v = make_float2(acc[mt][0][r], acc[mt][1][r]);
                if (add) {
                    const float2 o = *at;
                    v = make_float2(v.x + o.x, v.y + o.y);
                }
                *at = v;
            }
        }
    };
    if constexpr (KH == 2) {
        if (kh == 1u) stage_sums(false);
        __syncthreads();
        if (kh == 0u) stage_sums(true);
    } else {
        stage_sums(false);
    }
    __syncthreads();
    const bool gated = p.activation == kActSiluGate;
    const uint32_t ch = tid & 15u;  // 8 columns: 8 ch .. 8 ch + 7 of the tile
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
    // the thread's 8 sums of tile row `row`, as staged
    auto staged = [&](uint32_t row, float (&v)[8]) {
        const float* src = c_rows(row >> 5) + (row & 31u) * kTw + 8u * ch;
        const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
        v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    };
    // bias, gate, residual, rounding and the store of 8 finished sums of global row gm
    auto finish = [&](uint32_t gm, float (&v)[8]) {
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
            *reinterpret_cast<uint2*>(p.c + (size_t)gm * p.ldc + gn / 2u) = make_uint2(pack_bf16_rne(o[0], o[1]), pack_bf16_rne(o[2], o[3]));
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
                make_uint4(pack_bf16_rne(v[0], v[1]), pack_bf16_rne(v[2], v[3]), pack_bf16_rne(v[4], v[5]), pack_bf16_rne(v[6], v[7]));
        }
    };
    auto finish_tile = [&]() {
#pragma unroll
        for (uint32_t pass = 0; pass < 8u / KH; ++pass) {
            const uint32_t row = 16u * KH * pass + (tid >> 4);
            if (m0 + row >= p.m || gn >= p.n) continue;
            float v[8];
            staged(row, v);
            finish(m0 + row, v);
        }
    };
    if (p.splits == 1u) {
        finish_tile();
        return;
    }
    // ---- split-K: the protocol of the decode kernels.  The workspace holds one fp32 word per (split but the last, row,
    // column), kEmptyWord at rest.  Producers write their sums with device-scope stores and are done; the workgroup of the
    // last split (dispatched after them: blockIdx.y is the slow index) fetches them, again while any word is still empty,
    // adds them in split order with its own sums last, finishes the outputs and leaves the words empty.  Only it waits, and
    // only on workgroups that wait for nothing; the wait is bounded all the same.
    // Who moves what: thread t has the four columns 4 (t % 32) .. + 3 of tile rows t / 32 + kHStride i, i = 0 .. kHeld - 1, so that one
    // instruction of a wave covers two whole rows of the tile (512 contiguous bytes each): whole cache lines go out and come
    // in.  What the hand-over costs all the same is the reducing workgroup's fetch: 64 KiB per split through one CU, which
    // draws some 15-20 GB/s from beyond its L2 (3-5 us per split; measured with the fetch, the producers' stores and the
    // emptying switched off in turn), plus about 6 us for the producers' stores to arrive.
    const __amdgpu_buffer_rsrc_t ws = __builtin_amdgcn_make_buffer_rsrc(p.partials, 0, (int)p.partial_bytes, kBufferFlags);
    const uint32_t split_bytes = p.m * p.n * 4u;
    constexpr uint32_t kHStride = 8u * KH, kHeld = 16u / KH;
    const uint32_t hrow = tid >> 5, hcol = 4u * (tid & 31u);
    const uint32_t rows_here = p.m - m0 < kTw ? p.m - m0 : kTw;  // rows of this tile that exist
    const uint32_t mine = (n0 + hcol < p.n && hrow < rows_here) ? (rows_here - hrow + kHStride - 1u) / kHStride : 0u;  // of the thread's kHeld rows
    auto word_off = [&](uint32_t i) { return ((m0 + hrow + kHStride * i) * p.n + n0 + hcol) * 4u; };
    auto held = [&](uint32_t i) -> float4* {
        const uint32_t row = hrow + kHStride * i;
        return reinterpret_cast<float4*>(c_rows(row >> 5) + (row & 31u) * kTw + hcol);
    };
    if (ks != p.splits - 1u) {
        if (p.debug_flags & kDebugWithholdPartials) return;  // test hook: lets the reducer's wait run out
#pragma unroll
        for (uint32_t i = 0; i < kHeld; ++i) {
            if (i >= mine) continue;
            const float4 v = *held(i);
            const u32x4_t w4 = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
            __builtin_amdgcn_raw_buffer_store_b128(w4, ws, (int)word_off(i), (int)(ks * split_bytes), kAuxDeviceScope);
        }
        return;
    }
    float4 total[kHeld];
#pragma unroll
    for (uint32_t i = 0; i < kHeld; ++i) total[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    // First wait, at the price of one word per thread and split, until the producers' last stores show: a fetch of whole
    // tiles that comes too early moves 64 KiB per split of nothing through this CU.  (What a thread stored last is not
    // bound to arrive last: the fetch below checks every word on its own.)
    uint32_t fetch_limit = p.split_wait_limit;
    if (mine != 0u) {
        bool there = false;
        for (uint32_t tries = 0; !there && tries < p.split_wait_limit; ++tries) {
            if (tries) __builtin_amdgcn_s_sleep(2);
            asm volatile("" ::: "memory");
            there = true;
            for (uint32_t sp = 0; sp + 1u < p.splits; ++sp) {
                const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(ws, (int)word_off(mine - 1u), (int)(sp * split_bytes), kAuxDeviceScope);
                if (v[3] == kEmptyWord) there = false;
            }
        }
        if (!there) fetch_limit = 1u;  // the wait has run out: one fetch of what there is, no second wait of that length
    }
    for (uint32_t sp = 0; sp + 1u < p.splits; sp += 2u) {
        // two splits' words of all the thread's rows are fetched together (more bytes in flight per CU, fewer round trips),
        // and fetched again together while any is empty
        const bool pair = sp + 2u < p.splits;  // the same for every thread
        u32x4_t w[2][kHeld];
        // bit 16 j + i: words (j, i) are wanted and have not been seen complete yet; only those are fetched again
        uint32_t missing = 0u;
#pragma unroll
        for (uint32_t i = 0; i < kHeld; ++i)
            if (i < mine) missing |= (1u << i) | (pair ? 1u << (16u + i) : 0u);
        for (uint32_t tries = 0; missing != 0u && tries < fetch_limit; ++tries) {
            if (tries) __builtin_amdgcn_s_sleep(2);
            asm volatile("" ::: "memory");  // other workgroups write these words: every attempt really loads
#pragma unroll
            for (uint32_t j = 0; j < 2; ++j)
#pragma unroll
                for (uint32_t i = 0; i < kHeld; ++i)
                    if (missing & (1u << (16u * j + i)))
                        w[j][i] = __builtin_amdgcn_raw_buffer_load_b128(ws, (int)word_off(i), (int)((sp + j) * split_bytes), kAuxDeviceScope);
#pragma unroll
            for (uint32_t j = 0; j < 2; ++j)
#pragma unroll
                for (uint32_t i = 0; i < kHeld; ++i)
                    if ((missing & (1u << (16u * j + i))) && w[j][i][0] != kEmptyWord && w[j][i][1] != kEmptyWord && w[j][i][2] != kEmptyWord &&
                        w[j][i][3] != kEmptyWord)
                        missing &= ~(1u << (16u * j + i));
        }
        const bool complete = missing == 0u;
        // a word that never arrived is still the empty pattern, a NaN, and turns its sum into one; the workspace's header
        // remembers that it happened
        if (!complete) __hip_atomic_store(p.ws_header, kWorkspaceGaveUp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (uint32_t j = 0; j < 2; ++j)  // in split order
#pragma unroll
            for (uint32_t i = 0; i < kHeld; ++i) {
                if (i >= mine || (j == 1u && !pair)) continue;
                total[i].x += __uint_as_float(w[j][i][0]);
                total[i].y += __uint_as_float(w[j][i][1]);
                total[i].z += __uint_as_float(w[j][i][2]);
                total[i].w += __uint_as_float(w[j][i][3]);
            }
    }
    // the other splits' sums plus this workgroup's own, back where the finishing pass takes them from
#pragma unroll
    for (uint32_t i = 0; i < kHeld; ++i) {
        if (i >= mine) continue;
        float4* own = held(i);
        const float4 o = *own;
        *own = make_float4(total[i].x + o.x, total[i].y + o.y, total[i].z + o.z, total[i].w + o.w);
    }
    __syncthreads();
    finish_tile();
    // the words this workgroup consumed are empty again for the next launch (last: nothing waits for these stores)
    const u32x4_t empty4 = {kEmptyWord, kEmptyWord, kEmptyWord, kEmptyWord};
    for (uint32_t sp = 0; sp + 1u < p.splits; ++sp) {
#pragma unroll
        for (uint32_t i = 0; i < kHeld; ++i)
            if (i < mine) __builtin_amdgcn_raw_buffer_store_b128(empty4, ws, (int)word_off(i), (int)(sp * split_bytes), kAuxDeviceScope);
    }
}

template <int BITS, bool GROUPED, bool PACKED>
static hipError_t launch_prefill128_wreg_t(const GemmParams& p, hipStream_t stream)
{
    const uint32_t tiles = ((p.m + kTw - 1) / kTw) * ((p.n + kTw - 1) / kTw);
    const uint32_t grid = (tiles + 7u) / 8u * 8u;  // a whole number of workgroups per XCD; ids past the last tile exit at once
    // two waves per column group; with grouped scales, the copying wave on top
    // (at most 64 rows in all: the form that multiplies only the first four blocks of 16 rows)
    void (*kernel)(const GemmParams) = p.m <= 64u ? bfaintb_prefill128_wreg_kernel<BITS, GROUPED, PACKED, 2, GROUPED, 4>
                                                  : bfaintb_prefill128_wreg_kernel<BITS, GROUPED, PACKED, 2, GROUPED, 8>;
    return launch_kernel(kernel, dim3(grid, p.splits, 1), dim3(512 + (GROUPED ? 64 : 0), 1, 1), 0, stream, p);
}

// Whether this kernel can serve a launch: this library's own arithmetic (either order of the weights).
bool prefill128_wreg_serves(const GemmParams& p) { return !p.reference_arith; }

template <bool PACKED>
static hipError_t launch_prefill128_wreg_order(const GemmParams& p, int bits, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    if (bits == 8) return grouped ? launch_prefill128_wreg_t<8, true, PACKED>(p, stream) : launch_prefill128_wreg_t<8, false, PACKED>(p, stream);
    return grouped ? launch_prefill128_wreg_t<4, true, PACKED>(p, stream) : launch_prefill128_wreg_t<4, false, PACKED>(p, stream);
}

// packed: p.b is the buffer in the packed order (p.ldb_bytes is unused)
hipError_t launch_prefill128_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream)
{
    return packed ? launch_prefill128_wreg_order<true>(p, bits, stream) : launch_prefill128_wreg_order<false>(p, bits, stream);
}

}  // namespace bfaintb
