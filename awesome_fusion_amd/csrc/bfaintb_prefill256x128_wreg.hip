// Tiled variant, tiles of 256 rows x 128 columns, weights kept in registers: between the 128x128 tiles (at most 256 of
// them, one per CU) and the 256x256 tiles (which want several hundred to fill the machine) lie shapes with 257 .. 512
// small tiles, where the large tiles occupy a quarter to a half of the CUs and the small ones need a second round.  Tall
// tiles halve the small tiles' count and keep their structure (bfaintb_prefill128_wreg_kernel, whose comments apply):
//   256 threads = 4 waves, two by two: a wave owns 128 rows x 64 columns = 8 x 4 accumulators of
//   v_mfma_f32_16x16x32_bf16 and converts the weights of its 64 columns (the two waves above one another convert the
//   same ones: the vector unit has the room, LDS has not — four waves side by side would each read all of A).  Four
//   matrix instructions per A fragment read, two per converted weight.
//   A and the codes come in by the asynchronous copy, three steps ahead, into four stages each: 4 x 32 KiB of A
//   (256 rows x 64 k) and 4 x 8 KiB of codes: all 160 KiB of a CU's LDS.
//   A K-step is 16 units (block of 32 k, row block) of four fenced slots: the matrix instruction of each of the wave's
//   four column groups; around them the fragment of four units ahead, the code reads and the conversion of the next
//   step's weights (two pairs per unit) and two memory requests.
// Same reference kernel replaced (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:184-630), same order of addition
// per output as every other tiled kernel here (ascending k), so the same bits.  No split along k.  Row-major B, or B in
// the packed order (PACKED: what changes is said where the codes are copied and read).
#include <utility>
#include "bfaintb_device.hpp"

namespace bfaintb {

namespace {
constexpr uint32_t kTh = 256, kTw = 128, kTwK = 64;  // rows, columns, k per step
constexpr uint32_t kThStage = 256 * 128;     // bytes of one A stage
constexpr uint32_t kThCodeStage = 64 * 128;  // bytes of one stage of codes (8-bit; half of it used by 4-bit codes)

__device__ __forceinline__ uint32_t th_swz(uint32_t row, uint32_t chunk) { return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4); }

// acc += a x b with the accumulator pinned to the accumulation registers and updated in place.  Written as assembly
// because the compiler, left to itself with 128 accumulator registers, gives the instruction a destination other than
// its source and copies the sums back between steps (680 accumulator moves in the first build of this kernel).  What
// its hazard bookkeeping cannot see behind the assembly is kept safe by construction: the operands are written (LDS
// reads, conversions) long before, under wait counts the compiler does insert for assembly operands; the accumulators
// are written by ordinary instructions only at the very start (the whole prologue lies between that and the first
// matrix instruction) and read by them only in the epilogue, behind explicit idle cycles (th_settle).
__device__ __forceinline__ void th_mfma(f32x4_t& acc, const bf16x8_t& a, const bf16x8_t& b)
{
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void th_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
}  // namespace

template <int BITS, bool GROUPED, bool PACKED>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) bfaintb_prefill256x128_wreg_kernel(const GemmParams p)
{
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a0[kThStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a1[kThStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a2[kThStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_a3[kThStage];
    constexpr uint32_t kRowBytes = 128u * BITS / 8u;  // a tile row of codes
    // (the codes of one K-step: 64 rows; the arrays keep the 8-bit extent for both code widths — an extent that depends
    // on a template parameter, in an array the lambdas below capture, makes the host pass drop the kernel's launch
    // stub without a diagnostic)
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w0[kThCodeStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w1[kThCodeStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w2[kThCodeStage];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_w3[kThCodeStage];
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
    const uint32_t wr = wave >> 1, wc = wave & 1u;  // the wave's 128 rows x 64 columns of the tile
    const uint32_t c16 = lane & 15u, kq = lane >> 4;

    // ---- tile of this workgroup (the order of bfaintb_prefill128_kernel: the ids an XCD receives cover consecutive
    //      logical ids, which walk groups of 8 tile-rows column by column)
    //      Or, with p.tile_count set: the left and right halves of the 256x256 tiles p.tile_first .. + p.tile_count - 1 in the
    //      order of bfaintb_prefill_wreg_kernel — the thin last round that kernel leaves to this one.
    const uint32_t tiles_m = (p.m + kTh - 1) / kTh, tiles_n = (p.n + kTw - 1) / kTw;
    uint32_t m0, n0;
    if (p.tile_count != 0u) {
        const uint32_t wgs = 2u * p.tile_count;
        const uint32_t per_xcd = (wgs + 7u) / 8u;
        const uint32_t local = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
        if (local >= wgs) return;
        const uint32_t big = p.tile_first + (local >> 1), big_n = (p.n + 255u) / 256u;
        const uint32_t group = big / (4u * big_n);
        const uint32_t first_m = group * 4u;
        const uint32_t group_rows = tiles_m - first_m < 4u ? tiles_m - first_m : 4u;
        const uint32_t in_group = big - group * 4u * big_n;
        m0 = (first_m + in_group % group_rows) * kTh;
        n0 = (in_group / group_rows) * 256u + (local & 1u) * kTw;
        if (n0 >= p.n) return;  // the right half of a last, narrow tile
    } else {
        const uint32_t wgs = tiles_m * tiles_n;
        const uint32_t per_xcd = (wgs + 7u) / 8u;
        const uint32_t logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
        if (logical >= wgs) return;
        const uint32_t group = logical / (8u * tiles_n);
        const uint32_t first_m = group * 8u;
        const uint32_t group_rows = tiles_m - first_m < 8u ? tiles_m - first_m : 8u;
        const uint32_t in_group = logical - group * 8u * tiles_n;
        m0 = (first_m + in_group % group_rows) * kTh;
        n0 = (in_group / group_rows) * kTw;
    }

    const uint32_t rows_valid = p.m - m0 < kTh ? p.m - m0 : kTh;
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

    const uint32_t ksteps_all = (p.k + kTwK - 1u) / kTwK;
    const uint32_t ksteps = ksteps_all;
    constexpr uint32_t kbase = 0u;
    const uint32_t last_chunks = (p.k - (ksteps_all - 1u) * kTwK) / 8u;  // valid 16-byte chunks per row of A in the last step
    auto clamp = [&](uint32_t t) { return t < ksteps ? t : ksteps - 1u; };

    // A copy: instruction j (of 8) of wave w fills rows 64 w + 8 j .. + 7; lane l lands at row + l / 8, chunk position l % 8, so
    // it fetches chunk (l % 8) ^ ((row >> 1) & 7) = (l % 8) ^ (l / 16) for even j and that ^ 4 for odd j; the row advance
    // of j and the K advance sit in the scalar offset.  A chunk past the end of k (partial last step) is fetched from
    // beyond the extent and reads as zero; rows of B past k read as zero codes, finite weights, and multiply those zeros.
    const uint32_t a_row = 64u * wave + (lane >> 3);
    const uint32_t chunk_e = (lane & 7u) ^ ((lane >> 4) & 7u), chunk_o = chunk_e ^ 4u;
    const uint32_t a_voff_e = (a_row * p.lda + chunk_e * 8u) * 2u, a_voff_o = (a_row * p.lda + chunk_o * 8u) * 2u;
    const uint32_t a_last_e = chunk_e < last_chunks ? a_voff_e : a_extent, a_last_o = chunk_o < last_chunks ? a_voff_o : a_extent;
    auto dma_a = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = a_tile(stage_c) + wave * 8192u;
        const bool last = kbase + kt + 1u == ksteps_all;
        const uint32_t ve = last ? a_last_e : a_voff_e, vo = last ? a_last_o : a_voff_o;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16,
                                                     (j & 1u) ? vo : ve, (kbase + kt) * kTwK * 2u + j * 16u * p.lda, 0, 0);
    };

    // W codes.  Copy: a 16-byte-per-lane instruction fills 1024 bytes = kRowsPerCopy rows of the stage; the step's 64
    // rows take kCopies instructions, kCopiesPerWave for each wave.  Lane l lands at row l / kChunks of its block, chunk
    // position l % kChunks, and fetches the chunk the rotation puts there: position = chunk + kRot * (row / 8 % 4).
    constexpr uint32_t kChunks = kRowBytes / 16u;        // 8 or 4 chunks per row
    constexpr uint32_t kRowsPerCopy = 1024u / kRowBytes; // 8 or 16
    //
    // Packed weights: the chunk of a column block that holds the step (1024 bytes: all of it for 8-bit codes; for 4-bit
    // codes it spans two steps and is copied for each) is one instruction; wave w copies column blocks 2 w and 2 w + 1.
    // The chunk's 16-byte pieces are the lanes of the packed order: piece 16 kg + nl = rows 8 kg .. + 7 of both K-blocks
    // (4-bit: of four), column nl.  This kernel's lane (c16, kq) wants columns nl = 4 (c16 % 4) + j, j = 0 .. 3, of column
    // block 4 wc + c16 / 4: pieces 16 kq + nl.  So that a wave reads each j with one conflict-free instruction, piece
    // 16 g + 4 c + j of column block b is stored at position 16 j + 4 (g ^ (b % 4)) + c: the 16 lanes of one kq then read
    // 16 neighbouring pieces' worth of banks.
    constexpr uint32_t kCopiesPerWave = PACKED ? 2u : 64u / kRowsPerCopy / 4u;  // 2 or 1
    constexpr uint32_t kRot = BITS == 8 ? 4u : 2u;       // a wave's 16 lanes of one kq cover 64 (32) bytes of a row
    uint32_t w_voff[2];  // (fixed extent: see the note on the arrays above)
#pragma unroll
    for (uint32_t j = 0; j < kCopiesPerWave; ++j) {
        if constexpr (PACKED) {
            const uint32_t b = 2u * wave + j;
            const uint32_t g = ((lane >> 2) & 3u) ^ (b & 3u);
            w_voff[j] = b * slab_bytes + (16u * g + 4u * (lane & 3u) + (lane >> 4)) * 16u;
        } else {
            const uint32_t row = (kCopiesPerWave * wave + j) * kRowsPerCopy + lane / kChunks;  // within the step
            const uint32_t chunk = ((lane % kChunks) - kRot * ((row >> 3) & 3u)) & (kChunks - 1u);
            w_voff[j] = row * p.ldb_bytes + chunk * 16u;
        }
    }
    // where step kt's codes start, beyond the lane's offset: w_step * (kt >> w_shift)  (spelt out at the two copies: with
    // a lambda for it among the copy's arguments the host pass drops the kernel's launch stub without a diagnostic)
    const uint32_t w_step = PACKED ? 1024u : kTwK * p.ldb_bytes;
    constexpr uint32_t w_shift = (PACKED && BITS == 4) ? 1u : 0u;
    auto dma_w = [&](auto stage_c, uint32_t kt) {
        uint8_t* base = w_tile(stage_c) + kCopiesPerWave * wave * 1024u;
#pragma unroll
        for (uint32_t j = 0; j < kCopiesPerWave; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)(base + j * 1024u), 16, w_voff[j],
                                                     ((kbase + kt) >> w_shift) * w_step, 0, 0);
    };
    // Pick: this lane's 4 columns (byte offset wbyte of a row), rows 8 kq .. 8 kq + 7 of block blk of 32 k: row
    // 32 blk + 8 kq + r, whose block of 8 is 4 blk + kq, rotation kRot * kq.  One read per row: ds_read_b32 (u16 for
    // 4-bit codes), column j of the four in byte (nibble) j.
    const uint32_t wcol = 64u * wc + 4u * c16;  // within the tile
    const uint32_t wbyte = wcol * BITS / 8u;
    // (packed: the piece of the lane's first column; column j's is 256 j bytes on; 4-bit codes: + 8 in odd steps)
    const uint32_t w_rd = PACKED ? (4u * wc + (c16 >> 2)) * 1024u + ((4u * (kq ^ (c16 >> 2)) + (c16 & 3u)) << 4)
                                 : (8u * kq) * kRowBytes + ((((wbyte >> 4) + kRot * kq) & (kChunks - 1u)) << 4) + (wbyte & 15u);  // + 32 blk rows + r rows
    // Packed codes of a step as a lane reads them: [column j][K-block][half]: 8-bit codes: rows 4 half .. + 3 in the bytes
    // of a dword; 4-bit codes: [j][K-block][0] holds the 8 rows in its nibbles.
    struct PackedCodes {
        uint32_t d[4][2][2];
    };
    auto read_packed = [&](PackedCodes& pc, const uint8_t* src, uint32_t kt, uint32_t j) {  // src: the stage + w_rd
        if constexpr (BITS == 8) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src + 256u * j);
            pc.d[j][0][0] = v[0], pc.d[j][0][1] = v[1], pc.d[j][1][0] = v[2], pc.d[j][1][1] = v[3];
        } else {
            const u32x2_t v = *reinterpret_cast<const u32x2_t*>(src + 256u * j + 8u * ((kbase + kt) & 1u));
            pc.d[j][0][0] = v[0], pc.d[j][1][0] = v[1];
        }
    };
    // 4-bit: the two's-complement nibbles of a dword of 8 rows: even rows in the low nibbles of `ev`'s bytes, odd rows of `od`'s
    struct PackedNibbles {
        uint32_t ev[4][2], od[4][2];  // [column j][K-block]
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
    auto read_code = [&](const uint8_t* tile, uint32_t blk, uint32_t r) -> uint32_t {
        if constexpr (BITS == 8) return *reinterpret_cast<const uint32_t*>(tile + (32u * blk + r) * kRowBytes);
        else return *reinterpret_cast<const uint16_t*>(tile + (32u * blk + r) * kRowBytes);
    };
    // Scales go through a buffer resource so that the load is issued whatever the lane's column (the wait counts
    // below count requests): columns past n read other columns' scales, or zero beyond the array; their results are
    // never stored.
    const uint32_t scale_rows = GROUPED ? p.k / p.group_size : 1u;
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(p.scale), 0, (int)(((scale_rows - 1u) * p.lds + p.n) * 2u), kBufferFlags);
    const uint32_t s_voff = (n0 + wcol) * 2u;
    struct ScaleRaw {
        u32x2_t v[2];  // [block of 32 k]: the four columns' bf16 scales
    };
    auto block_group_scales = [&](ScaleRaw& sr, uint32_t kt, uint32_t blk) {
        uint32_t g = group_of_row(p, (kbase + kt) * kTwK + 32u * blk);
        if (g >= scale_rows) g = scale_rows - 1u;  // rows past k in a partial last step: any scale will do
        sr.v[blk] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, s_voff, g * p.lds * 2u, 0);
    };
    auto group_scales = [&](ScaleRaw& sr, uint32_t kt) {
        block_group_scales(sr, kt, 0);
        block_group_scales(sr, kt, 1);
    };
    auto widen_scales = [&](float (&out)[4], const u32x2_t& raw) {
        out[0] = make_col_scale_nibble<BITS>(raw[0] & 0xffffu);
        out[1] = make_col_scale_nibble<BITS>(raw[0] >> 16);
        out[2] = make_col_scale_nibble<BITS>(raw[1] & 0xffffu);
        out[3] = make_col_scale_nibble<BITS>(raw[1] >> 16);
    };
    float cs[4] = {0.f, 0.f, 0.f, 0.f};  // one scale per column: fixed
    if constexpr (!GROUPED) widen_scales(cs, __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, s_voff, 0, 0));
    struct Ops {
        uint32_t w[2][4][4];  // [block of 32 k][column j][dword]: the 8-element operand as 4 packed pairs
    };
    // the four codes of a read, ready for the conversion: as stored (8-bit codes: the excess of 128 comes off in the
    // multiplication, see scaled()); two's-complement nibbles, columns 0 and 2 in the low nibbles of bytes 0 and 1 of `e`,
    // columns 1 and 3 likewise in `o` (4-bit codes)
    struct Pre {
        uint32_t e, o;
    };
    auto prepare = [&](uint32_t x) -> Pre {
        Pre q;
        if constexpr (BITS == 8) {
            q.e = x;
            q.o = x;
        } else {
            q.e = x ^ 0x8888u;
            q.o = q.e >> 4;
            asm("" : "+v"(q.o));  // keep the shifted word: its bytes are picked by the conversion's own byte select
        }
        return q;
    };
    auto value = [&](const Pre& q, uint32_t j) -> float {
        if constexpr (BITS == 8) return (float)((q.e >> (8u * j)) & 0xffu);  // v_cvt_f32_ubyte0 .. 3
        else return j == 0 ? nibble_to_f32_sixteenth<0>(q.e) : j == 1 ? nibble_to_f32_sixteenth<0>(q.o) : j == 2 ? nibble_to_f32_sixteenth<1>(q.e) : nibble_to_f32_sixteenth<1>(q.o);
    };
    // value x scale.  8-bit codes: u s - 128 s in one fused operation — u s (8 x 8 bits), 128 s and their difference
    // (u - 128) s are all exact in fp32, so this is the product q s of the signed code, bit for bit (a zero code gives +0
    // where q s gives -0 for a negative scale: no sum can tell), and the sign flip of the codes is saved.
    auto scaled = [&](float f, float scale) -> float {
        if constexpr (BITS == 8) return __builtin_fmaf(f, scale, -128.0f * scale);
        else return f * scale;
    };
    auto block_scales = [&](float (&sc)[2][4], const ScaleRaw& sr) {
#pragma unroll
        for (uint32_t blk = 0; blk < 2; ++blk) {
            if constexpr (GROUPED) {
                widen_scales(sc[blk], sr.v[blk]);
            } else {
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) sc[blk][j] = cs[j];
            }
        }
    };
    // the operands of a whole step at once (the prologue's: step 0)
    auto convert_all = [&](Ops& ops, auto stage_c, const ScaleRaw& sr) {
        const uint8_t* tile = w_tile(stage_c) + w_rd;
        float sc[2][4];
        block_scales(sc, sr);
        if constexpr (PACKED) {
            PackedCodes pc;
            PackedNibbles nb;
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) read_packed(pc, tile, 0, j);
#pragma unroll
            for (uint32_t v = 0; v < 32; ++v) {
                const uint32_t blk = v >> 4, j = (v >> 2) & 3u, pr = v & 3u;
                float f0, f1;
                packed_values(pc, nb, blk, j, pr, f0, f1);
                ops.w[blk][j][pr] = pack_bf16_rne(scaled(f0, sc[blk][j]), scaled(f1, sc[blk][j]));
            }
            return;
        }
#pragma unroll
        for (uint32_t blk = 0; blk < 2; ++blk)
#pragma unroll
            for (uint32_t pr = 0; pr < 4; ++pr) {
                const Pre q0 = prepare(read_code(tile, blk, 2u * pr)), q1 = prepare(read_code(tile, blk, 2u * pr + 1u));
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) ops.w[blk][j][pr] = pack_bf16_rne(scaled(value(q0, j), sc[blk][j]), scaled(value(q1, j), sc[blk][j]));
            }
    };

    f32x4_t acc[8][4];
#pragma unroll
    for (int mt = 0; mt < 8; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[mt][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // fragment (mt, blk): row 128 wr + 16 mt + c16 of the tile, chunk 4 blk + kq (the swizzle repeats every 16 rows)
    bf16x8_t af[4];  // the fragments of the next few units, carried from step to step
    uint32_t a_rd[2];
#pragma unroll
    for (uint32_t blk = 0; blk < 2; ++blk) a_rd[blk] = th_swz(c16, 4u * blk + kq) + wr * 16384u;

    // One K-step.  `cur`: the operands of this step; `nxt` receives those of step kt + 1, converted from the codes in stage
    // S + 1; stage S holds this step's A; the copies of step kt + 3 go into stage S + 3 = S - 1, which every wave finished
    // reading (A during step kt - 1, the codes during step kt - 2) before the barrier at the top.  `s1`: the group scales
    // of step kt + 1 (requested one step ago), `s2` receives those of step kt + 2.
    // 16 units u = (block of 32 k, row block) of four fenced slots, one matrix instruction each (the wave's four column
    // groups).  Around them, per unit: the A fragment of unit u + kAhead (the last kAhead units fetch the next step's
    // first fragments); two of the 32 conversion pairs of the next step's weights (pair v = block v / 16, rows 2 (v / 4 % 4),
    // + 1, column v % 4: slots 0 and 2 flip signs and convert, slots 1 and 3 scale and round); in even units the two code
    // reads of the row pair two ahead; in slots 1 and 3 one memory request (the group scales, then the 8 copies of A, then
    // those of the codes).
    constexpr uint32_t kAhead = 4;
    constexpr uint32_t kUnits = 16;
    auto step = [&](auto stage_c, uint32_t kt, const Ops& cur, Ops& nxt, const ScaleRaw& s1, ScaleRaw& s2) {
        constexpr uint32_t S = decltype(stage_c)::value;
        using Next = std::integral_constant<uint32_t, (S + 1u) & 3u>;
        using Target = std::integral_constant<uint32_t, (S + 3u) & 3u>;
        // At most the requests of the step before this one may still be in flight: then this wave's part of this step's
        // AND the next step's A (requested three and two steps ago) and of the next step's codes (two steps ago) has
        // landed.  Behind the barrier every wave's has.
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 + kCopiesPerWave + (GROUPED ? 2 : 0)) : "memory");
        barrier_no_fence();  // (a fenced barrier would also wait for the copies of the steps ahead)
        const uint32_t kt3 = clamp(kt + 3), kt2 = clamp(kt + 2);
        const bool last3 = kbase + kt3 + 1u == ksteps_all;
        const uint32_t ve = last3 ? a_last_e : a_voff_e, vo = last3 ? a_last_o : a_voff_o;
        uint8_t* const a_dst = a_tile(Target{}) + wave * 8192u;
        uint8_t* const w_dst = w_tile(Target{}) + kCopiesPerWave * wave * 1024u;
        const uint8_t* const a_src = a_tile(stage_c);
        const uint8_t* const a_nxt = a_tile(Next{});
        const uint8_t* const w_src = w_tile(Next{}) + w_rd;
        uint32_t code[2][8];   // the codes of step kt + 1 as read: [block][row], four codes each
        Pre pre[2];            // the two rows of the pair at hand
        PackedCodes pc;        // ... or, from packed weights, the lane's 4 x 16 (8) bytes
        PackedNibbles nb;
        float sc[2][4];
        float f0 = 0.f, f1 = 0.f;
        block_scales(sc, s1);
        auto read_rows = [&](uint32_t g) {  // row pair g = (block g / 4, rows 2 (g % 4), + 1)
            const uint32_t blk = g >> 2, pr = g & 3u;
            code[blk][2u * pr] = read_code(w_src, blk, 2u * pr);
            code[blk][2u * pr + 1u] = read_code(w_src, blk, 2u * pr + 1u);
        };
        if constexpr (PACKED) {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) read_packed(pc, w_src, kt + 1u, j);
        } else {
            read_rows(0);
            read_rows(1);
        }
        __builtin_amdgcn_sched_barrier(0);
        // (the group scales first: the next step waits for them at its very start, and that wait then leaves the copies
        // requested behind them in flight — requested last, they made it a wait for everything)
        auto request = [&](uint32_t slot) {  // the memory request of the step's slot-th request slot
            // (one block's scales per slot: finding a group is a chain of five scalar instructions)
            constexpr uint32_t kFirstCopy = GROUPED ? 2u : 0u;
            if (GROUPED && slot < 2) {
                block_group_scales(s2, kt2, slot);
            } else if (slot >= kFirstCopy && slot < kFirstCopy + 8) {
                const uint32_t q = slot - kFirstCopy;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(a_dst + q * 1024u), 16, (q & 1u) ? vo : ve,
                                                         (kbase + kt3) * kTwK * 2u + q * 16u * p.lda, 0, 0);
            } else if (slot >= kFirstCopy + 8 && slot < kFirstCopy + 8 + kCopiesPerWave) {
                const uint32_t q = slot - kFirstCopy - 8u;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)(w_dst + q * 1024u), 16, w_voff[q],
                                                         ((kbase + kt3) >> w_shift) * w_step, 0, 0);
            }
        };
#pragma unroll
        for (uint32_t u = 0; u < kUnits; ++u) {
            const uint32_t blk = u >> 3, mt = u & 7u;
            const bf16x8_t a_now = af[u % kAhead];
#pragma unroll
            for (uint32_t h = 0; h < 2; ++h) {  // the unit's two conversion pairs, two slots each
                const uint32_t v = 2u * u + h;
                const uint32_t cblk = v >> 4, cpr = (v >> 2) & 3u, cj = v & 3u;
                const uint32_t j0 = 2u * h, j1 = 2u * h + 1u;  // the slots' column groups
                const bf16x8_t wf0 = __builtin_bit_cast(bf16x8_t, make_uint4(cur.w[blk][j0][0], cur.w[blk][j0][1], cur.w[blk][j0][2], cur.w[blk][j0][3]));
                const bf16x8_t wf1 = __builtin_bit_cast(bf16x8_t, make_uint4(cur.w[blk][j1][0], cur.w[blk][j1][1], cur.w[blk][j1][2], cur.w[blk][j1][3]));
                // ---- first slot of the pair
                th_mfma(acc[mt][j0], a_now, wf0);
                if (h == 0) {
                    if (u + kAhead < kUnits) af[u % kAhead] = *reinterpret_cast<const bf16x8_t*>(a_src + a_rd[(u + kAhead) >> 3] + ((u + kAhead) & 7u) * 2048u);
                    else af[u % kAhead] = *reinterpret_cast<const bf16x8_t*>(a_nxt + a_rd[0] + (u + kAhead - kUnits) * 2048u);
                    if constexpr (!PACKED)
                        if ((u & 1u) == 0u && (u >> 1) + 2u < 8u) read_rows((u >> 1) + 2u);
                }
                if constexpr (PACKED) {
                    packed_values(pc, nb, cblk, cj, cpr, f0, f1);
                } else {
                    if (cj == 0) {
                        pre[0] = prepare(code[cblk][2 * cpr]);
                        pre[1] = prepare(code[cblk][2 * cpr + 1]);
                    }
                    f0 = value(pre[0], cj);
                    f1 = value(pre[1], cj);
                }
                __builtin_amdgcn_sched_barrier(0);
                // ---- second slot
                th_mfma(acc[mt][j1], a_now, wf1);
                request(2u * u + h);
                nxt.w[cblk][cj][cpr] = pack_bf16_rne(scaled(f0, sc[cblk][cj]), scaled(f1, sc[cblk][cj]));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // ---- prologue: A tiles and codes of steps 0, 1, 2 -> stages 0, 1, 2; operands of step 0
    Ops ops0, ops1;
    ScaleRaw sa = {}, sb = {};  // group scales, alternating: sb = step 0 (then 2, ...), sa = step 1 (then 3, ...)
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
    convert_all(ops0, C0{}, sb);
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

    // ---- epilogue: fp32 sums -> LDS in [m][n] order, 128 rows at a time (rows 64 q .. 64 q + 63 of the half in the q-th A
    //      stage), then finished row-wise
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing asynchronous may still be writing LDS
    th_settle();                                       // the last matrix instructions have written their sums
    __syncthreads();                                   // ... and every wave is done reading the stages
    auto c_rows = [&](uint32_t q) -> float* { return reinterpret_cast<float*>(q == 0 ? lds_a0 : lds_a1); };
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
        const float* src = c_rows(row >> 6) + (row & 63u) * kTw + 8u * ch;
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
#pragma unroll
    for (uint32_t half = 0; half < 2; ++half) {
        if (half) __syncthreads();  // the first half has been read
        if (wr == half) {           // the half's rows are two waves' rows
#pragma unroll
            for (uint32_t mt = 0; mt < 8; ++mt) {
                float* base = c_rows(mt >> 2);
#pragma unroll
                for (uint32_t r = 0; r < 4; ++r) {
                    const uint32_t row = 16u * (mt & 3u) + 4u * kq + r;  // within the 64 rows of this array
                    *reinterpret_cast<float4*>(base + row * kTw + wcol) = make_float4(acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]);
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t pass = 0; pass < 8; ++pass) {
            const uint32_t row = 16u * pass + (tid >> 4);  // within the half
            const uint32_t gm = m0 + 128u * half + row;
            if (gm >= p.m || gn >= p.n) continue;
            float v[8];
            staged(row, v);
            finish(gm, v);
        }
    }
}

template <int BITS, bool GROUPED, bool PACKED>
static hipError_t launch_prefill256x128_wreg_t(const GemmParams& p, hipStream_t stream)
{
    const uint32_t tiles = p.tile_count != 0u ? 2u * p.tile_count : ((p.m + kTh - 1) / kTh) * ((p.n + kTw - 1) / kTw);
    const uint32_t grid = (tiles + 7u) / 8u * 8u;  // a whole number of workgroups per XCD; ids past the last tile exit at once
    void (*kernel)(const GemmParams) = bfaintb_prefill256x128_wreg_kernel<BITS, GROUPED, PACKED>;
    return launch_kernel(kernel, dim3(grid, 1, 1), dim3(256, 1, 1), 0, stream, p);
}

template <bool PACKED>
static hipError_t launch_prefill256x128_wreg_order(const GemmParams& p, int bits, hipStream_t stream)
{
    const bool grouped = p.group_size != 0;
    if (bits == 8) return grouped ? launch_prefill256x128_wreg_t<8, true, PACKED>(p, stream) : launch_prefill256x128_wreg_t<8, false, PACKED>(p, stream);
    return grouped ? launch_prefill256x128_wreg_t<4, true, PACKED>(p, stream) : launch_prefill256x128_wreg_t<4, false, PACKED>(p, stream);
}

// packed: p.b is the buffer in the packed order (p.ldb_bytes is unused)
hipError_t launch_prefill256x128_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream)
{
    if (p.reference_arith || p.splits != 1u) return hipErrorInvalidValue;  // this library's own arithmetic, k unsplit
    return packed ? launch_prefill256x128_wreg_order<true>(p, bits, stream) : launch_prefill256x128_wreg_order<false>(p, bits, stream);
}

}  // namespace bfaintb
