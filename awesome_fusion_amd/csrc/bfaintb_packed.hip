// Pre-packed weights: B reordered once, offline, into the operand order of v_mfma_f32_16x16x32_bf16, and the
// decode kernel that streams that order.
//
// The reference ships B to the device exactly as the host wrote it, row-major K x N
// (/root/reference/bfAintBGemm/mem_transfer.hpp:23-32, bfAintBGemm.cc:101-103), and its kernel re-reads
// it with a row stride (bf16gemm_kernel_gfx90a.s:239-262).  Row-major B forces a decode workgroup to own at
// least 128 columns (whole 128-byte lines per row), so n = 4096 yields 32 column blocks and the other CUs have
// to be filled by splitting K, with a second pass over partial sums.  In the packed order a block of 16 columns
// is one contiguous slab of k x 16 codes: n / 16 workgroups each stream their slab linearly and own their
// outputs outright — no split, no workspace, no second pass.
//
// Packed order ("mfma16"): column block nb = col / 16; K-chunks of R rows, R = 64 for 8-bit and 128 for 4-bit
// codes (k must be a multiple of R), kc = row / R, chunks = k / R.  Chunk (nb, kc) is 1024 bytes at
// (nb * chunks + kc) * 1024; lane l = 16 * kg + nl of a wave owns bytes 16 l .. 16 l + 15 of it:
//   8-bit codes: byte 8 h + r is B[64 kc + 32 h + 8 kg + r][16 nb + nl]                  (h = 0, 1; r = 0..7);
//   4-bit codes: byte 4 h + r / 2 holds, in nibble r & 1 (0 = low), B[128 kc + 32 h + 8 kg + r][16 nb + nl]  (h = 0..3).
//   So a lane's 16 bytes are, in order, its 8-element W operands of the chunk's K-blocks of 32 rows — column nl
//   of the block, rows 8 kg .. 8 kg + 7 of each K-block: one 128-bit load, no shuffling.
// Codes keep their stored form (excess-128 / excess-8); scales and bias are not reordered.
#include <type_traits>
#include "bfaintb_device.hpp"

namespace bfaintb {

namespace {

template <int BITS>
struct PackedFormat {
    static constexpr uint32_t kChunkRows = BITS == 8 ? 64u : 128u;
    static constexpr uint32_t kBlocks = kChunkRows / 32u;  // K-blocks (matrix instructions) per chunk
};

// byte offset in the packed payload of the code of (row, col); for 4-bit codes *nibble is 0 (low) or 1
template <int BITS>
__device__ __forceinline__ size_t packed_offset(uint32_t row, uint32_t col, uint32_t chunks, uint32_t* nibble)
{
    const uint32_t nb = col >> 4, nl = col & 15u;
    const uint32_t kc = row / PackedFormat<BITS>::kChunkRows, h = (row % PackedFormat<BITS>::kChunkRows) >> 5;
    const uint32_t kg = (row >> 3) & 3u, r = row & 7u;
    const size_t lane_slot = ((size_t)nb * chunks + kc) * 64u + 16u * kg + nl;
    if constexpr (BITS == 8) {
        *nibble = 0;
        return lane_slot * 16u + 8u * h + r;
    } else {
        *nibble = r & 1u;
        return lane_slot * 16u + 4u * h + (r >> 1);
    }
}

// one thread per packed byte: gathers its 1 or 2 codes from the row-major matrix
template <int BITS>
__global__ void __launch_bounds__(256) pack_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, uint32_t n, uint32_t k,
                                                   uint32_t ldb_bytes)
{
    const size_t total = (size_t)n * k * BITS / 8;
    const uint32_t chunks = k / PackedFormat<BITS>::kChunkRows;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t lane_slot = i >> 4;
        const uint32_t within = (uint32_t)(i & 15u);
        const uint32_t lane = (uint32_t)(lane_slot & 63u);
        const size_t chunk = lane_slot >> 6;
        const uint32_t kc = (uint32_t)(chunk % chunks), nb = (uint32_t)(chunk / chunks);
        const uint32_t nl = lane & 15u, kg = lane >> 4;
        const uint32_t col = 16u * nb + nl;
        if constexpr (BITS == 8) {
            const uint32_t h = within >> 3, r = within & 7u;
            const uint32_t row = 64u * kc + 32u * h + 8u * kg + r;
            dst[i] = src[(size_t)row * ldb_bytes + col];
        } else {
            const uint32_t h = within >> 2, r0 = (within & 3u) * 2u;
            const uint32_t row = 128u * kc + 32u * h + 8u * kg + r0;
            const uint32_t shift = (col & 1u) * 4u;
            const uint32_t lo = (src[(size_t)row * ldb_bytes + (col >> 1)] >> shift) & 15u;
            const uint32_t hi = (src[(size_t)(row + 1u) * ldb_bytes + (col >> 1)] >> shift) & 15u;
            dst[i] = (uint8_t)(lo | (hi << 4));
        }
    }
}

// one thread per row-major byte: the inverse
template <int BITS>
__global__ void __launch_bounds__(256) unpack_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, uint32_t n, uint32_t k,
                                                     uint32_t ldb_bytes)
{
    const uint32_t row_bytes = n * BITS / 8;
    const size_t total = (size_t)row_bytes * k;
    const uint32_t chunks = k / PackedFormat<BITS>::kChunkRows;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const uint32_t row = (uint32_t)(i / row_bytes), j = (uint32_t)(i % row_bytes);
        uint32_t nib;
        if constexpr (BITS == 8) {
            dst[(size_t)row * ldb_bytes + j] = src[packed_offset<8>(row, j, chunks, &nib)];
        } else {
            const size_t o0 = packed_offset<4>(row, 2u * j, chunks, &nib);
            const uint32_t lo = (src[o0] >> (4u * nib)) & 15u;
            const size_t o1 = packed_offset<4>(row, 2u * j + 1u, chunks, &nib);
            const uint32_t hi = (src[o1] >> (4u * nib)) & 15u;
            dst[(size_t)row * ldb_bytes + j] = (uint8_t)(lo | (hi << 4));
        }
    }
}

// Column-major B (n rows of k codes, k contiguous; 4-bit: byte j of a column holds rows 2j and 2j+1, low nibble first)
// -> the packed order.  A lane's 16 bytes of a chunk are whole runs of its column: 2 x 8 bytes (8-bit) or 4 x 4 bytes
// (4-bit, already in the packed nibble order), so this is a gather of aligned words.
template <int BITS>
__global__ void __launch_bounds__(256) pack_colmajor_kernel(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, uint32_t n, uint32_t k,
                                                            uint32_t ldb_bytes)
{
    const size_t slots = (size_t)n * k * BITS / 8 / 16;
    const uint32_t chunks = k / PackedFormat<BITS>::kChunkRows;
    for (size_t slot = (size_t)blockIdx.x * blockDim.x + threadIdx.x; slot < slots; slot += (size_t)gridDim.x * blockDim.x) {
        const uint32_t lane = (uint32_t)(slot & 63u);
        const size_t chunk = slot >> 6;
        const uint32_t kc = (uint32_t)(chunk % chunks), nb = (uint32_t)(chunk / chunks);
        const uint32_t nl = lane & 15u, kg = lane >> 4;
        const uint8_t* col = src + (size_t)(16u * nb + nl) * ldb_bytes;
        uint4 out;
        if constexpr (BITS == 8) {
            const uint2 h0 = *reinterpret_cast<const uint2*>(col + 64u * kc + 8u * kg);
            const uint2 h1 = *reinterpret_cast<const uint2*>(col + 64u * kc + 32u + 8u * kg);
            out = make_uint4(h0.x, h0.y, h1.x, h1.y);
        } else {
            const uint8_t* base = col + (128u * kc + 8u * kg) / 2u;
            out = make_uint4(*reinterpret_cast<const uint32_t*>(base), *reinterpret_cast<const uint32_t*>(base + 16u),
                             *reinterpret_cast<const uint32_t*>(base + 32u), *reinterpret_cast<const uint32_t*>(base + 48u));
        }
        *reinterpret_cast<uint4*>(dst + slot * 16u) = out;
    }
}

}  // namespace

hipError_t launch_pack_colmajor(uint8_t* dst, const uint8_t* src, uint32_t n, uint32_t k, uint32_t ldb_bytes, int bits, hipStream_t stream)
{
    const size_t slots = (size_t)n * k * (uint32_t)bits / 8 / 16;
    const uint32_t grid = (uint32_t)((slots + 255) / 256 < 65536 ? (slots + 255) / 256 : 65536);
    void (*kernel)(uint8_t*, const uint8_t*, uint32_t, uint32_t, uint32_t) = bits == 8 ? pack_colmajor_kernel<8> : pack_colmajor_kernel<4>;
    return launch_kernel(kernel, dim3(grid, 1, 1), dim3(256, 1, 1), 0, stream, dst, src, n, k, ldb_bytes);
}

hipError_t launch_pack(uint8_t* dst, const uint8_t* src, uint32_t n, uint32_t k, uint32_t ldb_bytes, int bits, bool unpack,
                       hipStream_t stream)
{
    const size_t total = (size_t)n * k * (uint32_t)bits / 8;
    const uint32_t grid = (uint32_t)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
    void (*kernel)(uint8_t*, const uint8_t*, uint32_t, uint32_t, uint32_t) =
        bits == 8 ? (unpack ? unpack_kernel<8> : pack_kernel<8>) : (unpack ? unpack_kernel<4> : pack_kernel<4>);
    return launch_kernel(kernel, dim3(grid, 1, 1), dim3(256, 1, 1), 0, stream, dst, src, n, k, ldb_bytes);
}

// ---------------------------------------------------------------------------------------------------------------
// Decode over packed weights.
//   grid = (n / 16, 1, ceil(m / (16 MB))); block = 8 waves.  A workgroup owns one column block (16 columns) and
//   MB blocks of 16 rows of A, over all of k; wave w takes the K-chunks w, w + 8, ... of the slab in batches: the
//   weight loads of a batch (one 128-bit load per chunk) and their activation loads are issued back to back, and
//   a wave keeps up to 8 KiB (8-bit) or 4 KiB (4-bit) of the slab in flight — large batches one at a time, or (long
//   k, per-channel scales) small batches with the next one loaded before the current one is converted.  Per K-block of 32
//   rows: one conversion of 8 weights and MB v_mfma_f32_16x16x32_bf16 with the operands swapped, as in the
//   row-major decode kernel (lane (nl, kg): W column nl, A row nl, rows 8 kg .. 8 kg + 7 of the K-block).  The
//   eight waves' accumulators meet in LDS and are added in wave order: the summation order is fixed.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kPackedWaves = 8;  // measured: 4 and 16 waves per workgroup are 12-19 % slower at n = k = 4096

// Chunks per batch.  Plain form: large batches, loaded and converted one at a time (for k up to 4096 with 8-bit codes
// a wave's only batch).  Pipelined form: small batches, two of them in flight, sized so that the raw chunks (4
// registers of codes, 4 per K-block and row block of activations) stay under about 100 registers — that kernel is
// held to 128 so that two workgroups share a CU.
__host__ __device__ constexpr int packed_batch(int bits, int mb, bool pipelined)
{
    if (!pipelined) return (bits == 8 ? 8 : 4) / mb;
    return bits == 8 ? (mb == 1 ? 3 : 2) : (mb == 1 ? 2 : 1);
}
// How a kernel instance finds its scales: one per output channel; one per K-chunk (groups are whole chunks), loaded
// with the chunk; one per K-block of 32 rows (groups of 32 or 64 rows), also loaded with the chunk.
enum { kScalePerChannel = 0, kScalePerChunk = 1, kScalePerBlock = 2 };

enum { kPackedPlain = 0, kPackedPipelined = 1, kPackedOneBatch = 2 };

template <int BITS, int SCALES, int MB, int MODE>
__device__ __forceinline__ void decode_packed_body(const GemmParams& p)
{
    constexpr uint32_t kBlocks = PackedFormat<BITS>::kBlocks;
    constexpr uint32_t kChunkRows = PackedFormat<BITS>::kChunkRows;
    constexpr bool GROUPED = SCALES != kScalePerChannel;
    constexpr uint32_t kScalesPerChunk = SCALES == kScalePerBlock ? PackedFormat<BITS>::kBlocks : 1u;
    constexpr bool PIPELINED = MODE == kPackedPipelined;
    constexpr int kBatch = packed_batch(BITS, MB, PIPELINED);
    __shared__ float red[kPackedWaves][MB][16][16 + 4];  // [wave][row block][A row][W column], rows padded

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t nl = lane & 15u, kg = lane >> 4;
    uint32_t nb = blockIdx.x;
    const uint32_t rb = blockIdx.z;
    if constexpr (GROUPED) {
        // Four neighbouring slabs share a 128-byte line of every row of scales.  Workgroups that follow one another in
        // dispatch order sit on different XCDs, each with an L2 of its own, and every one of the four fetched that line
        // from memory.  Within whole runs of 32 workgroups, the four that share an XCD (ids 8 apart) take four neighbouring slabs.
        const uint32_t run = nb & ~31u;
        if (run + 32u <= gridDim.x) nb = run + 4u * (nb & 7u) + ((nb >> 3) & 3u);
    }
    const uint32_t chunks = p.k / kChunkRows;

    const uint8_t* slab = p.b + ((size_t)nb * chunks) * 1024u + lane * 16u;
    const uint32_t col = 16u * nb + nl;
    const uint16_t* aptr[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        uint32_t arow = 16u * (MB * rb + mb) + nl;
        if (arow >= p.m) arow = p.m - 1u;  // rows past m repeat the last one; their sums are never stored
        aptr[mb] = p.a + (size_t)arow * p.lda + 8u * kg;
    }
    const uint16_t* sptr = p.scale + col;

    float cs = 0.f;
    if constexpr (!GROUPED) cs = make_col_scale<BITS>(*sptr);

    f32x4_t acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    struct Batch {
        uint4 w[kBatch];
        uint4 a[kBatch][kBlocks][MB];
        uint32_t s[kBatch][kScalesPerChunk];
    };
    // all loads of a batch, back to back (chunks past the end re-read the last one; compute() skips them)
    auto load = [&](Batch& b, uint32_t base) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            uint32_t c = base + (uint32_t)i * kPackedWaves;
            if (c >= chunks) c = chunks - 1u;
            // (non-temporal: read once, streamed past the caches' other contents)
            const u32x4_t wv = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(slab + (size_t)c * 1024u));
            b.w[i] = make_uint4(wv[0], wv[1], wv[2], wv[3]);
#pragma unroll
            for (uint32_t h = 0; h < kBlocks; ++h)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) b.a[i][h][mb] = *reinterpret_cast<const uint4*>(aptr[mb] + kChunkRows * c + 32u * h);
            if constexpr (GROUPED) {
#pragma unroll
                for (uint32_t h = 0; h < kScalesPerChunk; ++h) b.s[i][h] = sptr[(size_t)group_of_row(p, kChunkRows * c + 32u * h) * p.lds];
            }
        }
    };
    // GUARDED: the batch may reach past the last chunk (wave-uniform tests); whole batches run as one straight block
    auto compute = [&](const Batch& b, uint32_t base, auto guarded_c) {
        constexpr bool GUARDED = decltype(guarded_c)::value;
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const uint32_t c = base + (uint32_t)i * kPackedWaves;
            if (!GUARDED || c < chunks) {
                const uint32_t wd[4] = {b.w[i].x, b.w[i].y, b.w[i].z, b.w[i].w};
#pragma unroll
                for (uint32_t h = 0; h < kBlocks; ++h) {
                    float s = cs;
                    if constexpr (GROUPED) s = make_col_scale<BITS>(b.s[i][SCALES == kScalePerBlock ? h : 0u]);
                    uint4 w;
                    if constexpr (BITS == 8) {
                        const uint32_t lo = codes8_to_s8(wd[2 * h]), hi = codes8_to_s8(wd[2 * h + 1]);
                        w.x = pack_bf16_rne(sbyte_to_f32<0>(lo) * s, sbyte_to_f32<1>(lo) * s);
                        w.y = pack_bf16_rne(sbyte_to_f32<2>(lo) * s, sbyte_to_f32<3>(lo) * s);
                        w.z = pack_bf16_rne(sbyte_to_f32<0>(hi) * s, sbyte_to_f32<1>(hi) * s);
                        w.w = pack_bf16_rne(sbyte_to_f32<2>(hi) * s, sbyte_to_f32<3>(hi) * s);
                    } else {
                        // nibble r of the dword is row r: even rows from the low nibbles, odd rows from the high ones
                        uint32_t ev, od;
                        codes4_to_s8x16(wd[h], ev, od);
                        w.x = pack_bf16_rne(sbyte_to_f32<0>(ev) * s, sbyte_to_f32<0>(od) * s);
                        w.y = pack_bf16_rne(sbyte_to_f32<1>(ev) * s, sbyte_to_f32<1>(od) * s);
                        w.z = pack_bf16_rne(sbyte_to_f32<2>(ev) * s, sbyte_to_f32<2>(od) * s);
                        w.w = pack_bf16_rne(sbyte_to_f32<3>(ev) * s, sbyte_to_f32<3>(od) * s);
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, w),
                                                                          __builtin_bit_cast(bf16x8_t, b.a[i][h][mb]), acc[mb], 0, 0, 0);
                }
            }
        }
    };

    constexpr uint32_t kStride = kPackedWaves * kBatch;
    uint32_t base = wave;
    if constexpr (MODE == kPackedOneBatch) {
        // the launcher has checked that the slab is exactly one batch per wave: straight-line code, every load first
        Batch b;
        load(b, base);
        compute(b, base, std::false_type{});
    } else if constexpr (!PIPELINED) {
        for (; base + kStride - kPackedWaves < chunks; base += kStride) {  // batches whose every chunk exists
            Batch b;
            load(b, base);
            compute(b, base, std::false_type{});
        }
        if (base < chunks) {
            Batch b;
            load(b, base);
            compute(b, base, std::true_type{});
        }
    } else {
        // two batches in flight: the loads of the next batch are issued before the current one is converted
        auto compute_any = [&](const Batch& b, uint32_t at) {
            if (at + kStride - kPackedWaves < chunks) compute(b, at, std::false_type{});
            else compute(b, at, std::true_type{});
        };
        Batch b0, b1;
        if (base < chunks) load(b0, base);
        while (base < chunks) {
            if (base + kStride < chunks) load(b1, base + kStride);
            compute_any(b0, base);
            base += kStride;
            if (base >= chunks) break;
            if (base + kStride < chunks) load(b0, base + kStride);
            compute_any(b1, base);
            base += kStride;
        }
    }

    // acc[mb][r] of lane (nl, kg) is the sum for A row nl of block mb, W column 4 kg + r of the column block
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
        *reinterpret_cast<float4*>(&red[wave][mb][nl][4u * kg]) = make_float4(acc[mb][0], acc[mb][1], acc[mb][2], acc[mb][3]);
    __syncthreads();
    auto wave_sum = [&](uint32_t mb, uint32_t j, uint32_t i) {
        float sum = red[0][mb][j][i];
#pragma unroll
        for (int w = 1; w < kPackedWaves; ++w) sum += red[w][mb][j][i];
        const uint32_t c = 16u * nb + i;
        if (p.bias != nullptr) sum += bf16_bits_to_f32(p.bias[c]);
        return sum;
    };
    if (p.activation == kActSiluGate) {
        // columns (2 ip, 2 ip + 1) of the block are (gate, up) of output column 8 nb + ip
        for (uint32_t t = tid; t < 128u * MB; t += 64u * kPackedWaves) {
            const uint32_t mb = t >> 7, j = (t >> 3) & 15u, ip = t & 7u;
            const uint32_t row = 16u * (MB * rb + mb) + j;
            if (row < p.m) {
                float out = silu_gate(wave_sum(mb, j, 2u * ip), wave_sum(mb, j, 2u * ip + 1u));
                const uint32_t c = 8u * nb + ip;
                if (p.residual != nullptr) out += bf16_bits_to_f32(p.residual[(size_t)row * p.ldr + c]);
                p.c[(size_t)row * p.ldc + c] = (uint16_t)(pack_bf16_rne(out, 0.f) & 0xffffu);
            }
        }
        return;
    }
    for (uint32_t t = tid; t < 256u * MB; t += 64u * kPackedWaves) {
        const uint32_t mb = t >> 8, j = (t >> 4) & 15u, i = t & 15u;  // row block, A row, W column
        const uint32_t row = 16u * (MB * rb + mb) + j;
        if (row < p.m) {
            float sum = wave_sum(mb, j, i);
            const uint32_t c = 16u * nb + i;
            if (p.residual != nullptr) sum += bf16_bits_to_f32(p.residual[(size_t)row * p.ldr + c]);
            p.c[(size_t)row * p.ldc + c] = (uint16_t)(pack_bf16_rne(sum, 0.f) & 0xffffu);
        }
    }
}

// (no more than four waves per SIMD asked for: told that eight are possible, the compiler delays loads to save registers)
template <int BITS, int SCALES, int MB>
__global__ void __launch_bounds__(64 * kPackedWaves) __attribute__((amdgpu_waves_per_eu(2, 4)))
bfaintb_decode_packed_kernel(const GemmParams p)
{
    decode_packed_body<BITS, SCALES, MB, kPackedPlain>(p);
}

// (the 128-register form of the attribute: measured 6 % faster here than the looser one above, which wins for the loop)
template <int BITS, int SCALES, int MB>
__global__ void __launch_bounds__(64 * kPackedWaves) __attribute__((amdgpu_waves_per_eu(4)))
bfaintb_decode_packed_one_batch_kernel(const GemmParams p)
{
    decode_packed_body<BITS, SCALES, MB, kPackedOneBatch>(p);
}

// (at most 128 registers, so that two workgroups share a CU)
template <int BITS, int MB>
__global__ void __launch_bounds__(64 * kPackedWaves) __attribute__((amdgpu_waves_per_eu(4)))
bfaintb_decode_packed_pipelined_kernel(const GemmParams p)
{
    decode_packed_body<BITS, kScalePerChannel, MB, kPackedPipelined>(p);
}

template <int BITS, int SCALES>
static hipError_t launch_decode_packed_t(const GemmParams& p, hipStream_t stream)
{
    // two row blocks per workgroup once there are more than 16 rows: the weights are converted once for both
    const uint32_t mb = p.m > 16u ? 2u : 1u;
    const uint32_t chunks = p.k / PackedFormat<BITS>::kChunkRows;
    // the pipelined form when a wave has more than one plain batch of chunks and scales are per channel (measured: 9 %
    // faster at k = 11008 with per-channel scales, 10-25 % slower than the plain form with grouped ones)
    const bool pipelined = SCALES == kScalePerChannel && chunks > (uint32_t)(kPackedWaves * packed_batch(BITS, (int)mb, false));
    const bool one_batch = chunks == (uint32_t)(kPackedWaves * packed_batch(BITS, (int)mb, false));
    void (*kernel)(const GemmParams) =
        mb == 2u ? (pipelined   ? bfaintb_decode_packed_pipelined_kernel<BITS, 2>
                    : one_batch ? bfaintb_decode_packed_one_batch_kernel<BITS, SCALES, 2>
                                : bfaintb_decode_packed_kernel<BITS, SCALES, 2>)
                 : (pipelined   ? bfaintb_decode_packed_pipelined_kernel<BITS, 1>
                    : one_batch ? bfaintb_decode_packed_one_batch_kernel<BITS, SCALES, 1>
                                : bfaintb_decode_packed_kernel<BITS, SCALES, 1>);
    return launch_kernel(kernel, dim3(p.n / 16u, 1, (p.m + 16u * mb - 1u) / (16u * mb)), dim3(64 * kPackedWaves, 1, 1), 0, stream, p);
}

template <int BITS>
static hipError_t launch_decode_packed_b(const GemmParams& p, hipStream_t stream)
{
    if (p.group_size == 0) return launch_decode_packed_t<BITS, kScalePerChannel>(p, stream);
    if (p.group_size % PackedFormat<BITS>::kChunkRows == 0) return launch_decode_packed_t<BITS, kScalePerChunk>(p, stream);
    return launch_decode_packed_t<BITS, kScalePerBlock>(p, stream);
}

hipError_t launch_decode_packed(const GemmParams& p, int bits, hipStream_t stream)
{
    return bits == 8 ? launch_decode_packed_b<8>(p, stream) : launch_decode_packed_b<4>(p, stream);
}

}  // namespace bfaintb
