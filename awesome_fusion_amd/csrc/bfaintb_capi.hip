// C ABI of the library: argument validation, kernel-family choice, split-K sizing, launches.
// Stands where the reference driver packs its kernarg block and calls hipModuleLaunchKernel
// (/root/reference/bfAintBGemm/bfAintBGemm.cc:107-152); unlike GPU_CHECK_ERROR
// (gpu_utils.hpp:5-11, print and exit(0)) every failure is returned to the caller.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "bfaintb_device.hpp"
#include "../../include/bfaintb_gemm.h"

namespace bfaintb {
hipError_t launch_decode(const GemmParams& p, int bits, hipStream_t stream);
hipError_t launch_prefill(const GemmParams& p, int bits, hipStream_t stream, bool wreg);
hipError_t launch_dequant(uint16_t* w, const uint8_t* b, const uint16_t* scale, uint32_t n, uint32_t k, uint32_t ldb_bytes,
                          uint32_t ldw, int bits, uint32_t group_size, hipStream_t stream);
hipError_t launch_fill_u32(uint32_t* dst, uint32_t count, uint32_t value, hipStream_t stream);
hipError_t launch_probe_read(const void* src, size_t bytes, void* sink, hipStream_t stream);
hipError_t launch_pack_colmajor(uint8_t* dst, const uint8_t* src, uint32_t n, uint32_t k, uint32_t ldb_bytes, int bits, hipStream_t stream);
hipError_t launch_pack(uint8_t* dst, const uint8_t* src, uint32_t n, uint32_t k, uint32_t ldb_bytes, int bits, bool unpack,
                       hipStream_t stream);
hipError_t launch_decode_packed(const GemmParams& p, int bits, hipStream_t stream);
hipError_t launch_prefill_packed(const GemmParams& p, int bits, hipStream_t stream, bool wreg);
hipError_t launch_prefill128(const GemmParams& p, int bits, bool packed, hipStream_t stream);
hipError_t launch_prefill128_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream);
bool prefill128_wreg_serves(const GemmParams& p);
hipError_t launch_prefill256x128_wreg(const GemmParams& p, int bits, bool packed, hipStream_t stream);
hipError_t launch_decode_family_packed(const GemmParams& p, int bits, hipStream_t stream);
hipError_t decode_prepare_device();
}  // namespace bfaintb

// Split-K scratch of bfaintb_gemm_static: one array per GPU the library runs on, held until the process ends.  In host
// code this name is only a handle for hipGetSymbolAddress; device_state() resolves it once per device and everything
// else uses the resolved pointer.
#define BFAINTB_STATIC_SCRATCH_BYTES (16u << 20)
static __device__ __align__(256) unsigned char scratch[BFAINTB_STATIC_SCRATCH_BYTES];

namespace {

using bfaintb::GemmParams;
using bfaintb::kEmptyWord;

constexpr uint32_t kDecodeAutoMaxM = 32;       // AUTO always runs the decode family up to this m
constexpr uint32_t kDecodeFamilyAutoMaxM = 4096;  // ... and never beyond this one
constexpr uint32_t kDecodeMaxM = 32768;        // what the decode family accepts when forced
// Compute units the plans are made for: those of the device that is current when the first plan is made (256 where there
// is no device to ask: the part the estimates were fitted on), or what the tuning hook says.  One count per process:
// workspace sizes and launches must agree, whichever device a later call runs on (a plan for another count is still a
// correct launch, only not the fastest one).
std::atomic<uint32_t> g_plan_cus_override{0};
uint32_t machine_cus()
{
    static const uint32_t device_cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            return (uint32_t)n;
        (void)hipGetLastError();
        return 256u;
    }();
    const uint32_t forced = g_plan_cus_override.load(std::memory_order_relaxed);
    return forced ? forced : device_cus;
}
// workgroups the decode launches aim at: 8-wave workgroups run one per CU; 4-wave ones a little under two per CU
uint32_t decode_target_wgs_narrow() { return machine_cus(); }
uint32_t decode_target_wgs() { return machine_cus() * 15u / 8u; }
constexpr uint32_t kMaxSplits = 64;

int check_format(uint32_t k, int bits, uint32_t group_size)
{
    if (bits != 8 && bits != 4) return BFAINTB_ERR_UNSUPPORTED;
    if (group_size != 0 && (group_size % 32u != 0 || k % group_size != 0)) return BFAINTB_ERR_UNSUPPORTED;
    return BFAINTB_OK;
}

// Row-major weights: n a multiple of 8 (of 16 for 4-bit codes: a lane reads 16 of them per row), k a multiple of 8 (one
// 16-byte chunk of activations).  The kernels run a partial last step for the rest of k (the reference kernel needs
// n % 64 == 0 and k % 64 == 0: bf16gemm_kernel_gfx90a.s:341-343, :402-408).
int check_shape(uint32_t m, uint32_t n, uint32_t k, int bits = 8)
{
    if (k == 0 || n % (bits == 4 ? 16u : 8u) != 0 || k % 8u != 0) return BFAINTB_ERR_BAD_SHAPE;
    if (m >= (1u << 31) || n >= (1u << 31) || k >= (1u << 31)) return BFAINTB_ERR_BAD_SHAPE;
    return BFAINTB_OK;
}

// tuning hook (bfaintb_debug_control): the only row-block size, in units of 16 rows, decode_plan_row_blocks may pick; 0 = free
std::atomic<uint32_t> g_force_row_block{0};

// Launch shape of the decode variant: columns and waves per workgroup, blocks of 16 rows of A per workgroup,
// rows of k per workgroup, workgroups along k.
struct DecodePlan {
    uint32_t cols, waves, mb, k_per_wg, splits;
    uint32_t unit_bits = 0;  // width of the codes where it is not the `bits` the plan is made with (4-bit codes planned as 8-bit ones)
};

// Rows of k per workgroup and the number of splits that results, for `splits` wanted.
static void set_splits(DecodePlan& pl, uint32_t k, int bits, uint32_t splits, bool packed = false)
{
    // rows one workgroup covers per pipeline step of its waves
    const uint32_t unit = 32u * (uint32_t)bfaintb::decode_blocks_per_step(pl.unit_bits ? (int)pl.unit_bits : bits, (int)pl.cols / 16, packed, (int)pl.mb) * pl.waves;
    if (splits > kMaxSplits) splits = kMaxSplits;
    if (splits < 1) splits = 1;
    uint32_t per = (k + splits - 1) / splits;
    per = (per + unit - 1) / unit * unit;
    pl.k_per_wg = per;
    pl.splits = (k + per - 1) / per;
}

// Rough time, in microseconds, of the decode family for more than 32 rows of A (fitted on a 256-CU part).
// Every block of 16*mb rows streams and dequantises all weights again: measured 16, 22 and 35 cycles per
// weight and lane for mb = 1, 2, 4 (the dequantisation plus mb matrix instructions per 8 weights, less well
// overlapped the fewer waves a SIMD holds); repeats of the stream mostly hit in cache; split-K partial sums
// are written, read and cleared, and cost two more trips to memory; with fewer than one wave per SIMD both the
// arithmetic and the stream slow down in proportion.  Fitted to measurements at N = 4096, 11008 and 28672.
struct FamilyEstimate {
    double core, partial;  // the stream or the arithmetic, whichever is longer; the split's hand-over
    double serial;         // what the ranking adds for the reducing workgroup's own fetches (not part of the time estimates)
};
static double decode_family_estimate_us(uint32_t m, uint32_t n, uint32_t k, int bits, const DecodePlan& pl, FamilyEstimate* parts = nullptr)
{
    const double weights = (double)n * k;
    const double row_blocks = (double)((m + 16u * pl.mb - 1u) / (16u * pl.mb));
    const double col_blocks = (double)((n + pl.cols - 1u) / pl.cols);
    const double waves = row_blocks * col_blocks * pl.splits * pl.waves;
    const double cus = (double)machine_cus();
    const double busy = waves >= 4.0 * cus ? 1.0 : waves / (4.0 * cus);
    // 8-bit codes, refitted to a scan over row-block size x split factor at m = 40 .. 512 on 4096 x 4096, 11008 x 4096,
    // 4096 x 11008 and 2048 x 8192 (the choice of row block then lands within 0.5 % of the best on all 27 points; the
    // constants before it picked 16-row blocks where 32-row blocks with twice the splits run 6-24 % faster): larger row
    // blocks cost a little less per weight than first fitted, every further row block re-streams half of B from beyond
    // the caches, and the stream slows with idle CUs, not with idle wave slots.
    const double cycles_per_weight = bits == 8 ? 10.0 + 5.0 * pl.mb : 10.0 + 6.25 * pl.mb;
    // workgroups beyond one per CU share a CU's arithmetic: the last, partly filled round costs a whole one
    // (measured at n = k = 4096, 64-row blocks: m = 512 -> 256 workgroups, 35 us; m = 640 -> 320 workgroups, 61 us)
    const double wgs = row_blocks * col_blocks * pl.splits;
    const double ragged = wgs > cus ? (double)(uint64_t)((wgs + cus - 1.0) / cus) * cus / wgs : 1.0;
    const double compute = row_blocks * weights * cycles_per_weight / (256.0 * cus) / 2000.0 / busy * ragged;  // 4 SIMDs x 64 lanes per CU at 2 GHz
    const double stream_busy = bits == 8 ? (wgs >= cus ? 1.0 : wgs / cus) : busy;
    const double stream = weights * bits / 8.0 * (1.0 + (bits == 8 ? 0.5 : 0.3) * (row_blocks - 1.0)) / 3.5e6 / stream_busy;
    const double partial = pl.splits > 1 ? 3.0 + 12.0 * (pl.splits - 1.0) * m * n / 1.5e6 : 0.0;
    // (for the ranking only: the reducing workgroup fetches the other splits' sums of its block one after the other through
    // its one CU — the larger the block and the more the splits, the longer.  48 x 2560 x 16384: 64-row blocks with k split
    // 12 ways 27.0 us, 32-row blocks split 6 ways, the same number of workgroups, 20.6)
    const double serial = pl.splits > 1 ? 0.0075 * (pl.splits - 1.0) * pl.mb * pl.mb * pl.mb : 0.0;
    if (parts != nullptr) *parts = FamilyEstimate{compute > stream ? compute : stream, partial, serial};
    return 5.0 + (compute > stream ? compute : stream) + partial + serial;
}

// The same estimate, corrected to what the family's own plan takes in absolute terms: the estimate above ranks the
// family's plans among themselves (row-block size x split factor) and is left as fitted for that; against the tiles
// its absolute value decides, and there it is 1.3 - 1.75 times the measured time wherever k is split (the hand-over
// term is several times too large for row blocks of up to 32 rows, about 1.5 times for 64-row blocks) and within 8 %
// without a split.  Corrections fitted on 62 shapes (m = 48 .. 1024 over 4096 x 4096, 11008 x 4096, 4096 x 11008,
// 8192 x 8192, 2048 x 8192, 28672 x 8192, both code widths: the pick is then the faster form on 58 of them, within 10 %
// on the other four); 4-bit codes: 0.76 of the whole estimate, which dates from before their conversion got cheaper.
static double decode_family_time_us(uint32_t m, uint32_t n, uint32_t k, int bits, const DecodePlan& pl)
{
    FamilyEstimate e;
    const double ranked = decode_family_estimate_us(m, n, k, bits, pl, &e) - e.serial;
    if (bits == 4) {
        // (one row block that is not full costs less, a full one a little more than the 0.76 says: 64-row blocks of the
        // 128-column form at m = 40 / 48 / 64 against the tiles, us: 11008 x 8192 32.4 / 36.3, 33.6 / 36.5, 36.5 / 36.8;
        // 32000 x 4096 31.1 / 32.6, 32.1 / 32.6, 34.9 / 33.1; 16384 x 8192 34.4 / 36.8, 37.0 / 37.0, 40.6 / 38.8)
        const double block_rows = 16.0 * pl.mb;
        if (m <= block_rows && pl.cols == 128u) {
            // (and CUs left idle slow the stream less than in proportion, as over packed weights: 86 column blocks x 2 splits)
            const double wgs = (double)((n + pl.cols - 1u) / pl.cols) * pl.splits, cus = (double)machine_cus();
            // (not below 0.65 of a round: 144 and 160 column blocks, unsplit, take all the estimate says and more — 18432 x 6144,
            // m = 40 / 64: 44.6 / 52.8 us, where the tiles with k split three ways take 41.9 / 43.7; 20480 x 4096, m = 64: 39.0
            // against the tiles' 34.8)
            const double idle = wgs < cus && wgs * 20.0 >= cus * 13.0 ? pow(wgs / cus, 0.45) : 1.0;
            return 0.80 * (0.65 + 0.35 * m / block_rows) * (5.0 + e.core * idle + e.partial);
        }
        // (32-row blocks in more than a round and a half of workgroups take 0.82 - 0.86 of it: 48 / 64 x 128256 x 4096 161 / 163 us,
        // 48 / 64 x 50304 x 4096 79 / 81, where the tiles take 138 / 146 and 66 / 67)
        const double wgs = (double)((m + 16u * pl.mb - 1u) / (16u * pl.mb)) * (double)((n + pl.cols - 1u) / pl.cols) * pl.splits;
        if (pl.mb == 2u && wgs * 2.0 > 3.0 * (double)machine_cus()) return 0.84 * ranked;
        // (beyond 256 rows, unsplit: ten row blocks and more over few column blocks take all the estimate says and up to 1.4
        // times it — 320 x 2816 x 6144: 39.9 us, the tiles 29.0; 512 x 1280 x 5120: 35.9 / 26.7; 320 x 12032 x 6144: 101.7 / 93.6)
        // (... and their 8-wave workgroups count as a busy machine in the estimate from 128 of them on: CUs left without one
        // are charged here)
        if (m > 256u && pl.splits == 1u) {
            const double cus = (double)machine_cus();
            return 5.0 + e.core * (wgs < cus ? cus / wgs : 1.0);
        }
        return 0.76 * ranked;
    }
    // (64-row blocks: the hand-over at 0.9 of its term — at 0.65 the family ran up to 13 % over the tiles' time at 48 - 64 rows
    // against 8192 x 11008 and 8192 x 8192; 5 of 105 shapes scanned are then more than 2.5 % off, the worst 96 x 4096 x 11008
    // at 13 %.  Scaling a single block by its fill, which suits 4-bit codes, sends those same shapes back to the family.)
    if (pl.splits > 1u) return 0.87 * (5.0 + e.core + (pl.mb == 4u ? 0.9 : 0.2) * e.partial);
    return (pl.mb == 4u ? 1.05 : 0.93) * (5.0 + e.core);
}

// The tiled variant runs 128x128 tiles while those fit one per CU: four times the workgroups of
// 256x256 tiles, each with a quarter of the work per K-step.  Measured against the large tiles (8-bit, k = 4096, us):
// m x n = 256 x 4096: 48 / 59, 1024 x 4096: 58 / 66, 512 x 8192 (4-bit, k = 8192): 112 / 137; with more tiles the
// large ones win (1536 x 4096: 81 / 72, 512 x 11008: 80 / 68).
// (One gap: a few tall tiles more than CUs — 640 x 11008 makes 258 — would go to 129 large tiles on half the machine, 82 us;
// the small tiles take it in two rounds, 430 of them, in 66 us.  So: also up to two rounds of small tiles where the tall
// ones do not fit one round and the large ones fill at most 60 % of the CUs.)
static bool prefill_small_tiles(uint32_t m, uint32_t n, int bits)
{
    const uint64_t cus = machine_cus();
    const uint64_t small = (uint64_t)((m + 127u) / 128u) * ((n + 127u) / 128u);
    if (small <= cus) return true;
    // One row of tiles: 256-row tiles would spend half their matrix instructions or more on rows that do not exist, however
    // many rounds the small ones take (us, small / large, 8-bit and 4-bit codes: 64 x 128256 x 4096, 1002 small tiles, 152 / 187
    // and 148 / 203; 128 x 128256 x 4096 171 / 202 and 163 / 210; 96 x 50304 x 4096, 393 tiles, 71 / 86 and 69 / 101;
    // 128 x 36864 x 8192, 288 tiles, 134 / 157 and 135 / 135; from 129 rows on the large tiles win: 192 x 50304 x 4096 132 / 97)
    if (m <= 128u) return true;
    // 4-bit codes: two rounds of small tiles beat one of tall ones while the second round is about a third full (the tall
    // kernel converts every weight in two waves; us, small / tall, on two boxes: 1152 x 4096 x 4096, 288 tiles: 65.8 / 70.7
    // and 68.9 / 70.9; 512 x 11008 x 4096, 344: 65.9 / 71.1; with 384 to 448 tiles the second box had them level or the tall
    // ones ahead by 2 %, and packed weights by up to 4 %; 8-bit codes the other way throughout: 63.1 / 59.2 at 288 tiles)
    if (bits == 4 && small * 20u <= cus * 27u) return true;
    const uint64_t tall = (uint64_t)((m + 255u) / 256u) * ((n + 127u) / 128u);
    const uint64_t large = (uint64_t)((m + 255u) / 256u) * ((n + 255u) / 256u);
    // (0.6 of the CUs at most: 640 x 12032 x 3584, 141 large tiles, 76.2 us; 470 small ones 67.6)
    return small <= 2u * cus && tall > cus && large * 5u <= cus * 3u;
}

// Between the two: more small tiles than CUs, but at most one tile of 256 rows x 128 columns per CU.  The large tiles would
// occupy a quarter to a half of the CUs there; the tall ones run one per CU at 0.94 us per K-step against the large tiles'
// 1.02 on twice the work (8-bit, 64 steps, us tall / large: 1536 x 4096: 61.0 / 66.0; 512 x 11008: 60.3 / 64.7; 2048 x 4096:
// 71.0 / 75.7; 128 steps, 1024 x 8192: 129 / 141; 4-bit, 768 x 8192: 138 / 140).
static bool prefill_tall_tiles(uint32_t m, uint32_t n, int bits)
{
    return !prefill_small_tiles(m, n, bits) && (uint64_t)((m + 255u) / 256u) * ((n + 127u) / 128u) <= machine_cus();
}

static bool is_prefill(int v)
{
    return v == BFAINTB_VARIANT_PREFILL || v == BFAINTB_VARIANT_PREFILL_256 || v == BFAINTB_VARIANT_PREFILL_128 ||
           v == BFAINTB_VARIANT_PREFILL_256_LDS || v == BFAINTB_VARIANT_PREFILL_128_LDS || v == BFAINTB_VARIANT_PREFILL_256X128;
}

// tile size of a tiled-variant launch: forced, or by shape
static bool use_small_tiles(int v, uint32_t m, uint32_t n, int bits)
{
    return v == BFAINTB_VARIANT_PREFILL_128 || v == BFAINTB_VARIANT_PREFILL_128_LDS || (v == BFAINTB_VARIANT_PREFILL && prefill_small_tiles(m, n, bits));
}

// Rough time of the tiled variant (prefill_estimate_us, below the plan of the small tiles).  Small tiles: a K-step takes 0.40 us on an empty machine and 0.55 us with a workgroup on every CU (the kernel that
// keeps the weights in registers), whichever order the weights are stored in.
// The small-tile kernel may split k: grid y walks the splits, each workgroup runs its share of
// the K-steps and the workgroup of the last split adds the others' sums (same workspace and protocol as the decode
// family).  Worth it while tiles x splits still fit one workgroup per CU.
struct TilePlan {
    uint32_t k_per_wg, splits;
    double us;
};
constexpr uint32_t kMaxTileSplits = 16;

static size_t split_workspace_bytes(uint32_t splits, uint32_t m, uint32_t n)
{
    if (splits <= 1) return 0;
    // the header, then one fp32 word per (split but the last, row, column), rounded up to 256 bytes
    return bfaintb::kWorkspaceHeaderBytes + ((((size_t)(splits - 1u) * m * n * sizeof(float)) + 255u) & ~(size_t)255u);
}

static TilePlan tile128_plan(uint32_t m, uint32_t n, uint32_t k, int bits, uint32_t forced_splits)
{
    const uint32_t ksteps = (k + 63u) / 64u;
    const double tiles = (double)((m + 127u) / 128u) * (double)((n + 127u) / 128u);
    const double cus = (double)machine_cus();
    const double fill = (double)m / (double)((m + 127u) / 128u * 128u);  // the share of the tiles' rows that exist
    auto shape = [&](uint32_t want) {
        TilePlan t;
        if (want > kMaxTileSplits) want = kMaxTileSplits;
        if (want < 1u) want = 1u;
        const uint32_t per = (ksteps + want - 1u) / want;
        t.k_per_wg = per * 64u;
        t.splits = (ksteps + per - 1u) / per;
        // the hand-over: the producers' device-scope stores have to arrive, then the reducing workgroup fetches the rows
        // of a tile that exist, per split, through its one CU, slower the more CUs do so at once.  What the measured times
        // leave after the K-steps (8-bit, us): 48 / 64 / 96 / 128 x 4096 x 4096, 4 splits of 32 tiles: 7.0 / 8.0 / 9.7 / 11.4;
        // 384 x 2048 x 8192, 4 x 48: 9.6; 384 x 4096 x 4096, 2 x 96: 4.5; 256 x 8192 x 8192, 2 x 128: 5.9; 512 x 4096 x
        // 4096, 2 x 128: 7.6.
        const double hand_over = t.splits > 1u ? 3.0 + (t.splits - 1.0) * (0.6 + 1.6 * fill + 0.008 * tiles) : 0.0;
        // a K-step (two waves per column group): 0.40 us (4-bit codes 0.41) on a nearly empty machine, rising with the
        // cube of the share of the CUs that hold a workgroup as the clock gives way (8-bit, n = k = 4096, us per step at
        // 160 / 192 / 224 / 256 workgroups: 0.425 / 0.44 / 0.50 / 0.55; 4-bit g128: 0.49 at 224, 0.55 - 0.56 at 256);
        // rows of a tile that do not exist are not copied (28672 x 8192 4-bit, m = 64 / 96 / 128: 0.435 / 0.45 / 0.48)
        const double wgs = tiles * t.splits;
        auto step_us = [&](double load) { return ((bits == 4 ? 0.41 : 0.40) + 0.15 * load * load * load) * (0.8 + 0.2 * fill); };
        // (more small tiles than CUs: whole rounds of them and a last one at the pace of its own load — 96 x 36864 x 8192, 288
        // tiles: 128 us, 122 over packed weights; 640 x 11008 x 4096, 430: 66; 96 x 50304 x 4096, 393: 72; beyond two rounds the
        // steps take 10 - 18 % longer than this: 64 / 96 / 128 x 128256 x 4096, four rounds: 152 / 162 / 171 us with 8-bit
        // codes, 148 / 154 / 163 with 4-bit ones)
        const double whole = (double)(uint64_t)(wgs / cus), rest = wgs - whole * cus;
        const double steps_us = whole * step_us(1.0) + (rest > 0.0 ? step_us(rest / cus) : 0.0);
        t.us = 4.0 + (wgs > 2.0 * cus ? 1.12 : 1.0) * per * steps_us + hand_over;
        // (three splits and more: the hand-over scatters more than this says, and where the row-blocked family is about as
        // fast it is the safer pick — 192 x 4096 x 4096: 25.5 against 22.9 us, 128 x 4096 x 11008: 39.0 against 34.3)
        if (t.splits > 2u) t.us *= 1.07;
        return t;
    };
    if (forced_splits) return shape(forced_splits);
    TilePlan best = shape(1);
    static const uint32_t kCandidates[] = {2, 3, 4, 6, 8};
    for (uint32_t s : kCandidates) {
        if (tiles * s > cus) break;
        const TilePlan t = shape(s);
        if (t.splits != s) continue;  // k does not divide that way
        // (at most 256 tiles' worth of sums in all, 14 MiB: within the 32-bit offsets of the kernel and within the scratch of
        // the entry point that brings its own)
        if (t.us < best.us) best = t;
    }
    // One row of tiles that leaves a third or more of the CUs idle (half to five eighths of a round) and a long k: three
    // splits, as the decode family does on such widths — the estimate has the two forms level, the machine does not (us,
    // unsplit / three splits, 8-bit and 4-bit codes: 48 x 18432 x 8192, 144 tiles, 56.0 / 47.2 and 50.3 / 42.9; 96 x 18432 x
    // 8192 62.1 / 57.3 and 59.2 / 54.0; 48 x 20480 x 8192, 160 tiles, 60.3 / 51.1 and 50.6 / 43.1).  The launch rounds a split's
    // workgroups up to a multiple of 8, and three splits must stay clear of two rounds: 170 tiles make 528 and lose (57.9 /
    // 69.7).  A shorter k gains little or loses (k = 6144: 35.3 / 33.4 at 48 rows, 42.5 / 43.4 at 96; k = 4096: 25.1 / 27.2).
    // (While the partial sums stay within the 14 MiB of the note above.)
    const double per_split = (double)(uint64_t)((tiles + 7.0) / 8.0) * 8.0;
    if (best.splits == 1u && m <= 128u && tiles * 2.0 > cus && per_split * 3.0 * 16.0 <= cus * 31.0 && k >= 8192u &&
        2ull * m * n * sizeof(float) <= (14ull << 20)) {
        TilePlan t = shape(3);
        t.us *= 0.88;  // (measured against what shape() says of them: 0.85 - 0.92)
        if (t.splits == 3u) best = t;
    }
    return best;
}

static double prefill_estimate_us(uint32_t m, uint32_t n, uint32_t k, int bits)
{
    if (prefill_small_tiles(m, n, bits)) return tile128_plan(m, n, k, bits, 0).us;
    const double cus = (double)machine_cus();
    if (prefill_tall_tiles(m, n, bits)) {
        // one tile of 256 rows x 128 columns per CU at most (8-bit, us per K-step: 512 x 11008 x 4096, 172 tiles: 0.87;
        // 768 x 8192 x 8192 and 1536 x 4096 x 4096, 192: 0.84 and 0.88; 2048 x 4096 x 4096 and x 11008, 256: 1.02 and 0.98)
        const double tiles = (double)((m + 255u) / 256u) * (double)((n + 127u) / 128u);
        const double load = tiles / cus;
        return 4.0 + (k / 64.0) * (0.83 + 0.17 * load * load * load);
    }
    // whole rounds of 256x256 tiles at what the board's power allows (4096^3: 1.55 us per K-step and round)
    const double tiles = (double)((m + 255u) / 256u) * (double)((n + 255u) / 256u);
    const double rounds = (double)(uint64_t)((tiles + cus - 1.0) / cus);
    return 4.0 + rounds * (k / 64.0) * 1.5;
}

// The decode family in row blocks: grid z walks blocks of 16*mb rows.  128 columns x 64 rows (mb = 4, 4 waves: one
// wave per SIMD, 128 accumulator registers) amortises the dequantisation best; smaller row blocks give more
// workgroups when columns x row blocks alone do not fill the machine.  Picked by estimate.  (Columns per workgroup
// are fixed by the code width here: what the kernels over packed weights need.)  max_mb: the largest row block to
// consider, in units of 16 rows; wide8: blocks of 16 rows of 4-bit codes run 8 waves instead of 4.
DecodePlan decode_plan_row_blocks(uint32_t m, uint32_t n, uint32_t k, int bits, uint32_t forced_splits, bool packed = false,
                                  uint32_t max_mb = 4u, bool wide8 = false, bool nibbles = false)
{
    DecodePlan best{};
    double best_t = 0.0;
    const uint32_t only_mb = g_force_row_block.load(std::memory_order_relaxed);
    for (uint32_t mb = bits == 8 ? max_mb : (max_mb < 2u ? max_mb : 2u); mb >= 1u; mb >>= 1) {
        if (only_mb != 0u && mb != only_mb && only_mb <= (bits == 8 ? max_mb : 2u)) continue;
        DecodePlan c;
        c.unit_bits = nibbles ? 4u : 0u;
        c.cols = bits == 8 ? 128u : 256u;
        c.waves = ((bits == 8 && mb <= 2u) || (wide8 && mb == 1u)) ? 8u : 4u;  // wide8: 4-bit codes, 256 columns x 8 waves
        c.mb = mb;
        const uint32_t tiles = ((n + c.cols - 1u) / c.cols) * ((m + 16u * mb - 1u) / (16u * mb));
        // 8-bit codes: split along k until the workgroups fill one round of the 256 CUs, not beyond: measured at m = 40 and 64 over
        // n x k = 4096 x 4096, 8192 x 8192, 11008 x 4096 and 4096 x 11008, every row-block size ran fastest with the most
        // workgroups that still fit one round (4096 x 4096, m = 40, 32-row blocks: 19.3 / 14.4 / 11.2 / 15.7 us with
        // 64 / 128 / 256 / 512 workgroups; 11008 x 4096: 21.2 us with 172, 25.4 us with 344).
        if (bits == 8 && forced_splits == 0) {
            // (at most 16 splits, 8 while k is short: 512 x 4096, m = 48: 11.0 us with 16 splits, 7.0 with 8; 1024 x 8192, m = 32:
            // 9.1 with 16, 10.1 with 8)
            uint32_t s = machine_cus() / (tiles ? tiles : 1u);
            const uint32_t most = k >= 8192u ? 16u : k / 512u > 8u ? k / 512u : 8u;
            if (s > most) s = most;
            for (; s > 1u; --s) {
                set_splits(c, k, bits, s, packed);
                if (c.splits == s) break;  // k divides that way
            }
            set_splits(c, k, bits, s < 1u ? 1u : s, packed);
            const double t = decode_family_estimate_us(m, n, k, bits, c);
            if (best_t == 0.0 || t < best_t) { best_t = t; best = c; }
            continue;
        }
        // 4-bit codes (256 columns per workgroup, so fewer workgroups to begin with): the split factor the estimate likes
        // best; filling the round as above over-splits long k here (4096 x 11008, m = 32: 32.5 against 21.6 us)
        for (uint32_t s = 1; s <= 16u; s += (s < 4u ? 1u : s < 8u ? 2u : 4u)) {
            if (forced_splits && s != 1u) break;
            set_splits(c, k, bits, forced_splits ? forced_splits : s, packed);
            if (!forced_splits && c.splits != s && s != 1u) continue;  // k does not divide that way
            if (!forced_splits && s > 1u && tiles * s > 3u * machine_cus()) break;
            double t = decode_family_estimate_us(m, n, k, bits, c);
            // (packed codes: the kernels of 16-row blocks are the weaker ones there, and the estimate's price of a split sends
            // 17 to 32 rows against many columns to them — 32000 x 4096, m = 32: 47.8 us in two blocks of 16 rows, 32.0 in one of
            // 32 with k split in two; 28672 x 4096: 36.9 / 30.5; 13824 x 5120: 29.8 / 25.4.  With two thirds of that price the
            // pick is within 3 % of the better form on all 45 shapes scanned; for row-major codes the full price picks better.)
            if (packed) t -= 4.0 * (c.splits - 1.0) * m * n / 1.5e6;
            // (row-major codes: only the one block of 32 rows with k split in two is priced too high — 17 to 32 rows against
            // 224 to 250 blocks of columns went to two blocks of 16 rows without a split, a round of workgroups filled exactly:
            // 32000 x 4096, m = 32: 32.1 us against 28.1; 28672 x 4096: 31.2 / 29.1)
            else if (c.splits == 2u && mb == 2u) t -= 3.0 * m * n / 1.5e6;
            if (best_t == 0.0 || t < best_t) { best_t = t; best = c; }
        }
    }
    // 4-bit codes in rows, one block of 32 rows, one workgroup per column block and a third or more of the CUs idle: three splits,
    // as for 16 rows (decode_plan) — the estimate's price of a split keeps it from them while k is short (m = 24 / 32,
    // 36864 x 4096: 40.7 / 41.0 us unsplit, 36.6 / 37.6 split three ways; with k = 8192 the estimate picks the three itself)
    if (bits == 4 && !packed && forced_splits == 0 && m <= 32u && best.mb == 2u && best.splits == 1u && best.cols == 256u) {
        const uint32_t cus = machine_cus(), col_blocks = (n + 255u) / 256u;
        if (col_blocks * 2u > cus && col_blocks * 3u <= cus * 2u) {
            DecodePlan probe = best;
            set_splits(probe, k, bits, 3u, packed);
            if (probe.splits == 3u) best = probe;
        }
    }
    return best;
}

// nibbles: the plan is for 4-bit codes in the 128-column form, which takes the launch shapes of 8-bit codes (bits == 8 here)
DecodePlan decode_plan(uint32_t m, uint32_t n, uint32_t k, int bits, uint32_t forced_splits, bool packed = false, bool nibbles = false)
{
    // 4-bit codes in rows also have a 128-column form (a lane loads 4 bytes of a row, 16 lanes half a cache line — the
    // kernel gives the two halves of a line to workgroups that share an L2): twice the column blocks, so half the splits
    // for the same number of workgroups, and 8 waves from one row on.  It takes the launch shape 8-bit codes of the same
    // n x k would get.  Measured against the 256-column plan over 15 weight shapes x m = 1 .. 64 (us, 128 / 256 columns): up
    // to 24 MiB of codes every m gains (2048 x 8192: 7.8 / 9.6 at m = 1, 9.8 / 14.1 at 16, 12.4 / 17.7 at 64; 4096 x 4096:
    // 6.8 / 7.9, 8.0 / 10.7, 11.4 / 15.4; 6144 x 4096: 8.4 / 9.1, 10.0 / 11.3, 16.1 / 21.2; 4096 x 11008: 11.0 / 11.3, 13.4 /
    // 16.3, 21.4 / 26.3; 11008 x 4096: 11.3 / 11.2, 12.3 / 13.2, 14.6 / 18.9 at 24); up to 40 MiB from 16 rows on (8192 x
    // 8192, m = 16 / 24 / 32: 15.4 / 15.8, 17.4 / 21.3, 18.7 / 21.4; 5120 x 13824: 17.4 / 19.4, 19.6 / 24.3, 20.9 / 24.5; with
    // fewer rows the two are level); up to 64 MiB from 17 rows on, where the 256-column form needs row blocks of its own
    // (8192 x 11008, m = 20 / 24 / 32: 21.3 / 24.7, 22.1 / 25.9, 23.5 / 26.3; 11008 x 8192: 23.3 / 27.1, 24.2 / 27.6, 26.2 / 28.7;
    // 32000 x 4096: 22.8 / 26.0, 23.6 / 25.8, 25.3 / 26.7; 14336 x 8192 and 16384 x 8192: level; 12288 x 12288, 72 MiB: 38.0 /
    // 34.9, 42.8 / 37.3).  More weights stream better in whole lines per workgroup (14336 x 8192, m = 8 /
    // 16: 22.8 / 19.9, 25.1 / 21.2; 16384 x 8192, m = 1 .. 16: 12 - 15 % slower; 12288 x 12288, m = 8 .. 32: 10 - 44 %; 8192 x
    // 28672, m = 1 .. 32: 9 - 31 %; 28672 x 8192: 2 - 5 %).
    if (bits == 4 && !packed) {
        const uint64_t code_bytes = (uint64_t)n * k / 2u;
        if (code_bytes <= (24ull << 20) || (m >= 16u && code_bytes <= (40ull << 20)) || (m > 16u && code_bytes <= (64ull << 20)))
            return decode_plan(m, n, k, 8, forced_splits, false, true);
    }
    const uint64_t weight_bytes = (uint64_t)n * k * (uint32_t)bits / 8u;
    // 4-bit codes, 17 to 32 rows, a small or narrow matrix (row-major only: the kernels over packed 4-bit codes are built
    // for 4 waves): the two 16-row blocks run 8 waves each (m = 32, 1024 x 4096: 10.5 against 13.7 us, 17 rows: 10.6 / 17.2; 2048 x 8192:
    // 15.3 / 18.4; 4096 x 4096: 14.3 / 16.6; larger matrices lose: 4096 x 11008: 26.5 / 21.8)
    if (bits == 4 && m > 16 && m <= 32 && forced_splits == 0 && !packed && (weight_bytes <= (8ull << 20) || n <= 2048u))
        return decode_plan_row_blocks(m, n, k, bits, 0, false, 1u, true, nibbles);
    // 8-bit codes, more than 32 rows, but so few columns that even 16-row blocks make at most 40 workgroups per split: only
    // those (the 32- and 64-row kernels spend longer in their reductions than such a launch has; 768 x 5120, m = 48: 7.5
    // against 10.8 us; 1536 x 8960: 10.8 / 14.3; 256 x 7168, m = 128: 7.8 / 11.7; with more blocks the larger ones win:
    // 2048 x 8192, m = 128: 20.2 / 16.3)
    if (bits == 8 && m > 32 && forced_splits == 0 && (uint64_t)((n + 127u) / 128u) * ((m + 15u) / 16u) <= machine_cus() * 5u / 32u)
        return decode_plan_row_blocks(m, n, k, bits, 0, packed, 1u, false, nibbles);
    // More than 32 rows of A; 4-bit codes from 17 rows on: three blocks of 16 rows with their own workgroups beat one
    // 32-row block (n = k = 4096, m = 32: 15.8 against 21.4 us; 28672 x 8192, group 128: 46.5 against 53.0 us).
    if (m > 32 || (bits == 4 && m > 16)) return decode_plan_row_blocks(m, n, k, bits, forced_splits, packed, 4u, false, nibbles);
    DecodePlan pl;
    pl.unit_bits = nibbles ? 4u : 0u;
    // 8-bit codes, 17 to 32 rows, a small or narrow matrix: one 32-row block per workgroup cannot fill the machine without
    // splitting k further than it likes; two blocks of 16 rows with their own workgroups (the second stream hits in cache)
    // and the split that fills one round do (m = 32, n x k = 1024 x 4096: 7.0 against 8.9 us; 2048 x 8192: 10.9 against
    // 14.0; 1024 x 16384: 11.7 against 16.3; 4096 x 2048: 7.9 against 9.3; 4096 x 4096: 10.7 against 10.8; beyond 16 MiB
    // at more than 2048 columns the one block wins: 3072 x 8192: 15.4 against 14.4)
    if (bits == 8 && m > 16 && forced_splits == 0 && (weight_bytes <= (16ull << 20) || n <= 2048u))
        return decode_plan_row_blocks(m, n, k, bits, 0, packed, 1u, false, nibbles);
    {
        // 8-bit codes, 128 columns x 8 waves ("narrow": a lane loads 8 bytes of a row, 16 lanes one 128-byte line)
        // needs half the splits of 256 columns x 4 waves ("wide") for the same number of waves, so half the
        // partial-sum traffic.  Narrow workgroups run one per CU, so they pay for a ragged last round of 256.
        // Measured (n = 4096, 8192, 11008, 28672): narrow wins while the weights are few (latency-bound
        // launch), for m >= 8 (partial sums weigh most), and elsewhere when its best split factor fills whole
        // rounds; otherwise large matrices stream better in 256-byte row segments.  4-bit codes: wide.
        const bool few = weight_bytes <= (32ull << 20);
        // the split-K partial sums (written, read back and cleared as fp32) stay below a quarter of the weight bytes
        uint32_t cap = (uint32_t)(((uint64_t)k * (uint32_t)bits) / (256u * (m ? m : 1u)));
        if (cap < 1) cap = 1;
        // ... unless the weights are few: such launches are bound by latency, not by traffic, and want workgroups
        // (n = k = 4096, m = 32: 10.7 us with 8 splits against 12.6 us with 4; 16 splits are slower again)
        if (few && cap < 8u) cap = 8u;
        // narrow, large matrix: every further split costs traffic and a longer reduction; whole rounds count
        const uint32_t narrow_blocks = (n + 127u) / 128u;
        uint32_t narrow_splits = 1;
        double best = 0.0;
        const uint32_t cus = machine_cus();
        for (uint32_t s = 1; s <= cap && s <= 16u; ++s) {
            // (only the factors k divides into: another one would be rounded to its neighbour, whose workgroups may fill
            // the rounds far worse — 4-bit codes, 11008 x 8192: 5 splits, 430 workgroups, would have become 4 and 344:
            // 24.3 us at m = 16 against 22.0 with 2 splits)
            DecodePlan probe{};
            probe.unit_bits = nibbles ? 4u : 0u;
            probe.cols = 128u;
            probe.waves = 8u;
            probe.mb = m <= 16 ? 1u : 2u;
            set_splits(probe, k, bits, s, packed);
            if (probe.splits != s) continue;
            // Packed weights, and 4-bit codes in this form: one round of workgroups at most.  Measured over packed weights,
            // best factor within a round against the best beyond, us.  4-bit codes at m = 4 / 16 / 32: 12288 x 12288 2 splits
            // 26.3 / 28.3 / 33.8, 5 splits 28.8 / 30.6 / 36.2; 22016 x 4096 1 split 20.2 / 21.6 / 24.4, 4 splits 21.1 / 22.5 / 28.0;
            // 14336 x 8192 2 splits 21.1 / 23.7 / 27.1, 4 splits 23.6 / 25.9 / 30.9; only 16384 x 8192 likes two rounds (4 splits
            // 26.1 / 27.4 / 32.3 against 2 splits 29.2 / 29.9 / 32.4).  8-bit codes at m = 8 / 16 / 32: 11008 x 8192 2 splits
            // 20.0 / 21.0 / 24.3, 8 splits 24.5 / 25.3 / 29.9; 22016 x 4096 1 split 18.7 / 19.5 / 22.0, 4 splits 23.3 / 23.9 / 27.9;
            // 12288 x 12288 2 splits 30.5 / 32.7 / 36.3, 5 splits 30.6 / 31.6 / 36.1.  (8-bit codes in rows are within 7 % of
            // their best factor as the formula below picks it: 11008 x 8192, m = 8: 5 splits 22.5, 2 splits 21.0.)
            if ((nibbles || packed) && s > 1u && narrow_blocks * s > cus) break;
            const double rounds = (double)((narrow_blocks * s + cus - 1u) / cus);
            const double g = rounds / s + 0.04 * s * 4096.0 / k;  // time of the rounds + what a split costs, both relative to one pass over k
            if (best == 0.0 || g < best) { best = g; narrow_splits = s; }
        }
        const uint32_t narrow_wgs = narrow_blocks * narrow_splits;
        // (one round, at least 95 % full.  Several rounds of narrow workgroups lose to the wide form however well they fill them,
        // m = 1 / 8 / 16: 36864 x 4096, 6 splits x 288 blocks = 6.75 rounds, 39.8 / 43.3 / 47.9 us, its best factor, 2, 37.1 /
        // 39.4 / 42.7, wide 31.5 / 33.2 / 35.4; 24576 x 4096, 4 x 192 = 3 rounds, 23.6 / 25.7 / 28.2 against 20.5 / 21.8 / 23.5)
        const bool fills_rounds = narrow_wgs <= cus && narrow_wgs * 20u >= cus * 19u;
        // m >= 8 on a wide matrix: once 256-column blocks fill their one round with at most 3 splits (more than 64 of
        // them) their partial sums no longer outweigh the better stream (m = 8 / 16 / 32, wide against narrow:
        // 22016 x 4096 20.9 / 22.7 / 28.2 against 21.9 / 23.4 / 31.6 us; 28672 x 8192 46.2 / 48.3 / 54.2 against 49.8 / 53.1 /
        // 61.5; 18944 x 3584 16.9 / 18.3 / 24.0 against 18.0 / 19.9 / 25.1; with fewer blocks narrow stays ahead:
        // 11008 x 4096 13.9 / 14.9 / 17.9 against 13.8 / 16.5 / 22.1; 14336 x 4096 17.2 / 18.5 / 21.4 against 17.6 / 19.0 / 25.1)
        const bool many_wide_blocks = (n + 255u) / 256u > cus / 4u;
        // (n not a multiple of 16: only the 8-codes-per-lane shape can read the last columns)
        // (packed weights: the kernels are built for 128 columns; packed 4-bit codes: the 256-column form, 4 waves, is at
        // best 6 % ahead — 16384 x 8192 and 32000 x 4096 up to 16 rows — and up to 30 % behind)
        // (... and up to 96 MiB of weights: beyond, 256-column blocks win again unless the narrow ones fill their rounds — m = 8 /
        // 16, wide against narrow: 12288 x 12288 29.3 / 31.9 against 34.3 / 37.4 us; 14336 x 8192 24.8 / 26.9 against 26.2 / 28.3;
        // 32000 x 4096, 250 narrow blocks, stays narrow: 25.0 / 25.2 against 23.7 / 24.5)
        // (whole rounds decide up to 160 MiB: 8192 x 28672, 224 MiB, 4 splits x 64 blocks: narrow 41.5 - 47.9 us at m = 1 .. 16, wide
        // 39.7 - 45.5)
        const bool narrow = bits == 8 && (few || (fills_rounds && weight_bytes <= (160ull << 20)) || n % 16u != 0 ||
                                          (m >= 8 && (packed || (!many_wide_blocks && weight_bytes <= (96ull << 20)))) || (nibbles && packed));
        pl.cols = narrow ? 128u : 256u;
        // 4-bit codes, 8 to 16 rows: the same 256 columns with 8 waves (twice the waves to hide the activation loads and
        // the matrix instructions behind; n = k = 4096, m = 16: 11.6 against 14.7 us, 1024 x 8192: 14.1 / 17.4,
        // 8192 x 8192: 17.2 / 19.2, 28672 x 8192: 36.2 / 37.5; m = 8: 10.1 / 11.2, 10.2 / 12.7, 15.7 / 17.8, 35.1 / 35.3;
        // no difference at m = 1).  The kernels over packed 4-bit codes are built for 4 waves.
        const bool wide8 = bits == 4 && m >= 8u && !packed;
        pl.waves = (narrow || wide8) ? 8u : 4u;
        pl.mb = m <= 16 ? 1u : 2u;
        uint32_t splits = forced_splits;
        if (splits == 0) {
            if (narrow && !few) {
                splits = narrow_splits;
            } else {
                // about 256 workgroups of 8 waves or 480 of 4: enough waves on every CU to keep the memory system busy
                const uint32_t col_blocks = (n + pl.cols - 1) / pl.cols;
                // (8 waves: one workgroup per CU, so never a few workgroups past a whole round - 4-bit codes, m = 8,
                // 11008 x 4096: 13.4 us with 5 splits = 215 workgroups, 16.7 with 6 = 258; 22016 x 4096: 20.5 / 28.9)
                // 4-bit codes with 4 waves like one round as well while the column blocks are few (m = 1: 8192 x 8192
                // 14.1 us with 256 workgroups, 15.7 with 416; 5120 x 5120 9.7 / 11.7; 8192 x 4096 10.6 / 11.8; from 100
                // column blocks on the 480 are as good or a little better: 28672 x 8192 35.0 against 36.0)
                // 8-bit codes with 4 waves: one round on every shape measured (m = 1: 11008 x 4096 12.7 us with 215 workgroups,
                // 13.2 with 473; 9216 x 4096 11.7 / 13.1; 5120 x 8192 12.8 / 15.7; 18944 x 3584 15.8 / 17.4; 22016 x 4096
                // 19.6 / 21.8; 28672 x 8192 43.8 / 44.8; a few workgroups past the round are the worst case: 258 -> 15.3 us)
                const bool one_round = pl.waves == 8u || bits == 8 || (bits == 4 && col_blocks <= cus / 4u);
                splits = one_round ? decode_target_wgs_narrow() / col_blocks : (decode_target_wgs() + col_blocks / 2) / col_blocks;
                if (splits > cap) splits = cap;
                // One workgroup per column block that leaves a third or more of the CUs idle: three splits, one and a half to two rounds,
                // once k is long enough to pay for them (m = 8 / 16, 1 split against 3: 4-bit 38400 x 8192 50.4 / 50.8 against
                // 42.1 / 43.4 us, 34816 x 8192 51.2 / 53.9 against 43.4 / 46.3; 8-bit, m = 1 / 8 / 16, 36864 x 8192 59.2 / 62.5 / 66.4
                // against 52.8 / 56.6 / 59.9; no difference at k = 4096: 4-bit 38400 x 4096 27.7 / 28.1 against 27.3 / 28.8)
                // (up to two thirds of a round, so that the three splits stay within two rounds: 40960 x 8192, 160 blocks, m = 1 / 8 / 16:
                // 8-bit 61.4 / 64.9 / 68.6 against 55.3 / 59.1 / 62.7, 4-bit at m = 8 / 16 54.0 / 57.1 against 45.4 / 48.9; 170 blocks alike)
                if (one_round && splits == 1u && col_blocks * 3u <= cus * 2u && col_blocks * 2u > cus && k > 4096u && cap >= 3u) {
                    DecodePlan probe = pl;
                    set_splits(probe, k, bits, 3u, packed);
                    if (probe.splits == 3u) splits = 3u;
                }
                // More column blocks of 4-bit codes, 4 waves: rounds of one workgroup per CU count here as well, and a few
                // workgroups past a round cost 10 - 20 %.  The same cost as for the narrow form (rounds over the splits + what
                // a split costs) ranks the factors as measured (m = 1, k = 4096, us by splits: 22016 columns 5: 16.4, 6: 17.1,
                // 7: 17.7, 8: 15.6; 26624 4: 18.0, 5: 21.5, 6: 20.2, 7: 18.9; 33280 3: 21.7, 4: 24.0, 5: 22.7, 6: 23.4;
                // 45056 2: 29.0, 3: 30.7, 4: 25.4, 5: 28.6; 34816 x 8192 3: 37.9, 4: 41.5, 5: 37.1, 6: 40.3; m = 4 alike).
                if (!one_round) {
                    double least = 0.0;
                    for (uint32_t s = 1; s <= cap && s <= 16u; ++s) {
                        DecodePlan probe = pl;
                        set_splits(probe, k, bits, s, packed);
                        if (probe.splits != s) continue;
                        // (between one and a half and three rounds: two workgroups of 4 waves per CU are what keeps the
                        // memory system busy - 22016 x 4096 with 2 splits, 172 workgroups, one round: 18.3 us)
                        if (col_blocks * s * 2u < cus * 3u || col_blocks * s > cus * 3u) continue;
                        const double rounds = (double)((col_blocks * s + cus - 1u) / cus);
                        const double g = rounds / s + 0.04 * s * 4096.0 / k;
                        if (least == 0.0 || g < least) { least = g; splits = s; }
                    }
                }
                // More column blocks than two rounds, fewer than 8 rows: the same cost picks among 1 to 4 splits (m = 1, 151936 x
                // 4096, 594 blocks, us with 1 / 2 / 3 / 4 splits: 8-bit 102.7 / 96.1 / 95.7 / 98.2, 4-bit 85.6 / 80.0 / 80.7 / 83.0;
                // 128256 x 4096, 501 blocks, 1.96 rounds, stays whole: 78.4 / 80.5 and 56.9 / 58.7; from 8 rows on the partial
                // sums take the gain back: m = 8, 594 blocks: 103.2 / 101.4 / 104.4)
                if (col_blocks > 2u * cus && m < 8u) {
                    double least = 0.0;
                    for (uint32_t s = 1; s <= cap && s <= 4u; ++s) {
                        DecodePlan probe = pl;
                        set_splits(probe, k, bits, s, packed);
                        if (probe.splits != s) continue;
                        const double rounds = (double)((col_blocks * s + cus - 1u) / cus);
                        const double g = rounds / s + 0.04 * s * 4096.0 / k;
                        if (least == 0.0 || g < least) { least = g; splits = s; }
                    }
                }
                // a narrow matrix reaches that target only with very many splits, whose waves then run a single step each
                // and whose partial sums the reducing workgroup must collect: beyond 16 splits (32 once k is long enough
                // for four steps per wave) the launch gets slower again.  Measured at m = 1, 16 splits against what the
                // target asks for: 4-bit 1024 x 8192 9.6 / 14.5 us, 1024 x 4096 7.7 / 9.0, 4096 x 8192 10.9 / 12.8,
                // 4096 x 11008 12.7 / 13.9; 8-bit 1024 x 8192 7.9 / 9.3, 256 x 16384 8.6 / 13.6; 32 splits: 4-bit
                // 1024 x 16384 12.2 (16: 14.0, 64: 15.5), 1024 x 28672 15.5 (16: 19.5, 56: 16.8).
                const uint32_t most = k >= (bits == 4 ? 16384u : 24576u) ? 32u : 16u;
                if (splits > most) splits = most;
            }
        }
        set_splits(pl, k, bits, splits, packed);
    }
    return pl;
}

// The decode family up to 32 rows of A; beyond that whichever of the two the estimates favour (the prefill
// kernel's 256x256 tiles leave most of the machine idle until m*n reaches a few hundred tiles).
int resolve_variant(uint32_t m, uint32_t n, uint32_t k, int bits, int variant)
{
    if (variant == BFAINTB_VARIANT_AUTO) {
        if (m <= kDecodeAutoMaxM) return BFAINTB_VARIANT_DECODE;
        if (m > kDecodeFamilyAutoMaxM) return BFAINTB_VARIANT_PREFILL;
        const DecodePlan pl = decode_plan(m, n, k, bits, 0);
        return decode_family_time_us(m, n, k, bits, pl) < prefill_estimate_us(m, n, k, bits) ? BFAINTB_VARIANT_DECODE : BFAINTB_VARIANT_PREFILL;
    }
    if (variant == BFAINTB_VARIANT_DECODE) return m <= kDecodeMaxM ? variant : BFAINTB_ERR_BAD_VARIANT;
    if (is_prefill(variant)) return variant;
    return BFAINTB_ERR_BAD_VARIANT;
}

// whether a tiled-variant launch over row-major weights goes to the small-tile kernel that can split k
static bool tiled_may_split(int v, uint32_t m, uint32_t n, int bits) { return use_small_tiles(v, m, n, bits) && v != BFAINTB_VARIANT_PREFILL_128_LDS; }

size_t workspace_need(uint32_t m, uint32_t n, uint32_t k, int bits, int variant, uint32_t forced_split)
{
    if (m == 0 || n == 0) return 0;
    if (variant == BFAINTB_VARIANT_DECODE) return split_workspace_bytes(decode_plan(m, n, k, bits, forced_split).splits, m, n);
    if (is_prefill(variant) && tiled_may_split(variant, m, n, bits)) return split_workspace_bytes(tile128_plan(m, n, k, bits, forced_split).splits, m, n);
    return 0;
}

inline bool misaligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

// ---- per-device set-up: kernel attributes, and the address and first filling of the static scratch ----
constexpr int kMaxDevices = 64;
struct DeviceState {
    std::atomic<int> ready{0};      // kernel attributes set on this device
    std::atomic<int> scratch_ready{0};  // static scratch resolved and filled with the empty pattern
    void* scratch_ptr = nullptr;
};
DeviceState g_devices[kMaxDevices];
std::mutex g_setup_mutex;
std::atomic<uint32_t> g_split_wait_limit{bfaintb::kDefaultSplitWaitLimit};
std::atomic<uint32_t> g_debug_flags{0};

bool stream_is_capturing(hipStream_t stream)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return status != hipStreamCaptureStatusNone;
}

// The current device's state, its kernels prepared.  The set-up makes runtime calls that are not stream operations, so
// it must not run for the first time under stream capture: such a call is refused (BFAINTB_ERR_NOT_INITIALISED) and
// bfaintb_init is the way to run it beforehand.
int device_state(hipStream_t stream, DeviceState** out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return BFAINTB_ERR_UNSUPPORTED;
    DeviceState& st = g_devices[dev];
    if (!st.ready.load(std::memory_order_acquire)) {
        if (stream_is_capturing(stream)) return BFAINTB_ERR_NOT_INITIALISED;
        std::lock_guard<std::mutex> lock(g_setup_mutex);
        if (!st.ready.load(std::memory_order_relaxed)) {
            e = bfaintb::decode_prepare_device();
            if (e != hipSuccess) return (int)e;
            st.ready.store(1, std::memory_order_release);
        }
    }
    *out = &st;
    return BFAINTB_OK;
}

int init_workspace_on(void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    if (workspace_bytes % 4 != 0 || workspace_bytes / 4 >= (1ull << 32) || workspace_bytes < bfaintb::kWorkspaceHeaderBytes)
        return BFAINTB_ERR_WORKSPACE;
    // every word becomes "no partial sum here" (and "no failure" in the header), then the header gets its mark; fill
    // kernels rather than hipMemsetAsync, so that the call may be recorded into a HIP graph
    hipError_t e = bfaintb::launch_fill_u32(static_cast<uint32_t*>(workspace), (uint32_t)(workspace_bytes / 4), kEmptyWord, stream);
    if (e == hipSuccess) e = bfaintb::launch_fill_u32(static_cast<uint32_t*>(workspace) + 1, 1u, bfaintb::kWorkspaceMagic, stream);
    return (int)e;
}

// The device's static scratch, resolved and (the first time, outside any capture) filled with the empty pattern.
int static_scratch(DeviceState& st, hipStream_t stream, void** out)
{
    if (!st.scratch_ready.load(std::memory_order_acquire)) {
        if (stream_is_capturing(stream)) return BFAINTB_ERR_NOT_INITIALISED;
        std::lock_guard<std::mutex> lock(g_setup_mutex);
        if (!st.scratch_ready.load(std::memory_order_relaxed)) {
            void* ptr = nullptr;
            hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return (int)e;
            if (ptr == nullptr) return BFAINTB_ERR_WORKSPACE;
            const int rc = init_workspace_on(ptr, BFAINTB_STATIC_SCRATCH_BYTES, stream);
            if (rc) return rc;
            e = hipStreamSynchronize(stream);  // once per device: every stream may use the scratch from here on
            if (e != hipSuccess) return (int)e;
            st.scratch_ptr = ptr;
            st.scratch_ready.store(1, std::memory_order_release);
        }
    }
    *out = st.scratch_ptr;
    return BFAINTB_OK;
}

}  // namespace

extern "C" {

int bfaintb_version(void) { return BFAINTB_VERSION; }

const char* bfaintb_error_string(int code)
{
    switch (code) {
        case BFAINTB_OK: return "success";
        case BFAINTB_ERR_NULL_POINTER: return "null device pointer";
        case BFAINTB_ERR_BAD_SHAPE: return "unsupported shape: need n % 8 == 0 (4-bit codes: n % 16 == 0), k % 8 == 0, k > 0, sizes below 2^31; pre-packed weights: n % 16 == 0, k % 64 == 0 (4-bit: k % 128 == 0)";
        case BFAINTB_ERR_BAD_LD: return "bad leading dimension: need lda >= k, n <= ldb < 2^27, ldc >= n, lda % 8 == 0, ldb % 16 == 0, ldc % 8 == 0";
        case BFAINTB_ERR_ALIGNMENT: return "pointer not 16-byte aligned";
        case BFAINTB_ERR_UNSUPPORTED: return "unsupported format: weight_bits must be 8 or 4; group_size 0 or a multiple of 32 that divides k";
        case BFAINTB_ERR_WORKSPACE: return "workspace missing or smaller than bfaintb_gemm_workspace_bytes reports";
        case BFAINTB_ERR_BAD_VARIANT: return "unknown kernel variant, or variant cannot run this shape";
        case BFAINTB_ERR_NOT_INITIALISED: return "first call on this device made under stream capture: call bfaintb_init() beforehand";
        case BFAINTB_ERR_WORKSPACE_POISONED: return "a split-K wait gave up on this workspace (results of that call hold NaNs): initialise it again";
        case BFAINTB_ERR_STATIC_SCRATCH: return "shape needs more split-K scratch than bfaintb_gemm_static holds (16 MiB): use bfaintb_gemm with a workspace";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown bfaintb error code";
}

int bfaintb_gemm_variant(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size)
{
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    e = check_shape(m, n, k, weight_bits);
    if (e) return e;
    return resolve_variant(m, n, k, weight_bits, BFAINTB_VARIANT_AUTO);
}

uint32_t bfaintb_gemm_split_k(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size)
{
    const int v = bfaintb_gemm_variant(m, n, k, weight_bits, group_size);
    if (v == BFAINTB_VARIANT_DECODE) return decode_plan(m, n, k, weight_bits, 0).splits;
    if (v == BFAINTB_VARIANT_PREFILL && tiled_may_split(v, m, n, weight_bits)) return tile128_plan(m, n, k, weight_bits, 0).splits;
    return 1;
}

size_t bfaintb_gemm_workspace_bytes_ex(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size, int variant,
                                       uint32_t split_k)
{
    if (check_format(k, weight_bits, group_size) || check_shape(m, n, k, weight_bits)) return 0;
    const int v = resolve_variant(m, n, k, weight_bits, variant);
    if (v < 0) return 0;
    return workspace_need(m, n, k, weight_bits, v, split_k);
}

size_t bfaintb_gemm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size)
{
    return bfaintb_gemm_workspace_bytes_ex(m, n, k, weight_bits, group_size, BFAINTB_VARIANT_AUTO, 0);
}

int bfaintb_workspace_init(void* workspace, size_t workspace_bytes, void* stream)
{
    if (workspace == nullptr || workspace_bytes == 0) return BFAINTB_OK;
    if (misaligned16(workspace)) return BFAINTB_ERR_ALIGNMENT;
    return init_workspace_on(workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int bfaintb_workspace_status(const void* workspace, void* stream)
{
    if (workspace == nullptr) return BFAINTB_ERR_NULL_POINTER;
    uint32_t header[2] = {0, 0};
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemcpyAsync(header, workspace, sizeof(header), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return (int)e;
    if (header[1] != bfaintb::kWorkspaceMagic) return BFAINTB_ERR_WORKSPACE;
    return header[0] == kEmptyWord ? BFAINTB_OK : BFAINTB_ERR_WORKSPACE_POISONED;
}

// The same two calls for the scratch of bfaintb_gemm_static, whose address the library keeps to itself.
int bfaintb_static_scratch_status(void* stream)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    DeviceState* dev = nullptr;
    int rc = device_state(st, &dev);
    if (rc) return rc;
    void* ptr = nullptr;
    rc = static_scratch(*dev, st, &ptr);
    if (rc) return rc;
    return bfaintb_workspace_status(ptr, stream);
}

int bfaintb_static_scratch_reset(void* stream)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    DeviceState* dev = nullptr;
    int rc = device_state(st, &dev);
    if (rc) return rc;
    void* ptr = nullptr;
    rc = static_scratch(*dev, st, &ptr);  // (the first call on a device fills it anyway)
    if (rc) return rc;
    return init_workspace_on(ptr, BFAINTB_STATIC_SCRATCH_BYTES, st);
}

int bfaintb_init(void* stream)
{
    hipStream_t st = static_cast<hipStream_t>(stream);
    DeviceState* dev = nullptr;
    int rc = device_state(st, &dev);
    if (rc) return rc;
    (void)machine_cus();  // the device's compute units, asked for here rather than by a first plan made under capture
    void* ptr = nullptr;
    return static_scratch(*dev, st, &ptr);
}

// The two hooks that change what split-K launches do are for the library's own tests: they work only in a process that
// has BFAINTB_TEST_HOOKS=1 in its environment (read when the first of them is asked for), so that a stray call in a host
// application cannot turn every split-K result of the process into NaNs.
static bool test_hooks_armed()
{
    static const bool armed = [] {
        const char* v = getenv("BFAINTB_TEST_HOOKS");
        return v != nullptr && strcmp(v, "1") == 0;
    }();
    return armed;
}

int bfaintb_debug_control(uint32_t what, uint32_t value)
{
    if ((what == BFAINTB_DEBUG_SPLIT_WAIT_LIMIT || what == BFAINTB_DEBUG_WITHHOLD_PARTIALS) && !test_hooks_armed()) return BFAINTB_ERR_UNSUPPORTED;
    switch (what) {
        case BFAINTB_DEBUG_SPLIT_WAIT_LIMIT:
            g_split_wait_limit.store(value ? value : bfaintb::kDefaultSplitWaitLimit);
            return BFAINTB_OK;
        case BFAINTB_DEBUG_WITHHOLD_PARTIALS:
            if (value) g_debug_flags.fetch_or(bfaintb::kDebugWithholdPartials);
            else g_debug_flags.fetch_and(~bfaintb::kDebugWithholdPartials);
            return BFAINTB_OK;
        case BFAINTB_DEBUG_FORCE_ROW_BLOCK:
            if (value != 0u && value != 1u && value != 2u && value != 4u) return BFAINTB_ERR_UNSUPPORTED;
            g_force_row_block.store(value);
            return BFAINTB_OK;
        case BFAINTB_DEBUG_PLAN_COMPUTE_UNITS:
            if (value > 4096u) return BFAINTB_ERR_UNSUPPORTED;
            g_plan_cus_override.store(value);
            return BFAINTB_OK;
        default: return BFAINTB_ERR_UNSUPPORTED;
    }
}

// what the epilogue descriptor asks for, checked: bias and residual pointers (either may be null) and the residual's row stride
struct Epilogue {
    const void* bias = nullptr;
    const void* residual = nullptr;
    uint32_t ldr = 0;
    uint32_t activation = BFAINTB_ACT_NONE;
    // not an epilogue but set the same way: the reference kernel's arithmetic (fp32 scales, W and C narrowed by truncation)
    bool reference_arith = false;
    // columns of C (and of the residual) for n columns of B
    uint32_t out_cols(uint32_t n) const { return activation == BFAINTB_ACT_SILU_GATE ? n / 2u : n; }
};

static int read_epilogue(Epilogue& out, const bfaintb_epilogue* ep, uint32_t n)
{
    if (ep == nullptr) return BFAINTB_OK;
    if (ep->activation != BFAINTB_ACT_NONE && ep->activation != BFAINTB_ACT_SILU_GATE) return BFAINTB_ERR_UNSUPPORTED;
    out.bias = ep->bias;
    out.residual = ep->residual;
    out.ldr = ep->ldr;
    out.activation = ep->activation;
    if (ep->residual != nullptr && (ep->ldr < out.out_cols(n) || ep->ldr % 8u != 0)) return BFAINTB_ERR_BAD_LD;
    if (ep->activation == BFAINTB_ACT_SILU_GATE && n % 16u != 0) return BFAINTB_ERR_BAD_SHAPE;  // n / 2 output columns, stored 8 at a time
    return BFAINTB_OK;
}

// points the kernel at a split-K workspace: header first, partial sums behind it
static int attach_workspace(GemmParams& p, void* workspace, size_t workspace_bytes, size_t need)
{
    if (workspace == nullptr || workspace_bytes < need) return BFAINTB_ERR_WORKSPACE;
    if (misaligned16(workspace)) return BFAINTB_ERR_ALIGNMENT;
    if (need >= (1ull << 31)) return BFAINTB_ERR_BAD_VARIANT;  // the kernel addresses the workspace with 32-bit offsets
    p.ws_header = static_cast<uint32_t*>(workspace);
    p.partials = reinterpret_cast<unsigned long long*>(static_cast<uint8_t*>(workspace) + bfaintb::kWorkspaceHeaderBytes);
    p.partial_bytes = (uint32_t)(need - bfaintb::kWorkspaceHeaderBytes);
    p.split_wait_limit = g_split_wait_limit.load(std::memory_order_relaxed);
    p.debug_flags = g_debug_flags.load(std::memory_order_relaxed);
    return BFAINTB_OK;
}

static int gemm_impl(void* c, const void* a, const void* b, const void* scale, const Epilogue& ep, uint32_t m, uint32_t n, uint32_t k,
                     uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                     size_t workspace_bytes, void* stream, int variant, uint32_t split_k, bool use_static_scratch = false)
{
    const void* bias = ep.bias;
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    if (ep.reference_arith && (weight_bits != 8 || group_size != 0)) return BFAINTB_ERR_UNSUPPORTED;
    e = check_shape(m, n, k, weight_bits);
    if (e) return e;
    if (lda < k || ldb < n || ldc < ep.out_cols(n) || lda % 8u != 0 || ldb % 16u != 0 || ldc % 8u != 0) return BFAINTB_ERR_BAD_LD;
    if (ldb >= (1u << 27)) return BFAINTB_ERR_BAD_LD;  // a lane's offset within 32 rows of B is kept in 32 bits
    const int v = resolve_variant(m, n, k, weight_bits, variant);
    if (v < 0) return v;
    if (m == 0 || n == 0) return BFAINTB_OK;
    if (c == nullptr || a == nullptr || b == nullptr || scale == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (misaligned16(c) || misaligned16(a) || misaligned16(b) || misaligned16(scale) || misaligned16(bias) || misaligned16(ep.residual))
        return BFAINTB_ERR_ALIGNMENT;

    GemmParams p{};
    p.bias = static_cast<const uint16_t*>(bias);
    p.residual = static_cast<const uint16_t*>(ep.residual);
    p.ldr = ep.ldr;
    p.activation = ep.activation;
    p.reference_arith = ep.reference_arith ? 1u : 0u;
    p.c = static_cast<uint16_t*>(c);
    p.a = static_cast<const uint16_t*>(a);
    p.b = static_cast<const uint8_t*>(b);
    p.scale = static_cast<const uint16_t*>(scale);
    p.m = m; p.n = n; p.k = k;
    p.lda = lda;
    p.ldb_bytes = weight_bits == 8 ? ldb : ldb / 2u;
    p.ldc = ldc;
    p.lds = n;
    p.group_size = group_size;
    bfaintb::set_group_division(p);
    p.cus = machine_cus();
    p.k_per_wg = k;
    p.splits = 1;
    hipStream_t st = static_cast<hipStream_t>(stream);

    const bool tiled = is_prefill(v);
    bool small_wreg = false;  // the small-tile kernel that keeps row-major weights in registers (and may split k)
    if (tiled) {
        // the prefill kernel addresses B and a 256-row panel of A through 32-bit buffer extents
        if ((uint64_t)k * p.ldb_bytes >= (1ull << 31) || (uint64_t)256 * lda * 2u >= (1ull << 31)) return BFAINTB_ERR_BAD_SHAPE;
#ifdef BFAINTB_TRACE
        p.trace = static_cast<unsigned long long*>(workspace);  // per-quarter cycle totals, 8 words per wave
        return (int)bfaintb::launch_prefill(p, weight_bits, st, v != BFAINTB_VARIANT_PREFILL_256_LDS);
#endif
        // row-major weights on small tiles: that form, unless the other one is asked for by name
        small_wreg = tiled_may_split(v, m, n, weight_bits) && bfaintb::prefill128_wreg_serves(p);
        if (small_wreg) {
            const TilePlan tp = tile128_plan(m, n, k, weight_bits, split_k);
            p.k_per_wg = tp.k_per_wg;
            p.splits = tp.splits;
        }
    } else {
        const DecodePlan pl = decode_plan(m, n, k, weight_bits, split_k);
        p.k_per_wg = pl.k_per_wg;
        p.splits = pl.splits;
        p.decode_waves = pl.waves;
        p.decode_cols = pl.cols;
        p.decode_mb = pl.mb;
    }
    // (every argument check comes before the first runtime call)
    const size_t need = split_workspace_bytes(p.splits, m, n);
    if (p.splits > 1 && !use_static_scratch) {
        e = attach_workspace(p, workspace, workspace_bytes, need);
        if (e) return e;
    }
    if (use_static_scratch && need > BFAINTB_STATIC_SCRATCH_BYTES) return BFAINTB_ERR_STATIC_SCRATCH;
    DeviceState* dev = nullptr;
    if (!tiled || (p.splits > 1 && use_static_scratch)) {
        e = device_state(st, &dev);
        if (e) return e;
    }
    if (p.splits > 1 && use_static_scratch) {
        e = static_scratch(*dev, st, &workspace);
        if (e) return e;
        e = attach_workspace(p, workspace, BFAINTB_STATIC_SCRATCH_BYTES, need);
        if (e) return e;
    }
    if (tiled) {
        if (small_wreg) return (int)bfaintb::launch_prefill128_wreg(p, weight_bits, false, st);
        if ((v == BFAINTB_VARIANT_PREFILL_256X128 || (v == BFAINTB_VARIANT_PREFILL && prefill_tall_tiles(m, n, weight_bits))) && !p.reference_arith)
            return (int)bfaintb::launch_prefill256x128_wreg(p, weight_bits, false, st);
        if (use_small_tiles(v, m, n, weight_bits)) return (int)bfaintb::launch_prefill128(p, weight_bits, false, st);
        return (int)bfaintb::launch_prefill(p, weight_bits, st, v != BFAINTB_VARIANT_PREFILL_256_LDS);
    }
#ifdef BFAINTB_TRACE
    // timestamp sink: behind the split-K area (instrumented callers pass a larger workspace)
    p.trace = reinterpret_cast<unsigned long long*>(static_cast<uint8_t*>(workspace) + ((workspace_need(m, n, k, weight_bits, BFAINTB_VARIANT_DECODE, split_k) + 255) & ~(size_t)255));
#endif
    return (int)bfaintb::launch_decode(p, weight_bits, st);
}

// the packed order has K-chunks of 64 rows for 8-bit and 128 rows for 4-bit codes
static int check_packed_shape(uint32_t n, uint32_t k, int weight_bits)
{
    const int e = check_shape(1, n, k);
    if (e) return e;
    return (n % 16u != 0 || k % (weight_bits == 4 ? 128u : 64u) != 0) ? BFAINTB_ERR_BAD_SHAPE : BFAINTB_OK;
}

size_t bfaintb_prepack_bytes(uint32_t n, uint32_t k, int weight_bits)
{
    if ((weight_bits != 8 && weight_bits != 4) || check_packed_shape(n, k, weight_bits)) return 0;
    return (size_t)n * k * (uint32_t)weight_bits / 8u;
}

int bfaintb_packed_header_init(bfaintb_packed_header* h, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size, int has_bias)
{
    if (h == nullptr) return BFAINTB_ERR_NULL_POINTER;
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    e = check_packed_shape(n, k, weight_bits);
    if (e) return e;
    memset(h, 0, sizeof(*h));
    memcpy(h->magic, "BFAINTB1", 8);
    h->header_bytes = (uint32_t)sizeof(*h);
    h->layout = BFAINTB_LAYOUT_MFMA16;
    h->weight_bits = (uint32_t)weight_bits;
    h->group_size = group_size;
    h->k = k;
    h->n = n;
    h->payload_bytes = (uint64_t)n * k * (uint32_t)weight_bits / 8u;
    h->scale_bytes = (uint64_t)(group_size ? k / group_size : 1u) * n * 2u;
    h->has_bias = has_bias ? 1u : 0u;
    return BFAINTB_OK;
}

int bfaintb_packed_header_check(const bfaintb_packed_header* h)
{
    if (h == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (memcmp(h->magic, "BFAINTB1", 8) != 0 || h->header_bytes != sizeof(*h) || h->layout != BFAINTB_LAYOUT_MFMA16)
        return BFAINTB_ERR_UNSUPPORTED;
    bfaintb_packed_header want;
    const int e = bfaintb_packed_header_init(&want, h->n, h->k, (int)h->weight_bits, h->group_size, (int)h->has_bias);
    if (e) return e;
    if (h->has_bias > 1u || h->reserved[0] || h->reserved[1] || h->reserved[2]) return BFAINTB_ERR_UNSUPPORTED;
    if (h->payload_bytes != want.payload_bytes || h->scale_bytes != want.scale_bytes) return BFAINTB_ERR_BAD_SHAPE;
    return BFAINTB_OK;
}

static int repack(void* dst, const void* src, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream, bool unpack)
{
    if (weight_bits != 8 && weight_bits != 4) return BFAINTB_ERR_UNSUPPORTED;
    const int e = check_packed_shape(n, k, weight_bits);
    if (e) return e;
    if (ldb < n || ldb % 16u != 0) return BFAINTB_ERR_BAD_LD;
    if (n == 0) return BFAINTB_OK;
    if (dst == nullptr || src == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (misaligned16(dst) || misaligned16(src)) return BFAINTB_ERR_ALIGNMENT;
    return (int)bfaintb::launch_pack(static_cast<uint8_t*>(dst), static_cast<const uint8_t*>(src), n, k,
                                     weight_bits == 8 ? ldb : ldb / 2u, weight_bits, unpack, static_cast<hipStream_t>(stream));
}

int bfaintb_prepack(void* packed, const void* b, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream)
{
    return repack(packed, b, n, k, ldb, weight_bits, stream, false);
}

int bfaintb_unpack(void* b, const void* packed, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream)
{
    return repack(b, packed, n, k, ldb, weight_bits, stream, true);
}

int bfaintb_prepack_colmajor(void* packed, const void* b, uint32_t n, uint32_t k, uint32_t ldb, int weight_bits, void* stream)
{
    if (weight_bits != 8 && weight_bits != 4) return BFAINTB_ERR_UNSUPPORTED;
    const int e = check_packed_shape(n, k, weight_bits);
    if (e) return e;
    if (ldb < k || ldb % 16u != 0) return BFAINTB_ERR_BAD_LD;  // elements between columns
    if (n == 0) return BFAINTB_OK;
    if (packed == nullptr || b == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (misaligned16(packed) || misaligned16(b)) return BFAINTB_ERR_ALIGNMENT;
    return (int)bfaintb::launch_pack_colmajor(static_cast<uint8_t*>(packed), static_cast<const uint8_t*>(b), n, k,
                                              weight_bits == 8 ? ldb : ldb / 2u, weight_bits, static_cast<hipStream_t>(stream));
}

// Packed weights, "DECODE": the slab-streaming kernel (one workgroup per 16 columns over all of k, no split, every block
// of 16 rows of A converts the slab again) or the decode family reading packed slabs (128 or 256 columns per workgroup,
// split along k).  The slab kernel wins while the rows are few; how few depends on the shape, so packed_uses_slab
// compares what each was measured to take.
static DecodePlan packed_family_plan(uint32_t m, uint32_t n, uint32_t k, int bits);

// The slab kernel against the family, by what each was measured to take: 28 weight shapes from 256 x 7168 to 28672 x 8192,
// m = 1 .. 32, both code widths; least-squares fits, 7 - 9 % rms (us).
// The slab kernel: a workgroup walks its 16 columns alone, two workgroups that share a CU at half the pace each, so a
// launch takes as many walks as the fullest CU has slabs — n / 16 over 256 CUs, rounded up (4-bit codes, 5120 x 5120,
// 320 slabs: 7.3 us, what 8192 x 5120 would take; 4096 x 4096: 3.5).  4-bit codes are bound by the CUs' vector
// arithmetic (1975 rows per us and walk); 8-bit codes by that (1544 rows per us) or by memory (6.2 TB/s).  Each
// further row of A costs 1.4 - 3.6 % of the walk up to 6 rows and 6 - 8 % from there (two blocks of 16 rows from m = 17).
// The family's 128-column form streams at about 4.4 TB/s (4-bit) or 5.6 TB/s (8-bit) with every CU busy, pays the
// split's hand-over, and hardly grows with m up to 16 rows (11 - 26 % more from 17).
// Where the two are close either choice is within a few per cent; where they are not the gap is up to 80 % (4-bit codes,
// 5120 x 13824, m = 16: slab 31.0, family 17.2; 13824 x 5120: 26.0 / 15.5; 4096 x 2048, m = 32: 5.5 / 6.9; 1024 x 16384,
// m = 1: 10.5 / 9.0.  8-bit codes, m = 8: 5120 x 13824 23.2 / 16.3; 13824 x 5120 20.2 / 15.0; 5120 x 5120 11.3 / 9.2;
// 2048 x 4096, m = 12: 5.5 / 6.9).  Picks on the scan, weights cold: 4-bit 9 of 252 more than 5 % off the faster kernel
// (worst 12 %), 8-bit 12 of 252 (worst 14 %); fixed row limits, as before: 22 of 196, up to 42 %.
static double packed_slab_walks(uint32_t n)
{
    const double cus = (double)machine_cus();
    const double slabs = n / 16.0;
    return slabs <= 4.0 * cus ? (double)(uint64_t)((slabs + cus - 1.0) / cus) : slabs / cus;
}
static double packed_family_fill(uint32_t m, uint32_t n, const DecodePlan& pl)
{
    const double cus = (double)machine_cus();
    const double wgs = (double)((n + pl.cols - 1u) / pl.cols) * pl.splits * ((m + 16u * pl.mb - 1u) / (16u * pl.mb));
    const double rounds = (double)(uint64_t)((wgs + cus - 1.0) / cus);
    return wgs / (rounds * cus);
}
static double packed8_slab_time_us(uint32_t m, uint32_t n, uint32_t k)
{
    const double walks = packed_slab_walks(n);
    const double rows = m <= 6u ? 1.0 + 0.0136 * (m - 1.0) : m <= 16u ? 1.068 + 0.0578 * (m - 6.0) : 0.856 + 0.0608 * m;
    // (from the third walk on a walk never takes less than 2.2 us: its start and its reduction weigh as much as 1300 rows —
    // k = 2048, m = 8 / 12: 10496 columns 10.2 us, 16384 columns 15.3, where rows alone would say 7.2 and 10.6; one or two
    // walks of a short k hide them behind the launch: 4096 x 2048 stays at 3.7 us)
    const double per_walk = (k / 1544.0 > 2.2 || walks <= 2.0) ? k / 1544.0 : 2.2;
    const double walk_us = walks * per_walk, stream_us = (double)n * k / 6.16e6;
    return 2.07 + 0.017 * m * walks + (walk_us > stream_us ? walk_us : stream_us) * rows;
}
static double packed8_family_time_us(uint32_t m, uint32_t n, uint32_t k, const DecodePlan& pl)
{
    // (a long k streams faster, the workgroups' starts and hand-overs weighing less: 6 x 15104 x 11008 28.8 us, 6 x 7168 x 14336
    // 20.6, where 5.63 TB/s would say 34.1 and 23.3)
    const double long_k = k <= 4096u ? 0.0 : k >= 12288u ? 1.0 : (k - 4096.0) / 8192.0;
    const double stream_us = (double)n * k / 1.0e6 / (5.63 * (1.0 + 0.12 * long_k) * pow(packed_family_fill(m, n, pl), 0.638));
    return 3.0 + 0.0885 * m + 0.118 * (pl.splits - 1.0) + stream_us * (1.0 - 0.0037 * m + (m > 16u ? 0.1076 : 0.0)) * (pl.cols == 256u ? 1.1 : 1.0);
}
static double packed4_slab_time_us(uint32_t m, uint32_t n, uint32_t k)
{
    const double rows = m <= 6u ? 1.0 + 0.031 * (m - 1.0) : m <= 16u ? 1.155 + 0.078 * (m - 6.0) : 1.267 + 0.0776 * m;
    // (more than seven slabs per CU: 5 % less than that — 32000 / 50304 / 128256 / 151936 x 4096, m = 1: 17.6 / 26.2 / 63.4 / 74.8 us;
    // 28672 x 8192, seven, is as the formula says: 31.1)
    const double many = n / 16.0 > 7.0 * (double)machine_cus() ? 0.95 : 1.0;
    // (from the third walk on a walk never takes less than 1.45 us, as for 8-bit codes: k = 2048, 12 x 10240 9.6 us, 8 x 9984 8.3)
    const double walks = packed_slab_walks(n);
    const double per_walk = (k / 1975.0 > 1.45 || walks <= 2.0) ? k / 1975.0 : 1.45;
    return 2.58 + many * walks * per_walk * rows;
}
static double packed4_family_time_us(uint32_t m, uint32_t n, uint32_t k, const DecodePlan& pl)
{
    // (more than one round of workgroups: 8 % more than the fill says — 50304 / 128256 / 151936 x 4096, m = 1: 35.6 / 71.6 / 86.8 us,
    // m = 16: 37.4 / 75.4 / 91.5)
    const double wgs = (double)((n + pl.cols - 1u) / pl.cols) * pl.splits * ((m + 16u * pl.mb - 1u) / (16u * pl.mb));
    const double stream_us = (double)n * k / 2.0e6 / (4.37 * pow(packed_family_fill(m, n, pl), 0.58)) * (wgs > (double)machine_cus() ? 1.08 : 1.0);
    return 4.71 + 0.067 * m + 0.144 * (pl.splits - 1.0) + stream_us * (1.0 + 0.0003 * m + (m > 16u ? 0.258 : 0.0));
}
static bool packed_uses_slab(uint32_t m, uint32_t n, uint32_t k, int bits)
{
    if (m > kDecodeAutoMaxM) return false;
    const DecodePlan pl = packed_family_plan(m, n, k, bits);
    if (bits == 8) return packed8_slab_time_us(m, n, k) <= packed8_family_time_us(m, n, k, pl);
    if (pl.cols != 128u) return m <= 8u;
    return packed4_slab_time_us(m, n, k) <= packed4_family_time_us(m, n, k, pl);
}

// The family's plan over packed weights.  8-bit codes: the one row-major weights get, as long as it uses the 128 columns
// per workgroup the packed kernels are built for.  4-bit codes: the row-block plan also below 33 rows of A (measured
// against the small-m plan: 8192 x 8192, m = 32: 28.9 / 36.4 us; 28672 x 8192, m = 24: 56.9 / 65.6 us).
static DecodePlan packed_family_plan(uint32_t m, uint32_t n, uint32_t k, int bits)
{
    if (bits == 8) {
        const DecodePlan pl = decode_plan(m, n, k, bits, 0, true);
        if (pl.cols == 128u) return pl;
    }
    // 4-bit codes: the 128-column form (8 column blocks of 16 per workgroup, 8 waves) with the launch shape 8-bit codes
    // would get, wherever that shape has 128 columns.  Against the 256-column form, whose kernels over packed 4-bit codes
    // run 4 waves (us, 128 / 256 columns): 1024 x 8192, m = 64 / 128: 8.9 / 18.3, 11.4 / 17.5; 4096 x 4096: 10.6 / 15.7,
    // 14.9 / 20.7; 8192 x 8192, m = 16 / 32: 15.5 / 19.9, 18.3 / 24.1; 28672 x 8192, m = 12 / 32 / 48: 37.0 / 49.4, 42.3 / 47.1,
    // 52.0 / 70.6; 8192 x 28672: 37.0 / 41.4, 43.9 / 50.3, 52.8 / 68.5; 8192 x 11008, m = 16 / 64: 19.0 / 23.9, 30.5 / 36.2; the
    // other way round at most 6 % (16384 x 8192, m = 12: 29.5 / 27.8; 32000 x 4096: 27.6 / 26.3).
    if (bits == 4) {
        const DecodePlan pl = decode_plan(m, n, k, 8, 0, true, true);
        if (pl.cols == 128u) return pl;
    }
    return decode_plan_row_blocks(m, n, k, bits, 0, true);
}

// The family's estimate against the tiles', over packed weights, corrected as decode_family_time_us corrects it for
// row-major weights, with what a scan of 11 weight shapes x 12 values of m (40 .. 2048) x both code widths fits.  8-bit
// codes: the family's kernels over packed weights run at 0.72 (row blocks up to 32 rows) to 0.78 (64 rows) of the
// estimate's stream and arithmetic, and the hand-over costs 0.35 and 0.7 of its term; the factors in use (0.76, 0.84)
// sit a little above that, where the pick on the scan's shapes is best.  4-bit codes: the family measures 0.69 - 0.84 of
// the whole estimate (their packed kernels have no 8-wave form) and the tiles over packed 4-bit codes 0.82 - 0.98 of
// theirs; 0.84 against the tiles' estimate as it stands picks best (2 of 116 shapes more than 3 % off, worst 9 %;
// 8-bit: 3 of 128, worst 15 % at 40 x 11008 x 4096).  Up to 64 rows the family used to be the rule, as it once was
// for row-major weights: 4-bit codes against 11008 and 28672 columns then ran 22 - 39 % over the tiles' time.
static double packed_family_time_us(uint32_t m, uint32_t n, uint32_t k, int bits, const DecodePlan& pl)
{
    FamilyEstimate e;
    const double ranked = decode_family_estimate_us(m, n, k, bits, pl, &e) - e.serial;
    // Beyond 256 rows, unsplit, more than two rounds of workgroups (five row blocks and more against very many columns):
    // all the estimate says (us, family / tiles: 320 x 44032 x 2048 8-bit 132 / 87; 384 x 37120 x 2048 4-bit 132 / 76).  With
    // fewer workgroups than that the factors below stand: 640 x 1024 x 2048 12.3 / 16.3.
    if (m > 256u && pl.splits == 1u) {
        const double wgs_ = (double)((n + pl.cols - 1u) / pl.cols) * (double)((m + 16u * pl.mb - 1u) / (16u * pl.mb));
        if (wgs_ > 2.0 * (double)machine_cus()) return 5.0 + e.core;
    }
    if (bits == 4) return (pl.cols == 128u ? 0.70 : 0.84) * ranked;  // (the 128-column form measures 0.52 - 0.79 of its estimate)
    // (a row block that is not full costs less: 64-row blocks at m = 40 / 48 / 64 measure 0.87 / 0.91 / 1.0 of the tiles' time
    // over 11 weight shapes where the estimate had them level — the rows past m are neither converted for nor multiplied)
    const double block_rows = 16.0 * pl.mb;
    const double fill = m < block_rows ? m / block_rows : 1.0;  // (with more blocks than one the estimate is right as it stands: 96 x 8192 x 8192)
    // (and a round of workgroups that leaves CUs idle slows the stream less than in proportion: 172 and 192 workgroups of 64
    // rows x 128 columns run at 0.80 and 0.85 of the pace of 256, not 0.67 and 0.75 — 11008 x 8192, 22016 x 4096, 12288 x 12288)
    const double wgs = (double)((n + pl.cols - 1u) / pl.cols) * pl.splits * (double)(uint64_t)((m + block_rows - 1.0) / block_rows);
    const double cus = (double)machine_cus();
    const double idle = wgs < cus ? pow(wgs / cus, 0.45) : 1.0;
    // (a single block, since its kernels start each workgroup's walk over k at a step of its own: 0.92 of that — at 64 rows
    // the family leads the tiles by 5 - 8 % on 11008 x 8192, 28672 x 8192, 32000 x 4096, 14336 x 8192, 12288 x 12288)
    const double base = m <= block_rows ? 0.57 : 0.65;
    return (pl.mb == 4u ? 0.84 : 0.76) * (base + 0.35 * fill) * (5.0 + e.core * idle + (pl.mb == 4u ? 0.7 : 0.35) * e.partial);
}
// Which kernel multiplies by packed weights: the decode kernels (the slab-streaming one while packed_uses_slab, the
// row-blocked family without a split along k beyond) or the tiled kernel, by the estimates that choose for row-major weights.
static int packed_variant(uint32_t m, uint32_t n, uint32_t k, int bits, int variant)
{
    if (variant == BFAINTB_VARIANT_DECODE) return m <= kDecodeMaxM ? variant : BFAINTB_ERR_BAD_VARIANT;
    if (is_prefill(variant)) return variant;
    if (variant != BFAINTB_VARIANT_AUTO) return BFAINTB_ERR_BAD_VARIANT;
    if (packed_uses_slab(m, n, k, bits) || m <= kDecodeAutoMaxM) return BFAINTB_VARIANT_DECODE;
    if (m > kDecodeFamilyAutoMaxM) return BFAINTB_VARIANT_PREFILL;
    const DecodePlan pl = packed_family_plan(m, n, k, bits);
    return packed_family_time_us(m, n, k, bits, pl) < prefill_estimate_us(m, n, k, bits) ? BFAINTB_VARIANT_DECODE : BFAINTB_VARIANT_PREFILL;
}

int bfaintb_gemm_prepacked_variant(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size)
{
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    e = check_shape(m, n, k);
    if (e) return e;
    e = check_packed_shape(n, k, weight_bits);
    if (e) return e;
    return packed_variant(m, n, k, weight_bits, BFAINTB_VARIANT_AUTO);
}

// Scratch of the packed path: the decode family (where the slab kernel is not used) and the small tiles split along k.
static size_t packed_workspace_need(uint32_t m, uint32_t n, uint32_t k, int bits, int v)
{
    if (m == 0 || n == 0) return 0;
    if (is_prefill(v)) return tiled_may_split(v, m, n, bits) ? split_workspace_bytes(tile128_plan(m, n, k, bits, 0).splits, m, n) : 0;
    if (v != BFAINTB_VARIANT_DECODE || packed_uses_slab(m, n, k, bits)) return 0;
    const DecodePlan pl = packed_family_plan(m, n, k, bits);
    if (pl.splits <= 1) return 0;
    return bfaintb::kWorkspaceHeaderBytes + ((((size_t)(pl.splits - 1u) * m * n * sizeof(float)) + 255u) & ~(size_t)255u);
}

size_t bfaintb_gemm_prepacked_workspace_bytes_ex(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size, int variant)
{
    if (check_format(k, weight_bits, group_size) || check_shape(m, n, k) || check_packed_shape(n, k, weight_bits)) return 0;
    const int v = packed_variant(m, n, k, weight_bits, variant);
    return v < 0 ? 0 : packed_workspace_need(m, n, k, weight_bits, v);
}

size_t bfaintb_gemm_prepacked_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size)
{
    return bfaintb_gemm_prepacked_workspace_bytes_ex(m, n, k, weight_bits, group_size, BFAINTB_VARIANT_AUTO);
}

static int gemm_prepacked_impl(void* c, const void* a, const void* packed_b, const void* scale, const Epilogue& ep, uint32_t m,
                               uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc, int weight_bits, uint32_t group_size,
                               void* workspace, size_t workspace_bytes, void* stream, int variant)
{
    const void* bias = ep.bias;
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    e = check_shape(m, n, k);
    if (e) return e;
    e = check_packed_shape(n, k, weight_bits);
    if (e) return e;
    if (lda < k || ldc < ep.out_cols(n) || lda % 8u != 0 || ldc % 8u != 0) return BFAINTB_ERR_BAD_LD;
    const int v = packed_variant(m, n, k, weight_bits, variant);
    if (v < 0) return v;
    if (m == 0 || n == 0) return BFAINTB_OK;
    if (c == nullptr || a == nullptr || packed_b == nullptr || scale == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (misaligned16(c) || misaligned16(a) || misaligned16(packed_b) || misaligned16(scale) || misaligned16(bias) ||
        misaligned16(ep.residual))
        return BFAINTB_ERR_ALIGNMENT;
    GemmParams p{};
    p.residual = static_cast<const uint16_t*>(ep.residual);
    p.ldr = ep.ldr;
    p.activation = ep.activation;
    p.c = static_cast<uint16_t*>(c);
    p.a = static_cast<const uint16_t*>(a);
    p.b = static_cast<const uint8_t*>(packed_b);
    p.scale = static_cast<const uint16_t*>(scale);
    p.bias = static_cast<const uint16_t*>(bias);
    p.m = m; p.n = n; p.k = k;
    p.lda = lda;
    p.ldc = ldc;
    p.lds = n;
    p.group_size = group_size;
    bfaintb::set_group_division(p);
    p.cus = machine_cus();
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (is_prefill(v)) {
        // a tile's 16 column blocks and a 256-row panel of A are addressed through 32-bit buffer extents
        if ((uint64_t)k * 256u * (uint32_t)weight_bits / 8u >= (1ull << 31) || (uint64_t)256 * lda * 2u >= (1ull << 31))
            return BFAINTB_ERR_BAD_SHAPE;
        if (tiled_may_split(v, m, n, weight_bits) && bfaintb::prefill128_wreg_serves(p)) {
            // small tiles: the kernel that keeps the weights in registers, with the plan (split along k included) and the
            // workspace protocol of the row-major path
            const TilePlan tp = tile128_plan(m, n, k, weight_bits, 0);
            p.k_per_wg = tp.k_per_wg;
            p.splits = tp.splits;
            if (p.splits > 1) {
                e = attach_workspace(p, workspace, workspace_bytes, packed_workspace_need(m, n, k, weight_bits, v));
                if (e) return e;
            }
            return (int)bfaintb::launch_prefill128_wreg(p, weight_bits, true, st);
        }
        if (v == BFAINTB_VARIANT_PREFILL_256X128 || (v == BFAINTB_VARIANT_PREFILL && prefill_tall_tiles(m, n, weight_bits))) {
            p.k_per_wg = k;
            p.splits = 1;
            return (int)bfaintb::launch_prefill256x128_wreg(p, weight_bits, true, st);
        }
        if (use_small_tiles(v, m, n, weight_bits)) return (int)bfaintb::launch_prefill128(p, weight_bits, true, st);
        return (int)bfaintb::launch_prefill_packed(p, weight_bits, st, v != BFAINTB_VARIANT_PREFILL_256_LDS);
    }
    if (!packed_uses_slab(m, n, k, weight_bits)) {
        // beyond a few dozen rows the row-blocked decode family (A reused across 128 or 256 columns) reads the packed
        // slabs: measured at n = k = 4096 and m = 64, 128, 256: 16, 20, 22 us against 18, 34, 63 us for the slab kernel.
        // Same plan as for row-major weights, split along k and workspace protocol included.
        if (m > kDecodeMaxM) return BFAINTB_ERR_BAD_VARIANT;
        const DecodePlan pl = packed_family_plan(m, n, k, weight_bits);
        p.k_per_wg = pl.k_per_wg;
        p.splits = pl.splits;
        p.decode_waves = pl.waves;
        p.decode_cols = pl.cols;
        p.decode_mb = pl.mb;
        if (p.splits > 1) {
            e = attach_workspace(p, workspace, workspace_bytes, packed_workspace_need(m, n, k, weight_bits, v));
            if (e) return e;
        }
        DeviceState* dev = nullptr;
        e = device_state(st, &dev);
        if (e) return e;
        return (int)bfaintb::launch_decode_family_packed(p, weight_bits, st);
    }
    return (int)bfaintb::launch_decode_packed(p, weight_bits, st);
}

int bfaintb_gemm_prepacked_ex(void* c, const void* a, const void* packed_b, const void* scale, const void* bias, uint32_t m,
                              uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc, int weight_bits, uint32_t group_size,
                              void* workspace, size_t workspace_bytes, void* stream, int variant)
{
    Epilogue ep;
    ep.bias = bias;
    return gemm_prepacked_impl(c, a, packed_b, scale, ep, m, n, k, lda, ldc, weight_bits, group_size, workspace, workspace_bytes,
                               stream, variant);
}

int bfaintb_gemm_prepacked_fused(void* c, const void* a, const void* packed_b, const void* scale, const bfaintb_epilogue* epilogue,
                                 uint32_t m, uint32_t n, uint32_t k, uint32_t lda, uint32_t ldc, int weight_bits, uint32_t group_size,
                                 void* workspace, size_t workspace_bytes, void* stream)
{
    Epilogue ep;
    const int e = read_epilogue(ep, epilogue, n);
    if (e) return e;
    return gemm_prepacked_impl(c, a, packed_b, scale, ep, m, n, k, lda, ldc, weight_bits, group_size, workspace, workspace_bytes,
                               stream, BFAINTB_VARIANT_AUTO);
}

int bfaintb_gemm_prepacked(void* c, const void* a, const void* packed_b, const void* scale, const void* bias, uint32_t m, uint32_t n,
                           uint32_t k, uint32_t lda, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                           size_t workspace_bytes, void* stream)
{
    return bfaintb_gemm_prepacked_ex(c, a, packed_b, scale, bias, m, n, k, lda, ldc, weight_bits, group_size, workspace,
                                     workspace_bytes, stream, BFAINTB_VARIANT_AUTO);
}

int bfaintb_gemm_ex(void* c, const void* a, const void* b, const void* scale, uint32_t m, uint32_t n, uint32_t k,
                    uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                    size_t workspace_bytes, void* stream, int variant, uint32_t split_k)
{
    return gemm_impl(c, a, b, scale, Epilogue{}, m, n, k, lda, ldb, ldc, weight_bits, group_size, workspace, workspace_bytes, stream,
                     variant, split_k);
}

int bfaintb_gemm_bias(void* c, const void* a, const void* b, const void* scale, const void* bias, uint32_t m, uint32_t n,
                      uint32_t k, uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                      size_t workspace_bytes, void* stream)
{
    Epilogue ep;
    ep.bias = bias;
    return gemm_impl(c, a, b, scale, ep, m, n, k, lda, ldb, ldc, weight_bits, group_size, workspace, workspace_bytes, stream,
                     BFAINTB_VARIANT_AUTO, 0);
}

int bfaintb_gemm_fused(void* c, const void* a, const void* b, const void* scale, const bfaintb_epilogue* epilogue, uint32_t m,
                       uint32_t n, uint32_t k, uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size,
                       void* workspace, size_t workspace_bytes, void* stream)
{
    Epilogue ep;
    const int e = read_epilogue(ep, epilogue, n);
    if (e) return e;
    return gemm_impl(c, a, b, scale, ep, m, n, k, lda, ldb, ldc, weight_bits, group_size, workspace, workspace_bytes, stream,
                     BFAINTB_VARIANT_AUTO, 0);
}

int bfaintb_gemm_reference_ex(void* c, const void* a, const void* b, const float* scale, uint32_t m, uint32_t n, uint32_t k, uint32_t lda,
                              uint32_t ldb, uint32_t ldc, void* workspace, size_t workspace_bytes, void* stream, int variant, uint32_t split_k)
{
    Epilogue ep;
    ep.reference_arith = true;
    return gemm_impl(c, a, b, scale, ep, m, n, k, lda, ldb, ldc, 8, 0, workspace, workspace_bytes, stream, variant, split_k);
}

int bfaintb_gemm_reference(void* c, const void* a, const void* b, const float* scale, uint32_t m, uint32_t n, uint32_t k, uint32_t lda,
                           uint32_t ldb, uint32_t ldc, void* workspace, size_t workspace_bytes, void* stream)
{
    return bfaintb_gemm_reference_ex(c, a, b, scale, m, n, k, lda, ldb, ldc, workspace, workspace_bytes, stream, BFAINTB_VARIANT_AUTO, 0);
}

int bfaintb_gemm(void* c, const void* a, const void* b, const void* scale, uint32_t m, uint32_t n, uint32_t k,
                 uint32_t lda, uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* workspace,
                 size_t workspace_bytes, void* stream)
{
    return bfaintb_gemm_ex(c, a, b, scale, m, n, k, lda, ldb, ldc, weight_bits, group_size, workspace, workspace_bytes,
                           stream, BFAINTB_VARIANT_AUTO, 0);
}

int bfaintb_gemm_static(void* c, const void* a, const void* b, const void* scale, uint32_t m, uint32_t n, uint32_t k, uint32_t lda,
                        uint32_t ldb, uint32_t ldc, int weight_bits, uint32_t group_size, void* stream)
{
    return gemm_impl(c, a, b, scale, Epilogue{}, m, n, k, lda, ldb, ldc, weight_bits, group_size, nullptr, 0, stream, BFAINTB_VARIANT_AUTO,
                     0, true);
}

size_t bfaintb_gemm_static_scratch_bytes(void) { return BFAINTB_STATIC_SCRATCH_BYTES; }

int bfaintb_dequant(void* w, const void* b, const void* scale, uint32_t n, uint32_t k, uint32_t ldb, uint32_t ldw,
                    int weight_bits, uint32_t group_size, void* stream)
{
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    if (k == 0 || n % (weight_bits == 4 ? 16u : 8u) != 0 || k % 2u != 0) return BFAINTB_ERR_BAD_SHAPE;
    if (ldb < n || ldw < n || ldb % 16u != 0 || ldw % 8u != 0) return BFAINTB_ERR_BAD_LD;
    if (n == 0) return BFAINTB_OK;
    if (w == nullptr || b == nullptr || scale == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (misaligned16(w) || misaligned16(b) || misaligned16(scale)) return BFAINTB_ERR_ALIGNMENT;
    return (int)bfaintb::launch_dequant(static_cast<uint16_t*>(w), static_cast<const uint8_t*>(b),
                                        static_cast<const uint16_t*>(scale), n, k, weight_bits == 8 ? ldb : ldb / 2u, ldw,
                                        weight_bits, group_size, static_cast<hipStream_t>(stream));
}

int bfaintb_probe_read(const void* src, size_t bytes, void* sink, void* stream)
{
    if (bytes == 0) return BFAINTB_OK;
    if (src == nullptr) return BFAINTB_ERR_NULL_POINTER;
    if (misaligned16(src)) return BFAINTB_ERR_ALIGNMENT;
    if (bytes / 16 / 512 / 4 >= (1ull << 31)) return BFAINTB_ERR_BAD_SHAPE;
    return (int)bfaintb::launch_probe_read(src, bytes, sink, static_cast<hipStream_t>(stream));
}

// What a call would launch, without launching it: the queries above rolled into one description, for callers that want
// to log or check the library's choice and for the scans that hold the choice against measurements.
int bfaintb_gemm_plan(uint32_t m, uint32_t n, uint32_t k, int weight_bits, uint32_t group_size, int packed, int variant, uint32_t split_k,
                      bfaintb_plan* out)
{
    if (out == nullptr) return BFAINTB_ERR_NULL_POINTER;
    memset(out, 0, sizeof(*out));
    int e = check_format(k, weight_bits, group_size);
    if (e) return e;
    e = check_shape(m, n, k, packed ? 8 : weight_bits);
    if (e) return e;
    if (packed) {
        e = check_packed_shape(n, k, weight_bits);
        if (e) return e;
    }
    const int v = packed ? packed_variant(m, n, k, weight_bits, variant) : resolve_variant(m, n, k, weight_bits, variant);
    if (v < 0) return v;
    out->compute_units = machine_cus();
    out->launches = 1;
    out->splits = 1;
    out->k_per_workgroup = k;
    if (m == 0 || n == 0) return BFAINTB_OK;
    if (v == BFAINTB_VARIANT_DECODE) {
        out->variant = v;
        if (packed && packed_uses_slab(m, n, k, weight_bits)) {
            out->kernel = BFAINTB_KERNEL_DECODE_SLAB;
            out->tile_rows = m <= 16u ? 16u : 32u;
            out->tile_cols = 16u;
            out->waves = 8u;
            out->workgroups = n / 16u * ((m + out->tile_rows - 1u) / out->tile_rows);
            return BFAINTB_OK;
        }
        const DecodePlan pl = packed ? packed_family_plan(m, n, k, weight_bits) : decode_plan(m, n, k, weight_bits, split_k);
        out->kernel = BFAINTB_KERNEL_DECODE_FAMILY;
        out->tile_rows = 16u * pl.mb;
        out->tile_cols = pl.cols;
        out->waves = pl.waves;
        out->splits = pl.splits;
        out->k_per_workgroup = pl.k_per_wg;
        out->workgroups = ((n + pl.cols - 1u) / pl.cols) * pl.splits * ((m + 16u * pl.mb - 1u) / (16u * pl.mb));
        out->workspace_bytes = split_workspace_bytes(pl.splits, m, n);
        return BFAINTB_OK;
    }
    // the tiled kernels
    if (use_small_tiles(v, m, n, weight_bits)) {
        out->variant = BFAINTB_VARIANT_PREFILL_128;
        out->tile_rows = out->tile_cols = 128u;
        const bool wreg = v != BFAINTB_VARIANT_PREFILL_128_LDS;
        out->kernel = wreg ? BFAINTB_KERNEL_TILES_128 : BFAINTB_KERNEL_TILES_128_LDS;
        out->waves = wreg ? 4u : 8u;
        if (wreg) {
            const TilePlan tp = tile128_plan(m, n, k, weight_bits, packed ? 0u : split_k);
            out->splits = tp.splits;
            out->k_per_workgroup = tp.k_per_wg;
        }
        out->workgroups = ((m + 127u) / 128u) * ((n + 127u) / 128u) * out->splits;
        out->workspace_bytes = split_workspace_bytes(out->splits, m, n);
        return BFAINTB_OK;
    }
    if (v == BFAINTB_VARIANT_PREFILL_256X128 || (v == BFAINTB_VARIANT_PREFILL && prefill_tall_tiles(m, n, weight_bits))) {
        out->variant = BFAINTB_VARIANT_PREFILL_256X128;
        out->kernel = BFAINTB_KERNEL_TILES_256X128;
        out->tile_rows = 256u;
        out->tile_cols = 128u;
        out->waves = 4u;
        out->workgroups = ((m + 255u) / 256u) * ((n + 127u) / 128u);
        return BFAINTB_OK;
    }
    out->variant = v == BFAINTB_VARIANT_PREFILL_256_LDS ? v : BFAINTB_VARIANT_PREFILL_256;
    out->kernel = v == BFAINTB_VARIANT_PREFILL_256_LDS ? BFAINTB_KERNEL_TILES_256_LDS : BFAINTB_KERNEL_TILES_256;
    out->tile_rows = out->tile_cols = 256u;
    out->waves = v == BFAINTB_VARIANT_PREFILL_256_LDS ? 8u : 4u;
    {
        const uint32_t tiles = ((m + 255u) / 256u) * ((n + 255u) / 256u);
        const uint32_t halves = bfaintb::thin_round_tiles(tiles, m, machine_cus());
        out->workgroups = tiles - halves;
        out->tail_workgroups = 2u * halves;
        out->launches = (tiles - halves != 0u ? 1u : 0u) + (halves != 0u ? 1u : 0u);
    }
    return BFAINTB_OK;
}

uint32_t bfaintb_prefill_tile(uint32_t m, uint32_t n) { return prefill_small_tiles(m, n, 8) ? 128u : 256u; }
uint32_t bfaintb_prefill_tile_cols(uint32_t m, uint32_t n) { return (prefill_small_tiles(m, n, 8) || prefill_tall_tiles(m, n, 8)) ? 128u : 256u; }

const char* bfaintb_kernel_name(int variant, int weight_bits, uint32_t group_size, uint32_t m)
{
    int v = variant;
    if (v == BFAINTB_VARIANT_AUTO) v = m <= kDecodeAutoMaxM ? BFAINTB_VARIANT_DECODE : BFAINTB_VARIANT_PREFILL;
    if (v == BFAINTB_VARIANT_DECODE) return "bfaintb_decode_kernel";
    // (row-major weights, plain or bias epilogue; the forms with both operands in LDS serve the rest)
    if (v == BFAINTB_VARIANT_PREFILL || v == BFAINTB_VARIANT_PREFILL_256) return "bfaintb_prefill_wreg_kernel";
    if (v == BFAINTB_VARIANT_PREFILL_256_LDS) return "bfaintb_prefill_kernel";
    if (v == BFAINTB_VARIANT_PREFILL_128) return "bfaintb_prefill128_wreg_kernel";
    if (v == BFAINTB_VARIANT_PREFILL_128_LDS) return "bfaintb_prefill128_kernel";
    if (v == BFAINTB_VARIANT_PREFILL_256X128) return "bfaintb_prefill256x128_wreg_kernel";
    (void)weight_bits;
    (void)group_size;
    return "";
}

}  // extern "C"
