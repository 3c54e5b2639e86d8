// C ABI of the SpMM operator (include/hspmm.h): plan creation (validation,
// upload, work partition), launch, timing.  Host code only; the kernels live in
// hspmm_kernels.hip.  Mirrors the host half of the reference's fp16_spmm
// (reference src/fp16.cu:221-281) split into create / run / bench / destroy so
// that a caller can keep A on the device across launches.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstdarg>
#include <cstring>
#include <string>
#include <vector>
#include <mutex>
#include <atomic>
#include <chrono>
#include <new>
#include <algorithm>

#include "../../include/hspmm.h"
#include "hspmm_device.h"
#include "partition.hpp"
#include "host_parallel.hpp"
#include "step_stream.hpp"

// The fixed scratch array of hspmm_run_static (see static_scratch_address below): device memory the
// library holds on every device it is loaded on, for callers that must not allocate.
constexpr size_t kStaticScratchBytes = HSPMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char hspmm_static_scratch[kStaticScratchBytes];

namespace {

thread_local std::string g_last_error;

int fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

#define HSPMM_HIP(call)                                                                      \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess)                                                                \
            return fail(HSPMM_ERR_DEVICE, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                        __FILE__, __LINE__);                                                 \
    } while (0)

// the same where a failure has to release something first: cleanup(code) is called with the error code and its result returned
#define HSPMM_HIP_OR(call, cleanup)                                                          \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess)                                                                \
            return cleanup(fail(HSPMM_ERR_DEVICE, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                                __FILE__, __LINE__));                                        \
    } while (0)

// The knobs of the reference's Scheduler singleton (reference src/scheduler.h:7-10),
// re-read as: prefetch depth, waves per workgroup, waves per SIMD, compute units.
struct Config {
    int buffer_stage = 0;
    int consumer_warp_num = 0;
    int producer_warp_group_num = 0;
    int sm_num = 0;
    int kernel_mode = 0;
    int fused_fixup = -1;               // 1: the last wave of a cut unit adds its partial sums; 0: second kernel;
                                        // -1: the former in the LDS-panel kernels, and in the gather kernels where few units are cut
    int pairing = 0;                    // 0 automatic, 1 never, 2 whenever two windows share a column list
    int group_cuts = 0;                 // 1: plans of hspmm_create_grouped cut a window only where the caller's groups end
    // Tuning overrides from the environment (HSPMM_*), read once by hspmm_create: a plan's behaviour does
    // not change with the environment afterwards and the launch path reads no variable.
    int panel_chunks = 0;               // chunks of panels (0: searched per N)
    int panel_max_windows = 0;          // 2 or 4: windows per unit of the panel stream (0: by matrix size)
    int aligned_small = -1;             // small matrices: waves per unit of the one-workgroup-per-unit partition (-1: by size; 0, 4, 8)
    int gather_bitmap = -1;             // gather kernels read single 16-bit windows as bitmap + stored elements (-1: by fill)
    int xcd_split = -1;                 // gather kernels: two feature blocks dealt out by XCD half (-1: by matrix, 0 never, 1 always)
    // (set through hspmm_set_panel_stream; builds with HSPMM_EXPERIMENTAL only)
    int panel_tall = 0;                 // LDS-panel waves with two units each
    int panel_packed = 0;               // ... and their tiles stored without zeros
    int panel_units_per_group = 0;      // consumer waves of a workgroup that get a unit (0: searched per N)
    // (builds with HSPMM_EXPERIMENTAL only)
    int panel_units = 0;                // workgroup shape of the fp32-MFMA LDS-panel kernels: 12, 13, 14 (0: by tile type)

    void read_environment()
    {
        if (const char *e = std::getenv("HSPMM_FUSED_FIXUP")) fused_fixup = std::atoi(e) != 0;
        if (const char *e = std::getenv("HSPMM_PANEL_CHUNKS")) panel_chunks = std::max(1, std::atoi(e));
        if (const char *e = std::getenv("HSPMM_PANEL_MAX_WINDOWS")) panel_max_windows = std::atoi(e) >= 4 ? 4 : 2;
        if (const char *e = std::getenv("HSPMM_XCD_SPLIT")) xcd_split = std::atoi(e) != 0;
        if (const char *e = std::getenv("HSPMM_GATHER_BITMAP")) gather_bitmap = std::atoi(e) != 0;
        if (const char *e = std::getenv("HSPMM_ALIGNED_SMALL")) { const int v = std::atoi(e); aligned_small = v == 4 || v == 8 ? v : 0; }
        if (const char *e = std::getenv("HSPMM_PANEL_UNITS_PER_GROUP")) panel_units_per_group = std::max(1, std::atoi(e));
#ifdef HSPMM_EXPERIMENTAL
        if (const char *e = std::getenv("HSPMM_PANEL_UNITS")) panel_units = std::atoi(e) == 14 ? 14 : std::atoi(e) == 13 ? 13 : 12;
#endif
    }
};
// cost model of partition.hpp (a range costs its steps + 1.5 per unit; a cut within 35 % of a mean range of a unit
// boundary snaps onto it; units up to a mean range + 32 steps are never cut)
constexpr double kWindowCost = 1.5, kSlack = 0.35, kWholeWindowMargin = 32.0;
constexpr double kAlignedFourFrom = 2.5;   // ways the balanced partition must cut every unit before one workgroup walks it
constexpr double kPanelWideCost = 1.25;    // a step of three or four windows, in steps of two
std::mutex g_cfg_mutex;
Config g_cfg;

constexpr uint32_t kMinTilesPerRange = 24;

}  // namespace

namespace hspmm_host {
void set_error(const std::string &msg) { g_last_error = msg; }
}

struct hspmm_plan {
    int dtype = 0;
    int device = 0;
    uint32_t rows = 0, cols = 0, W = 0, T = 0;
    uint32_t cw = 16, elem = 2;
    int compute_units = 0;
    Config cfg;
    // device copies of the format arrays as given: scalar kernel
    uint32_t *d_rowOffset = nullptr, *d_rowIdx = nullptr;
    uint32_t *d_a2b_raw = nullptr;
    void *d_data = nullptr;
    // the step stream of the MFMA kernels
    int G = 1;                          // windows per unit: 2 when windows were paired
    uint32_t n_units = 0, n_paired = 0, n_steps = 0;
    uint32_t *d_unitOffset = nullptr, *d_unitRow = nullptr;
    uint32_t *d_ids = nullptr;          // per step, lane order, padding renamed to the id in front of it
    void *d_tiles = nullptr;            // per step, lane order (== d_data for fp16 without pairs)
    // partition
    // partitions of the step stream: [0] for one feature block per wave range (built by
    // hspmm_create), [1] / [2] with a half / a quarter of the ranges for feature dimensions
    // that need 2-3 / 4 or more blocks, built on first use (more blocks = more waves per range)
    struct DevPartition {
        bool built = false;
        hspmm::Partition part;
        uint32_t *d_ranges = nullptr, *d_split = nullptr, *d_fix_slots = nullptr;
    };
    DevPartition parts[5];              // [0..2]: fewer ranges per level; [3]: level 0 with sums added per workgroup;
                                        // [4]: every unit cut into the ranges of one workgroup (aligned)
    int aligned_group = 0;              // waves of the workgroup that walks one unit in [4]; 0: units too short for it
    std::vector<uint32_t> h_unitOffset;
    std::vector<uint32_t> h_unitRow;       // first row of every unit | its windows less one (for hspmm_partition_as_groups)
    std::vector<uint32_t> h_winOffset, h_winRow;   // plans whose units merge windows: the caller's rowOffset and rowIdx
                                                   // (hspmm_partition_as_groups writes groups of the caller's tiles)
    std::vector<uint32_t> caller_cuts;     // hspmm_create_grouped with hspmm_set_group_cuts(1): the ends of the caller's groups,
                                           // the only places where the gather kernels' partition cuts a window
    // LDS-panel kernels (matrices whose windows touch a large share of the columns):
    // the unit stream re-tiled panel by panel, built by hspmm_create when it pays
    struct Panel {
        bool built = false;
        uint32_t n_panels = 0, n_steps = 0;
        uint32_t *d_poff = nullptr, *d_ids = nullptr, *d_step_panel = nullptr;
        void *d_tiles = nullptr;
        uint32_t *d_unitRow = nullptr;                           // the units of this stream (first row | paired bit)
        uint32_t n_units = 0, n_paired = 0, n_wide = 0;          // units of two or more / three or four windows
        int G = 1;
        bool quad = false;                                       // ids in the format of the 4x4x1 fp32 tile
        bool split = false;                                      // fp32 stream in the bf16 hi / lo form (Fp32Split)
        bool tall = false;                                       // two units per consumer wave: poff per pair of units,
                                                                 // their steps merged panel by panel
        bool packed = false;                                     // tiles without their zeros: masks, values, step_voff
        double unit_lines = 0.0;                                 // 128-byte lines of tiles and ids per unit and panel (tall streams)
        uint64_t *d_masks = nullptr;
        void *d_vals = nullptr;
        uint32_t *d_step_voff = nullptr;
        double density = 0.0;                                    // steps per unit and 128 columns of the gather stream
    } panel;
    // Bitmap stream of the gather kernels (single 16-bit windows whose tiles are mostly zeros): per tile 8 words
    // of header (the reference's tcBit words of the tile, bit counts, position of the first stored element) and
    // the stored elements of all tiles in ascending bit order - nnzOffset / tcBit / data of the reference's BTCF_MTX
    struct Bitmap {
        bool built = false;
        uint32_t *d_header = nullptr;
        void *d_vals = nullptr;
        uint64_t stored = 0;
        bool from_caller = false;     // header and elements are the caller's tcBit / nnzOffset / data, uploaded as they came
    } bm;
    // What launches write besides C, one set per stream that has launched this plan (launches on different
    // streams may overlap in time): the first stream seen gets set 0, every other stream a set of its own at its
    // first launch - except a stream that is being captured (no allocation under capture) and streams beyond
    // kMaxStreamBuffers, which share set 0.
    struct StreamBuffers {
        hipStream_t stream = nullptr;
        bool unowned = false;               // made by hspmm_prepare before any launch: the first stream to launch takes it
        float *d_scratch = nullptr;         // partial sums of cut units
        size_t scratch_bytes = 0;
        uint32_t *d_arrive = nullptr;       // arrival counters of cut units, zero between launches
        size_t arrive_words = 0;
        uint32_t *d_vector = nullptr;       // a single 16-bit feature widened to words: cols words of B, then rows words
                                            // of C (made by the first launch with N = 1, or by hspmm_prepare(plan, 1))
    };
    static constexpr size_t kMaxStreamBuffers = 16;
    std::vector<StreamBuffers> buffers;
    size_t fixed_bytes = 0;
    // Every real column list strictly ascending and padding only behind a window's last column: what the
    // reference's converters write (reference src/utils/convert.h:166-181).  The gather and all-shapes
    // kernels take any list; merging windows and the LDS-panel stream need this order.
    bool canonical = true;
    // What a launch may still have to build (a partition for a wider N, larger scratch) is built under
    // this mutex; everything else in the plan is immutable after hspmm_create.
    std::mutex mu;
    // Superseded scratch buffers stay allocated until hspmm_destroy: launches recorded earlier (HIP
    // graphs) carry their addresses.
    std::vector<void *> retired;
    size_t retired_bytes = 0;               // partial-sum buffers among them (counters are part of fixed_bytes)
    std::atomic<uint32_t> last_family{0};   // kernel family of the last hspmm_run: 0 none yet, 1 all-shapes, 2 gather, 3 LDS-panel, 4 clear
    // matrix instructions of the last launch's main kernel: kind (hspmm_plan_info::last_mfma_kind) and count
    std::atomic<uint32_t> last_mfma_kind{0};
    std::atomic<uint64_t> last_mfma_count{0};
    void note_launch(uint32_t family, uint32_t kind, uint64_t count)
    {
        last_family.store(family, std::memory_order_relaxed);
        last_mfma_kind.store(kind, std::memory_order_relaxed);
        last_mfma_count.store(count, std::memory_order_relaxed);
    }
};

namespace {

using namespace hspmm_host;   // the stream builders of step_stream.hpp

// HSPMM_TIMING=1 in the environment: hspmm_create prints what each of its phases took (stderr).
struct PhaseTimer {
    bool on = std::getenv("HSPMM_TIMING") != nullptr;
    std::chrono::steady_clock::time_point last = std::chrono::steady_clock::now();
    void mark(const char *what)
    {
        if (!on) return;
        const auto now = std::chrono::steady_clock::now();
        std::fprintf(stderr, "hspmm_create: %-28s %8.2f ms\n", what, std::chrono::duration<double, std::milli>(now - last).count());
        last = now;
    }
};

template <typename T>
int upload(T **dst, const T *src, size_t n, size_t *acc_bytes)
{
    const size_t bytes = (n ? n : 1) * sizeof(T);
    HSPMM_HIP(hipMalloc(reinterpret_cast<void **>(dst), bytes));
    if (n) HSPMM_HIP(hipMemcpy(*dst, src, n * sizeof(T), hipMemcpyHostToDevice));
    *acc_bytes += bytes;
    return HSPMM_OK;
}

// canonical (optional): whether every window's real column ids ascend strictly with padding only behind
// the window's last column, as the reference's converter writes them (src/utils/convert.h:166-181).
int validate_format(uint32_t rows, uint32_t cols, uint32_t W, uint32_t T, uint32_t cw,
                    const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data, const uint32_t *rowIdx,
                    bool *canonical = nullptr)
{
    if (canonical) *canonical = true;
    if (W == 0) {
        if (T != 0) return fail(HSPMM_ERR_INVALID, "total_tiles = %u with no effective row window", T);
        return HSPMM_OK;
    }
    if (!rowOffset || !tcA2B || !data || !rowIdx) return fail(HSPMM_ERR_INVALID, "null format array");
    if (rows == 0 || cols == 0) return fail(HSPMM_ERR_INVALID, "empty matrix with %u effective windows", W);
    if (uint64_t(W) > (uint64_t(rows) + 7u) / 8u)
        return fail(HSPMM_ERR_INVALID, "eff_row_windows = %u exceeds the %u windows of %u rows", W, (rows + 7u) / 8u, rows);
    if (rowOffset[0] != 0) return fail(HSPMM_ERR_INVALID, "rowOffset[0] = %u, expected 0", rowOffset[0]);
    for (uint32_t w = 0; w < W; ++w) {
        if (rowOffset[w + 1] <= rowOffset[w])
            return fail(HSPMM_ERR_INVALID, "rowOffset not strictly increasing at window %u", w);
        if (rowIdx[w] % HSPMM_ROW_WINDOW != 0 || rowIdx[w] >= rows)
            return fail(HSPMM_ERR_INVALID, "rowIdx[%u] = %u is not a window start inside %u rows", w, rowIdx[w], rows);
        if (w && rowIdx[w] <= rowIdx[w - 1])
            return fail(HSPMM_ERR_INVALID, "rowIdx not strictly increasing at window %u", w);
    }
    if (rowOffset[W] != T)
        return fail(HSPMM_ERR_INVALID, "rowOffset[%u] = %u differs from total_tiles = %u", W, rowOffset[W], T);
    for (uint32_t t = 0; t < T; ++t) {
        const uint32_t *ids = tcA2B + size_t(t) * cw;
        if (ids[0] == HSPMM_IDX_MAX) return fail(HSPMM_ERR_INVALID, "tile %u starts with a padding column", t);
        bool pad = false;
        for (uint32_t k = 0; k < cw; ++k) {
            if (ids[k] == HSPMM_IDX_MAX) { pad = true; continue; }
            if (pad) return fail(HSPMM_ERR_INVALID, "tile %u: column id after padding", t);
            if (ids[k] >= cols) return fail(HSPMM_ERR_INVALID, "tile %u: column id %u >= cols %u", t, ids[k], cols);
        }
    }
    if (canonical) {
        std::atomic<bool> ok{true};
        hspmm_host::parallel_blocks(W, 4096, [&](size_t wb, size_t we) {
            for (size_t w = wb; w < we && ok.load(std::memory_order_relaxed); ++w) {
                const uint32_t *c = tcA2B + size_t(rowOffset[w]) * cw;
                const size_t n = size_t(rowOffset[w + 1] - rowOffset[w]) * cw;
                size_t real = n;
                while (real && c[real - 1] == HSPMM_IDX_MAX) --real;
                bool good = n - real < cw;                      // padding only in the window's last tile
                for (size_t i = 1; i < real && good; ++i) good = c[i] != HSPMM_IDX_MAX && c[i] > c[i - 1];
                if (!good) ok.store(false, std::memory_order_relaxed);
            }
        });
        *canonical = ok.load();
    }
    return HSPMM_OK;
}

int choose_ranges(const hspmm_plan *p)
{
    const int waves_per_simd = p->cfg.producer_warp_group_num > 0 ? p->cfg.producer_warp_group_num : 4;
    uint64_t g = uint64_t(p->compute_units) * 4u * uint64_t(waves_per_simd);
    const uint64_t cap = (uint64_t(p->n_steps) + kMinTilesPerRange - 1) / kMinTilesPerRange;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return int(g);
}

int build_and_upload_partition(hspmm_plan *p, int level, uint32_t group = 1, bool aligned = false)
{
    hspmm_plan::DevPartition &dp = p->parts[aligned ? 4 : group > 1 ? 3 : level];
    if (dp.built || p->W == 0) return HSPMM_OK;
    const double window_cost = kWindowCost, slack = kSlack, margin = kWholeWindowMargin;
    uint32_t target = uint32_t(choose_ranges(p)) >> level;
    const uint32_t floor_ranges = uint32_t(p->compute_units) * 4u;       // at least one range per SIMD
    if (target < floor_ranges) target = std::min<uint32_t>(floor_ranges, uint32_t(choose_ranges(p)));
    dp.part = aligned ? hspmm::build_aligned_partition(p->n_units, p->h_unitOffset.data(), group)
                      : hspmm::build_partition(p->n_units, p->h_unitOffset.data(), target, window_cost, slack, margin, group,
                                               p->caller_cuts.empty() ? nullptr : &p->caller_cuts);
    const auto &part = dp.part;
    std::vector<uint32_t> rw(part.ranges.size() * hspmm::kRangeWords, 0u);
    for (size_t i = 0; i < part.ranges.size(); ++i) {
        uint32_t *d = rw.data() + i * hspmm::kRangeWords;
        d[0] = part.ranges[i].tile_begin; d[1] = part.ranges[i].tile_end; d[2] = part.ranges[i].first_window;
        d[3] = part.ranges[i].head_slot; d[4] = part.ranges[i].tail_slot;
        d[5] = part.ranges[i].head_split; d[6] = part.ranges[i].tail_split;
        d[7] = part.ranges[i].combine;
    }
    std::vector<uint32_t> sw(part.split.size() * hspmm::kFixWords, 0u);
    for (size_t i = 0; i < part.split.size(); ++i) {
        uint32_t *d = sw.data() + i * hspmm::kFixWords;
        d[0] = part.split[i].window; d[1] = part.split[i].slot_begin; d[2] = part.split[i].slot_count;
    }
    int rc;
    if ((rc = upload(&dp.d_ranges, rw.data(), rw.size(), &p->fixed_bytes))) return rc;
    if ((rc = upload(&dp.d_split, sw.data(), sw.size(), &p->fixed_bytes))) return rc;
    if ((rc = upload(&dp.d_fix_slots, part.fix_slots.data(), part.fix_slots.size(), &p->fixed_bytes))) return rc;
    dp.built = true;
    return HSPMM_OK;
}

// The bitmap stream of the gather kernels (Fp16TileDWB in spmm_mfma_kernel.hpp) from the uncompressed 8 x 16 tiles
// of a 16-bit matrix, made on the device from the tiles already uploaded (p->d_data): per tile the bitmap of the
// reference's CSR2BTCF (bit 16 r + k for element (r, k), reference src/utils/convert.h:83-101; an element is stored
// when its bit pattern is not +0) as four 32-bit words, the bit counts of words 0, 0..1 and 0..2 in bytes 1..3 of
// word 4, and in word 5 the position of the tile's first stored element in `vals` (the reference's nnzOffset),
// where the stored elements follow tile after tile in bit order.  Leaves p->bm.built false when the positions
// would not fit 31 bits.  (On the host this took 29 ms for the 257 MB of tiles of the 2^20 power-law graph.)
int bitmap_from_uploaded_tiles(hspmm_plan *p, uint32_t T)
{
    const uint32_t n_blocks = hspmm::bitmap_scan_blocks(T);
    const size_t header_bytes = size_t(T) * (p->elem == 2u ? 32u : 16u);     // fp32 tiles (8 x 8): two mask words, position, count
    const size_t spare = 8u / p->elem;                                        // a lane may read 8 bytes from the last element on
    uint64_t *d_sums = nullptr;
    HSPMM_HIP(hipMalloc(reinterpret_cast<void **>(&p->bm.d_header), header_bytes));        // (released by hspmm_destroy)
    HSPMM_HIP(hipMalloc(reinterpret_cast<void **>(&d_sums), (size_t(n_blocks) + 1u) * sizeof(uint64_t)));
    auto done = [&](int code) { (void)hipFree(d_sums); return code; };
    HSPMM_HIP_OR(hspmm::launch_bitmap_header(int(p->elem), p->d_data, p->bm.d_header, T, d_sums, nullptr), done);
    uint64_t stored = 0;
    HSPMM_HIP_OR(hipMemcpy(&stored, d_sums + n_blocks, sizeof(stored), hipMemcpyDeviceToHost), done);
    if (stored + spare >= (uint64_t(1) << 31)) {                // positions are 32-bit
        (void)hipFree(p->bm.d_header);
        p->bm.d_header = nullptr;
        return done(HSPMM_OK);
    }
    char *dv = nullptr;
    HSPMM_HIP_OR(hipMalloc(reinterpret_cast<void **>(&dv), (size_t(stored) + spare) * p->elem), done);
    p->bm.d_vals = dv;
    HSPMM_HIP_OR(hipMemset(dv + size_t(stored) * p->elem, 0, spare * p->elem), done);
    HSPMM_HIP_OR(hspmm::launch_bitmap_pack(int(p->elem), p->d_data, p->bm.d_header, dv, T, d_sums, nullptr), done);
    HSPMM_HIP_OR(hipStreamSynchronize(nullptr), done);
    p->bm.stored = stored;
    p->bm.built = true;
    p->fixed_bytes += header_bytes + (size_t(stored) + spare) * p->elem;
    return done(HSPMM_OK);
}

// Re-tiles the matrix panel by panel for the LDS-panel kernels (spmm_panel_kernel.hpp):
// inside every window the columns of one panel of kPanelRows columns get tiles of
// their own.  Every step carries the number of panels it lies behind the step in
// front of it (4 bits; a longer run of panels without a step gets an all-zero step
// every 15 panels).  Returns false when the kernels would not pay (criteria inside).
bool build_panel_stream(hspmm_plan *p, const StepStream &gather_st, const uint32_t *rowOffset, const uint32_t *tcA2B,
                        const void *data, const uint32_t *rowIdx, bool forced, int *rc_out)
{
    *rc_out = HSPMM_OK;
    PhaseTimer timer;
    const uint32_t cw = p->cw, W = p->W;
    // fp32: products of bf16 hi / lo parts (Fp32Split) unless the caller asked for fp32 products
    const bool split = p->dtype == HSPMM_TF32 && p->cfg.kernel_mode != 5;
    const uint32_t KP = (cw == 16 || split) ? hspmm::kPanelRowsWide : hspmm::kPanelRowsFp32;
    const uint32_t NP = (p->cols + KP - 1) / KP;
    constexpr uint32_t kMaxJump = 15;
    if (gather_st.unitRow.empty() || NP == 0) return false;
    // worth it when a unit has a few steps in every 128 columns it meets: the panel image is
    // then read from LDS several times per load from the L2.  Measured break-even against the gather
    // kernels on uniformly random matrices: 1.2 tiles per 128 columns for the kernels built on the
    // 16-bit MFMA (8192 x 8192 at 2 %, fp16: 31 against 34 us at N = 128, 56 against 110 at N = 512; at
    // 1 %: 29 against 16 and 48 against 42), about 2 for the fp32 MFMA forms.
    const double density = double(gather_st.n_steps) / (double(gather_st.unitRow.size()) * double((p->cols + 127u) / 128u));
    if (!forced && density < ((cw == 16 || split) ? 1.2 : 2.0)) return false;
    if (uint64_t(gather_st.unitRow.size()) * (NP + 1) > (1ull << 28)) return false;
    // columns per re-tiled step: the kernels built on 16-bit MFMAs contract 32 columns per step, the fp32
    // MFMA kernels a tile's 8
    const uint32_t rw = (cw == 16 || split) ? 32u : cw;
    // The units of this stream.  The kernels built on the 16-bit MFMA run groups of up to four adjacent
    // windows with one column list as one unit, and give neighbours the union of their lists wherever
    // that saves work (merge_groups); the fp32 MFMA forms walk the units of the gather kernels.
    Unioned un;
    StepStream st = gather_st;
    if (rw == 32 && p->cfg.pairing != 1 && W > 1) {
        // Units of three and four windows halve the LDS reads per row but leave half as many, twice as
        // long waves: measured on pruned and block-clustered 16-bit matrices they pay once the units
        // still fill the compute units at small N (16384 rows: 1.0 - 1.2 x, 28672 rows: 1.2 - 1.3 x;
        // 8192 and 11008 rows: 0.93 - 1.1 x up to N = 512, 1.2 - 1.3 x only from N = 2048 on), and for
        // fp32 storage in bf16 parts, with twice the MFMAs per LDS read, they gain nothing (0.82 - 1.2 x).
        // Pairing mode 2 takes them wherever windows qualify.
        const double wide_cost = kPanelWideCost;
        uint32_t max_windows = (p->cfg.pairing == 2 || cw == 16) ? 4u : 2u;
#ifndef HSPMM_EXPERIMENTAL
        if (split) max_windows = 2u;            // (units of four windows in bf16 parts measured 0.82 - 1.2 x: not built)
#endif
        size_t min_wide_units = p->cfg.pairing == 2 ? 0u : size_t(p->compute_units) * 3u / 2u;
        if (p->cfg.panel_max_windows) {                                                           // tuning override
            max_windows = uint32_t(p->cfg.panel_max_windows);
            min_wide_units = 0;
#ifndef HSPMM_EXPERIMENTAL
            if (split) max_windows = 2u;
#endif
        }
        std::vector<uint32_t> first, count;
        group_windows(W, cw, uint32_t(p->elem), KP, rw, max_windows, wide_cost, min_wide_units, rowOffset, tcA2B, data,
                      rowIdx, un, first, count);
        st = StepStream();
        st.unitOffset.push_back(0);
        uint32_t widest = 1;
        for (size_t g = 0; g < first.size(); ++g) {
            const uint32_t w = first[g];
            st.unitWindow.push_back(w);
            st.unitRow.push_back(rowIdx[w] | (count[g] - 1u));
            st.unitOffset.push_back(st.unitOffset.back() + (rowOffset[w + 1] - rowOffset[w]));
            st.n_paired += count[g] >= 2u;
            st.n_wide += count[g] >= 3u;
            widest = std::max(widest, count[g]);
        }
        st.n_steps = st.unitOffset.back();
        st.G = widest >= 3u ? 4 : int(widest);
    }
    timer.mark("  panel: units of windows");
    const uint32_t U = uint32_t(st.unitRow.size());
    const uint32_t T = rowOffset[W];
    // Two units per consumer wave (merge_unit_pairs below): the second unit's first step follows whatever step of
    // the first unit lies in front of it, so it, too, may be at most kMaxJump panels from its predecessor - every
    // unit of such a stream gets its all-zero steps from panel 0 on, not only behind its first step.
    const bool tall_stream = rw == 32 && st.G <= 2 && U >= 2 && (p->cfg.panel_tall > 0 || p->cfg.panel_packed > 0);
    const size_t es = p->elem, src_tile_bytes = size_t(8) * cw * es, tile_bytes = size_t(8) * rw * es;
    // Two passes over the windows, both on all cores: the steps every window gets, then the steps.
    std::vector<uint32_t> rt_rowOffset(size_t(W) + 1, 0u), rt_panel;
    const uint8_t *src_data = static_cast<const uint8_t *>(data);
    auto real_columns = [&](uint32_t w) {
        const uint32_t *col = tcA2B + size_t(rowOffset[w]) * cw;
        uint32_t nreal = (rowOffset[w + 1] - rowOffset[w]) * cw;
        while (nreal && col[nreal - 1] == HSPMM_IDX_MAX) --nreal;
        return nreal;
    };
    const size_t windows_per_worker = std::max<size_t>(1, (size_t(1) << 14) / std::max<uint32_t>(1u, T / W));
    hspmm_host::parallel_blocks(W, windows_per_worker, [&](size_t wb, size_t we) {
        for (size_t w = wb; w < we; ++w) {
            const uint32_t *col = tcA2B + size_t(rowOffset[w]) * cw;
            const uint32_t nreal = real_columns(uint32_t(w));
            uint32_t i = 0, tiles = 0, last_pn = 0;
            while (i < nreal) {
                const uint32_t pn = col[i] / KP, a = i;
                while (i < nreal && col[i] / KP == pn) ++i;
                while ((tiles || tall_stream) && pn - last_pn > kMaxJump) { last_pn += kMaxJump; ++tiles; }
                tiles += (i - a + rw - 1) / rw;
                last_pn = pn;
            }
            rt_rowOffset[w + 1] = tiles;
        }
    });
    for (uint32_t w = 0; w < W; ++w) rt_rowOffset[w + 1] += rt_rowOffset[w];
    const size_t RT = rt_rowOffset[W];
    hspmm_host::ZeroedBuffer<uint32_t> rt_ids(RT * rw);
    rt_panel.assign(RT, 0u);
    hspmm_host::ZeroedBuffer<uint8_t> rt_data(RT * tile_bytes);
    hspmm_host::parallel_blocks(W, windows_per_worker, [&](size_t wb, size_t we) {
        for (size_t w = wb; w < we; ++w) {
            const uint32_t t0 = rowOffset[w];
            const uint32_t *col = tcA2B + size_t(t0) * cw;
            const uint32_t nreal = real_columns(uint32_t(w));
            uint32_t i = 0, last_pn = 0;
            size_t at = rt_rowOffset[w];                             // next step of the window
            while (i < nreal) {
                const uint32_t pn = col[i] / KP, a = i;
                while (i < nreal && col[i] / KP == pn) ++i;
                while ((at > rt_rowOffset[w] || tall_stream) && pn - last_pn > kMaxJump) {   // all-zero step that only carries the jump
                    last_pn += kMaxJump;
                    rt_panel[at++] = last_pn;
                }
                const uint32_t cnt = i - a, nt = (cnt + rw - 1) / rw;
                // The columns of every step.  16-bit MFMA forms: one LDS instruction reads, in each block of 16
                // lanes, the rows of four columns of the step (block g, instruction h: columns 8g + 4h .. + 3), the
                // LDS serves two blocks (g = 0, 1 or g = 2, 3) at a time, and rows whose numbers differ mod 8 lie
                // in different banks.  So a step should hold every remainder mod 8 at most four times, dealt out over
                // the four sets of eight columns that are read together.  Any choice of columns makes a step: the
                // window's columns in this panel, ordered by remainder (stable), are dealt out over the panel's
                // steps in turn - a step then holds floor or ceil of every remainder's share (pruned weights at 10 %:
                // about 26 of 32 rows per remainder and 7 steps; consecutive columns per step gave five or six of one
                // remainder in most steps, one conflict cycle per LDS read) and the steps are equally full.
                uint32_t perm[hspmm::kPanelRowsWide];
                if (rw == 32) {
                    uint32_t m = 0;
                    for (uint32_t res = 0; res < 8; ++res)
                        for (uint32_t k = a; k < i; ++k)
                            if (((col[k] - pn * KP) & 7u) == res) perm[m++] = k;
                }
                for (uint32_t tl = 0; tl < nt; ++tl, ++at) {
                    rt_panel[at] = pn;
                    // n columns: rw == 32: perm[tl], perm[tl + nt], ... (in remainder order); else consecutive ones
                    const uint32_t n = rw == 32 ? (cnt - tl + nt - 1) / nt : std::min(rw, cnt - tl * rw);
                    auto source = [&](uint32_t k) { return rw == 32 ? perm[tl + k * nt] : a + tl * rw + k; };
                    uint32_t order[32];
                    if (rw == 32) {
                        for (uint32_t k = 0; k < rw; ++k) {
                            const uint32_t set = k % 4, e = k / 4;          // set = 2 * (g / 2) + h
                            const uint32_t g = 2 * (set / 2) + e / 4, h = set % 2;
                            order[8 * g + 4 * h + e % 4] = k;
                        }
                    } else {
                        for (uint32_t k = 0; k < rw; ++k) order[k] = k;
                    }
                    uint8_t *dt_tile = rt_data.data() + at * tile_bytes;
                    for (uint32_t k = 0; k < rw; ++k) {
                        const uint32_t from = order[k];
                        // Padding (its tile column stays zero) takes the row of a real column that is read together
                        // with it - entries four apart are in one set - so that it asks for no bank of its own: lanes
                        // that read one address are served together.
                        uint32_t real = from;
                        while (real >= n && real >= 4u) real -= 4u;
                        if (real >= n) real = n - 1;
                        const uint32_t srci = source(real);
                        rt_ids[at * rw + k] = col[srci] - pn * KP;      // row inside the panel
                        if (from >= n) continue;
                        const uint8_t *st_tile = src_data + size_t(t0 + srci / cw) * src_tile_bytes;
                        for (uint32_t r = 0; r < 8; ++r)
                            std::memcpy(dt_tile + (size_t(r) * rw + k) * es, st_tile + (size_t(r) * cw + srci % cw) * es, es);
                    }
                }
                last_pn = pn;
            }
        }
    });
    timer.mark("  panel: steps per panel");
    // the units with the re-tiled step counts
    StepStream ps;
    ps.G = st.G; ps.unitRow = st.unitRow; ps.unitWindow = st.unitWindow; ps.n_paired = st.n_paired; ps.n_wide = st.n_wide;
    ps.unitOffset.assign(1, 0u);
    for (uint32_t u = 0; u < U; ++u) {
        const uint32_t w = st.unitWindow[u];
        ps.unitOffset.push_back(ps.unitOffset.back() + (rt_rowOffset[w + 1] - rt_rowOffset[w]));
    }
    ps.n_steps = ps.unitOffset.back();
    // padding inside every panel must not eat the gain
    // (fp32 MFMA forms only: the measurements above include the padding of the 32-column steps)
    if (!forced && rw == cw && double(ps.n_steps) > 1.35 * double(gather_st.n_steps)) return false;
    // poff[u][pn]: first step of unit u at or behind panel pn; step_panel[s]: panel of step s
    std::vector<uint32_t> poff(size_t(U) * (NP + 1)), step_panel(ps.n_steps ? ps.n_steps : 1, 0u);
    // fp32, per step four words: word g packs the panel rows quarter-wave g reads (ids g and g + 4, 7 bits
    // each) and in bits 28..31 the panels the step lies behind its predecessor.
    // 16-bit types, per step one word per four lanes (word q = l / 4, g = q / 4): 9 x the panel rows of
    // columns 8g + q % 4 (bits 4..15) and 8g + 4 + q % 4 (bits 16..27); bits 0..3: the panel count.
    const uint32_t id_words = rw == 32 ? 16u : 4u;
    std::vector<uint32_t> ids(size_t(ps.n_steps) * id_words);
    // fp32 single windows run through the 4x4x1 instruction, which wants row offsets (see Fp32Quad)
    const bool quad = p->dtype == HSPMM_TF32 && !split && st.G == 1;
    hspmm_host::parallel_blocks(U, 16, [&](size_t ub, size_t ue) {
        for (size_t u = ub; u < ue; ++u) {
            const uint32_t t0 = rt_rowOffset[st.unitWindow[u]], n = ps.unitOffset[u + 1] - ps.unitOffset[u];
            uint32_t *po = poff.data() + size_t(u) * (NP + 1);
            uint32_t at = 0;
            for (uint32_t pn = 0; pn <= NP; ++pn) {
                while (at < n && rt_panel[t0 + at] < pn) ++at;
                po[pn] = ps.unitOffset[u] + at;
            }
            for (uint32_t i = 0; i < n; ++i) {
                const uint32_t *src = rt_ids.data() + size_t(t0 + i) * rw;
                uint32_t *dst = ids.data() + size_t(ps.unitOffset[u] + i) * id_words;
                const uint32_t jump = i ? rt_panel[t0 + i] - rt_panel[t0 + i - 1] : 0u;     // <= kMaxJump by construction
                step_panel[ps.unitOffset[u] + i] = rt_panel[t0 + i];
                if (rw == 32) {
                    for (uint32_t q = 0; q < 16; ++q) {
                        const uint32_t c0 = 8u * (q >> 2) + (q & 3u);
                        dst[q] = jump | (src[c0] * 9u) << 4 | (src[c0 + 4] * 9u) << 16;
                    }
                    continue;
                }
                for (uint32_t g = 0; g < 4; ++g) {
                    if (quad)   // byte offsets of rows g and g + 4 inside the panel image; the jump in bits 0..3 of word 0
                        dst[g] = (src[g] << 8 | (g == 0 ? jump : 0u)) | (src[g + 4] << 8) << 16;
                    else
                        dst[g] = (src[g] | src[g + 4] << 7) | jump << 28;
                }
            }
        }
    });
    timer.mark("  panel: ids, offsets");
    hspmm_plan::Panel &pl = p->panel;
    int rc;
    hspmm_host::ZeroedBuffer<uint32_t> tiles = split      ? lane_order_split_steps(ps, rt_rowOffset.data(), rt_data.data())
                                  : cw == 16 ? lane_order_wide_steps(ps, rt_rowOffset.data(), rt_data.data())
                                             : lane_order_tiles(ps, p->dtype, rt_rowOffset.data(), rt_data.data());
    // Two units per consumer wave, and tiles without their zeros (kernels built on the 16-bit MFMA, units of one
    // or two windows): fewer 128-byte lines through the compute units' L1s (one copy of a panel in LDS serves
    // twice the rows; a packed step is its stored values and 64 bytes of masks).  Measured, the lines go down
    // by a third and by 60 % and the time does not: what binds these kernels is the LDS reads and MFMAs of a
    // step, which a SIMD runs one after the other.  Both are therefore taken on request only
    // (hspmm_set_panel_stream, HSPMM_PANEL_TALL / HSPMM_PANEL_PACKED).
    timer.mark("  panel: tiles in lane order");
    bool tall = false, packed = false;
    if (tall_stream) {
        tall = true;
        const size_t tile_words = split ? 512u : 256u;
        merge_unit_pairs(U, NP, tile_words, ps.unitOffset, poff, step_panel, ids, tiles);
        packed = p->cfg.panel_packed > 0;
    }
    if ((rc = upload(&pl.d_poff, poff.data(), poff.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
    if ((rc = upload(&pl.d_step_panel, step_panel.data(), step_panel.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
    if ((rc = upload(&pl.d_ids, ids.data(), ids.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
    if (packed) {
        std::vector<uint64_t> masks;
        std::vector<uint8_t> vals;
        std::vector<uint32_t> step_voff;
        pack_steps(ps.n_steps, split, tiles, masks, vals, step_voff);
        if (vals.size() >= (size_t(1) << 32)) packed = false;        // positions are 32-bit byte offsets in the kernel
        else {
            uint8_t *dv = nullptr;
            if ((rc = upload(&pl.d_masks, masks.data(), masks.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
            if ((rc = upload(&dv, vals.data(), vals.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
            pl.d_vals = dv;
            if ((rc = upload(&pl.d_step_voff, step_voff.data(), step_voff.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
        }
    }
    if (!packed) {
        uint32_t *dt = nullptr;
        if ((rc = upload(&dt, tiles.data(), tiles.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
        pl.d_tiles = dt;
    }
    pl.tall = tall; pl.packed = packed;
    if (tall) {
        size_t stored = 0;
        const uint16_t *hv = reinterpret_cast<const uint16_t *>(tiles.data());
        if (packed) for (size_t i = 0, n = tiles.size() * 2; i < n; ++i) stored += hv[i] != 0;
        const double step_bytes = 64.0 + (packed ? 64.0 + 2.0 * double(stored) / double(std::max<uint32_t>(ps.n_steps, 1u))
                                                 : double(tiles.size()) * 4.0 / double(std::max<uint32_t>(ps.n_steps, 1u)));
        pl.unit_lines = step_bytes * double(ps.n_steps) / (double(U) * double(NP)) / 128.0;
    }
    if ((rc = upload(&pl.d_unitRow, st.unitRow.data(), st.unitRow.size(), &p->fixed_bytes))) { *rc_out = rc; return false; }
    pl.n_units = U; pl.G = st.G; pl.n_paired = st.n_paired; pl.n_wide = st.n_wide;
    pl.n_panels = NP; pl.n_steps = ps.n_steps; pl.quad = quad; pl.split = split; pl.density = density; pl.built = true;
    timer.mark("  panel: upload");
    return true;
}

struct Choice {
    bool scalar;
    int layout, V, block_feat;
    bool narrow;
};

// split_features: prefer the load width of one 128-byte line per row and feature block (blocks with XCDs of their own, see
// spmm_mfma_kernel), where the feature dimension allows it.
// N: features of the launch; ld: elements from one row of B and C to the next (N, or more for a range of the features).
Choice choose_kernel(const hspmm_plan *p, const void *dB, const void *dC, uint32_t N, uint32_t ld, bool split_features = false)
{
    Choice c{};
    const uintptr_t align = reinterpret_cast<uintptr_t>(dB) | reinterpret_cast<uintptr_t>(dC);
    const uint64_t row_bytes = uint64_t(ld) * p->elem;
    c.narrow = p->cols < (1u << 24) && row_bytes < (1u << 24) && uint64_t(p->cols) * row_bytes <= (1ull << 32);
    const int mode = p->cfg.kernel_mode;
    if (mode == 1) { c.scalar = true; return c; }
    if (p->dtype != HSPMM_TF32) {
        if ((N % 2 != 0 && N >= 3) || (N % 2 == 0 && (align & 3u))) {
            // rows that start on odd halves (an odd N, or B or C itself): one word per lane, loaded wherever it
            // lies; the lane with the last feature of an odd N owns it alone (mark_half_lane in spmm_mfma_kernel.hpp)
            c.layout = hspmm::kLayoutX4; c.V = 1; c.block_feat = 32;
            return c;
        }
        if (N % 2 != 0) { c.scalar = true; return c; }
        // word loads measured equal to or faster than wide loads wherever both apply
        const bool dw_ok = (N % 64 == 0);
        if (mode != 2 && (dw_ok || mode == 3) && N % 32 == 0) {
            c.layout = hspmm::kLayoutDW;
            c.V = (N % 128 == 0) ? 4 : (N % 64 == 0) ? 2 : 1;
            // one 128-byte line per row and feature block while that gives at most eight blocks
            if (split_features && (N == 128 || N == 256 || N == 512)) c.V = 2;
            c.block_feat = 32 * c.V;
            return c;
        }
        c.layout = hspmm::kLayoutX4;
        // the narrowest block of features (32 V) that covers N: a wave multiplies its whole block whatever N is
        // (power-law graph, N = 32: 293 -> 225 us with V = 1 instead of 2; N = 48: V = 2 instead of 4)
        if (N % 8 == 0 && !(align & 15u) && N > 64) c.V = 4;
        else if (N % 4 == 0 && !(align & 7u) && N > 32) c.V = 2;
        else c.V = 1;
        if (split_features && c.V == 4 && (N == 128 || N == 256 || N == 512)) c.V = 2;
        c.block_feat = 32 * c.V;
        return c;
    }
    if (align & 3u) { c.scalar = true; return c; }
    c.layout = hspmm::kLayoutX4;
    if (N % 4 == 0 && !(align & 15u) && N > 32) c.V = 4;         // (as above: blocks of 16 V features)
    else if (N % 2 == 0 && !(align & 7u) && N > 16) c.V = 2;
    else c.V = 1;
    // (feature blocks of one 128-byte line with XCDs of their own, what the 16-bit types gain from, lose here:
    // power-law graph 2^20 in fp32, N = 64: 590 -> 714 us, N = 128: 1191 -> 1337 us)
    c.block_feat = 16 * c.V;
    return c;
}

// How a launch gets the memory it needs beyond the plan's fixed arrays.
//   kLaunch:  hspmm_run - may build a partition and grow the plan's scratch buffer (under the plan's mutex)
//   kPrepare: hspmm_prepare - builds and grows exactly like kLaunch and launches nothing
//   kStatic:  hspmm_run_static - partial sums go to the library's fixed device array; builds and allocates nothing
enum class RunMode { kLaunch, kPrepare, kStatic };

// The fixed scratch array of hspmm_run_static: one copy per device, held from the moment the library is
// loaded on that device until the process ends.  Host code never passes the array's name to a kernel (on
// the host it names a stand-in, not device memory): the device address is looked up once per device with
// hipGetSymbolAddress and that pointer is what launches carry.
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void *g_static_scratch_ptr[kMaxDevices] = {};

// `device` must be the current device.
int static_scratch_address(int device, float **out)
{
    if (device < 0 || device >= kMaxDevices) return fail(HSPMM_ERR_UNSUPPORTED, "device %d: at most %d devices", device, kMaxDevices);
    std::lock_guard<std::mutex> lk(g_static_mutex);
    if (!g_static_scratch_ptr[device]) {
        void *ptr = nullptr;
        HSPMM_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(hspmm_static_scratch)));
        if (!ptr) return fail(HSPMM_ERR_DEVICE, "hipGetSymbolAddress gave no address for the static scratch array");
        g_static_scratch_ptr[device] = ptr;
    }
    *out = static_cast<float *>(g_static_scratch_ptr[device]);
    return HSPMM_OK;
}

// The set of buffers a launch on stream s uses (see hspmm_plan::StreamBuffers); create = false (hspmm_run_static,
// which allocates nothing): the stream's own set if it has one, else set 0, null if there is none yet.
// Called with the plan's mutex held; the reference is good until the mutex is released.
hspmm_plan::StreamBuffers *buffers_for(hspmm_plan *p, hipStream_t s, bool create)
{
    for (auto &b : p->buffers)
        if (b.stream == s && !b.unowned) return &b;
    // the set hspmm_prepare made before any launch goes to the first stream that launches (also one under capture)
    if (!p->buffers.empty() && p->buffers[0].unowned) {
        p->buffers[0].stream = s;
        p->buffers[0].unowned = false;
        return &p->buffers[0];
    }
    if (!create) return p->buffers.empty() ? nullptr : &p->buffers[0];
    bool own_set = p->buffers.size() < hspmm_plan::kMaxStreamBuffers;
    if (own_set && !p->buffers.empty() && s != nullptr) {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &status) != hipSuccess || status != hipStreamCaptureStatusNone) own_set = false;
    }
    if (!own_set && !p->buffers.empty()) return &p->buffers[0];
    p->buffers.emplace_back();
    p->buffers.back().stream = s;
    return &p->buffers.back();
}

// The sets of buffers a call fills: that of the stream; hspmm_prepare (no stream, nothing launched): every set
// there is, set 0 made if there is none.  Called with the plan's mutex held.
std::vector<hspmm_plan::StreamBuffers *> sets_for(hspmm_plan *p, hipStream_t s, RunMode mode)
{
    std::vector<hspmm_plan::StreamBuffers *> sets;
    if (mode != RunMode::kPrepare) {
        sets.push_back(buffers_for(p, s, true));
        return sets;
    }
    if (p->buffers.empty()) {
        p->buffers.emplace_back();
        p->buffers.back().unowned = true;
    }
    for (auto &b : p->buffers) sets.push_back(&b);
    return sets;
}

// Arrival counters of the in-kernel reduction (never used by hspmm_run_static).
// Called with the plan's mutex held.
int ensure_arrive(hspmm_plan *p, hipStream_t s, size_t words, RunMode mode, uint32_t **out)
{
    for (hspmm_plan::StreamBuffers *b : sets_for(p, s, mode)) {
        if (words > b->arrive_words) {
            uint32_t *fresh = nullptr;
            HSPMM_HIP(hipMalloc(reinterpret_cast<void **>(&fresh), words * 4));
            if (mode == RunMode::kPrepare) {
                // no stream yet: cleared now, and waited for, so that any stream may launch afterwards
                HSPMM_HIP(hipMemset(fresh, 0, words * 4));
                HSPMM_HIP(hipStreamSynchronize(nullptr));
            } else {
                // cleared by a kernel on the launching stream, in front of the launch that counts in it
                HSPMM_HIP(hspmm::launch_fill_zero(fresh, words * 4, s));
            }
            if (b->d_arrive) p->retired.push_back(b->d_arrive);
            b->d_arrive = fresh;
            b->arrive_words = words;
            p->fixed_bytes += words * 4;
        }
        *out = b->d_arrive;
    }
    return HSPMM_OK;
}

// The buffer for `bytes` of partial sums.  kStatic: the device's fixed array (bytes must fit).  Else the
// buffer of the stream's set, grown when too small (sizes are powers of two, so the superseded buffers, which stay
// allocated until hspmm_destroy, never add up to more than the current one).  Called with the plan's mutex held.
int scratch_for(hspmm_plan *p, hipStream_t s, size_t bytes, RunMode mode, float **out)
{
    if (mode == RunMode::kStatic) {
        if (bytes > kStaticScratchBytes)
            return fail(HSPMM_ERR_UNSUPPORTED,
                        "hspmm_run_static: this launch needs %zu bytes of partial sums, the fixed array holds %zu "
                        "(use hspmm_run)", bytes, kStaticScratchBytes);
        return static_scratch_address(p->device, out);
    }
    for (hspmm_plan::StreamBuffers *b : sets_for(p, s, mode)) {
        if (bytes > b->scratch_bytes) {
            size_t cap = size_t(1) << 16;
            while (cap < bytes) cap <<= 1;
            float *fresh = nullptr;
            HSPMM_HIP(hipMalloc(reinterpret_cast<void **>(&fresh), cap));
            if (b->d_scratch) { p->retired.push_back(b->d_scratch); p->retired_bytes += b->scratch_bytes; }
            b->d_scratch = fresh;
            b->scratch_bytes = cap;
        }
        *out = b->d_scratch;
    }
    return HSPMM_OK;
}

}  // namespace

static int run_impl(hspmm_plan *p, const void *dB, void *dC, uint32_t N, void *stream, hipEvent_t mid, RunMode mode);

extern "C" {

const char *hspmm_last_error(void) { return g_last_error.c_str(); }

int hspmm_configure(int buffer_stage, int consumer_warp_num, int producer_warp_group_num, int sm_num)
{
#ifdef HSPMM_EXPERIMENTAL
    if (buffer_stage < 0 || buffer_stage > 8 || buffer_stage == 5 || buffer_stage == 7)
        return fail(HSPMM_ERR_INVALID, "buffer_stage %d: supported depths are 1, 2, 3, 4, 6, 8 (0 = default)", buffer_stage);
#else
    if (buffer_stage != 0 && (buffer_stage < 2 || buffer_stage > 4))
        return fail(HSPMM_ERR_INVALID, "buffer_stage %d: supported depths are 2, 3, 4 (0 = default)", buffer_stage);
#endif
    if (consumer_warp_num < 0 || consumer_warp_num > hspmm::kMaxWavesPerGroup)
        return fail(HSPMM_ERR_INVALID, "consumer_warp_num %d outside 0..%d", consumer_warp_num, hspmm::kMaxWavesPerGroup);
    if (producer_warp_group_num < 0 || producer_warp_group_num > 16)
        return fail(HSPMM_ERR_INVALID, "producer_warp_group_num %d outside 0..16", producer_warp_group_num);
    if (sm_num < 0 || sm_num > 4096) return fail(HSPMM_ERR_INVALID, "sm_num %d outside 0..4096", sm_num);
    std::lock_guard<std::mutex> lk(g_cfg_mutex);
    g_cfg.buffer_stage = buffer_stage;
    g_cfg.consumer_warp_num = consumer_warp_num;
    g_cfg.producer_warp_group_num = producer_warp_group_num;
    g_cfg.sm_num = sm_num;
    return HSPMM_OK;
}

void hspmm_get_config(int *buffer_stage, int *consumer_warp_num, int *producer_warp_group_num, int *sm_num)
{
    std::lock_guard<std::mutex> lk(g_cfg_mutex);
    if (buffer_stage) *buffer_stage = g_cfg.buffer_stage;
    if (consumer_warp_num) *consumer_warp_num = g_cfg.consumer_warp_num;
    if (producer_warp_group_num) *producer_warp_group_num = g_cfg.producer_warp_group_num;
    if (sm_num) *sm_num = g_cfg.sm_num;
}

int hspmm_set_kernel_mode(int mode)
{
    if (mode < 0 || mode > 5) return fail(HSPMM_ERR_INVALID, "kernel mode %d outside 0..5", mode);
    std::lock_guard<std::mutex> lk(g_cfg_mutex);
    g_cfg.kernel_mode = mode;
    return HSPMM_OK;
}

int hspmm_set_window_pairing(int mode)
{
    if (mode < 0 || mode > 2) return fail(HSPMM_ERR_INVALID, "pairing mode %d outside 0..2", mode);
    std::lock_guard<std::mutex> lk(g_cfg_mutex);
    g_cfg.pairing = mode;
    return HSPMM_OK;
}

int hspmm_set_group_cuts(int mode)
{
    if (mode < 0 || mode > 1) return fail(HSPMM_ERR_INVALID, "group cuts mode %d outside 0..1", mode);
    std::lock_guard<std::mutex> lk(g_cfg_mutex);
    g_cfg.group_cuts = mode;
    return HSPMM_OK;
}

int hspmm_has_experimental(void)
{
#ifdef HSPMM_EXPERIMENTAL
    return 1;
#else
    return 0;
#endif
}

int hspmm_set_panel_stream(int mode)
{
    if (mode < 0 || mode > 2) return fail(HSPMM_ERR_INVALID, "panel stream mode %d outside 0..2", mode);
#ifndef HSPMM_EXPERIMENTAL
    if (mode != 0)
        return fail(HSPMM_ERR_UNSUPPORTED, "panel stream mode %d needs a library built with EXPERIMENTAL=1 (the default "
                    "stream measured faster)", mode);
#endif
    std::lock_guard<std::mutex> lk(g_cfg_mutex);
    g_cfg.panel_tall = mode >= 1;
    g_cfg.panel_packed = mode == 2;
    return HSPMM_OK;
}

static int partition_preview(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                             uint32_t group, uint32_t words, uint32_t *ranges, uint32_t capacity_ranges,
                             uint32_t *n_ranges, uint32_t *n_split_windows, uint32_t *n_partial_slots,
                             const std::vector<uint32_t> *allowed_cuts = nullptr)
{
    if (eff_row_windows && !rowOffset) return fail(HSPMM_ERR_INVALID, "null rowOffset");
    if (group < 1 || group > uint32_t(hspmm::kMaxWavesPerGroup))
        return fail(HSPMM_ERR_INVALID, "group %u outside 1..%d", group, hspmm::kMaxWavesPerGroup);
    for (uint32_t w = 0; w < eff_row_windows; ++w)
        if (rowOffset[w + 1] <= rowOffset[w] || rowOffset[0] != 0)
            return fail(HSPMM_ERR_INVALID, "rowOffset must start at 0 and increase strictly");
    const hspmm::Partition part =
        hspmm::build_partition(eff_row_windows, rowOffset, target_ranges, kWindowCost, kSlack, kWholeWindowMargin, group, allowed_cuts);
    if (n_ranges) *n_ranges = uint32_t(part.ranges.size());
    if (n_split_windows) *n_split_windows = uint32_t(part.split.size());
    if (n_partial_slots) *n_partial_slots = part.n_slots;
    if (ranges) {
        const size_t n = part.ranges.size() < capacity_ranges ? part.ranges.size() : capacity_ranges;
        for (size_t i = 0; i < n; ++i) {
            uint32_t *d = ranges + words * i;
            d[0] = part.ranges[i].tile_begin; d[1] = part.ranges[i].tile_end;
            d[2] = part.ranges[i].first_window;
            d[3] = part.ranges[i].head_slot; d[4] = part.ranges[i].tail_slot;
            if (words > 5) d[5] = part.ranges[i].combine;
        }
    }
    return HSPMM_OK;
}

int hspmm_partition_preview(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                            uint32_t *ranges, uint32_t capacity_ranges, uint32_t *n_ranges,
                            uint32_t *n_split_windows, uint32_t *n_partial_slots)
{
    return partition_preview(eff_row_windows, rowOffset, target_ranges, 1, 5, ranges, capacity_ranges, n_ranges,
                             n_split_windows, n_partial_slots);
}

int hspmm_partition_preview_grouped(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                                    uint32_t group, uint32_t *ranges, uint32_t capacity_ranges, uint32_t *n_ranges,
                                    uint32_t *n_split_windows, uint32_t *n_partial_slots)
{
    return partition_preview(eff_row_windows, rowOffset, target_ranges, group, 6, ranges, capacity_ranges, n_ranges,
                             n_split_windows, n_partial_slots);
}

int hspmm_partition_preview_group_cuts(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                                       uint32_t total_groups, const uint32_t *groupOffset, uint32_t *ranges,
                                       uint32_t capacity_ranges, uint32_t *n_ranges, uint32_t *n_split_windows,
                                       uint32_t *n_partial_slots)
{
    if (!groupOffset) return fail(HSPMM_ERR_INVALID, "null groupOffset");
    if (eff_row_windows && !rowOffset) return fail(HSPMM_ERR_INVALID, "null rowOffset");
    // every window boundary must be the end of a group
    uint32_t g = 0;
    for (uint32_t w = 0; w <= eff_row_windows; ++w) {
        while (g < total_groups && groupOffset[g] < rowOffset[w]) {
            if (groupOffset[g + 1] <= groupOffset[g]) return fail(HSPMM_ERR_INVALID, "groupOffset does not increase at group %u", g);
            ++g;
        }
        if (g > total_groups || groupOffset[g] != rowOffset[w])
            return fail(HSPMM_ERR_INVALID, "window boundary %u (tile %u) is not the end of a group", w, rowOffset[w]);
    }
    const std::vector<uint32_t> cuts(groupOffset, groupOffset + size_t(total_groups) + 1u);
    return partition_preview(eff_row_windows, rowOffset, target_ranges, 1, 5, ranges, capacity_ranges, n_ranges,
                             n_split_windows, n_partial_slots, &cuts);
}

int hspmm_partition_preview_aligned(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t group,
                                    uint32_t *ranges, uint32_t capacity_ranges, uint32_t *n_ranges)
{
    if (eff_row_windows && !rowOffset) return fail(HSPMM_ERR_INVALID, "null rowOffset");
    if (group != uint32_t(hspmm::kMaxWavesPerGroup) && group != uint32_t(hspmm::kAlignedGroupWaves))
        return fail(HSPMM_ERR_INVALID, "group %u: %d or %d", group, hspmm::kMaxWavesPerGroup, hspmm::kAlignedGroupWaves);
    for (uint32_t w = 0; w < eff_row_windows; ++w)
        if (rowOffset[0] != 0 || rowOffset[w + 1] < rowOffset[w] + group)
            return fail(HSPMM_ERR_INVALID, "rowOffset must start at 0 and every window needs at least %u tiles", group);
    const hspmm::Partition part = hspmm::build_aligned_partition(eff_row_windows, rowOffset, group);
    if (n_ranges) *n_ranges = uint32_t(part.ranges.size());
    if (ranges) {
        const size_t n = part.ranges.size() < capacity_ranges ? part.ranges.size() : capacity_ranges;
        for (size_t i = 0; i < n; ++i) {
            uint32_t *d = ranges + 6 * i;
            d[0] = part.ranges[i].tile_begin; d[1] = part.ranges[i].tile_end; d[2] = part.ranges[i].first_window;
            d[3] = part.ranges[i].head_slot; d[4] = part.ranges[i].tail_slot; d[5] = part.ranges[i].combine;
        }
    }
    return HSPMM_OK;
}

int hspmm_panel_units_preview(int dtype, uint32_t rows, uint32_t cols, uint32_t eff_row_windows, uint32_t total_tiles,
                              const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data, const uint32_t *rowIdx,
                              uint32_t max_windows, uint32_t *n_groups, uint32_t *group_first, uint32_t *group_count,
                              uint32_t *new_rowOffset, uint32_t *new_total_tiles, uint32_t capacity_tiles,
                              uint32_t *new_tcA2B, void *new_data)
{
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16)
        return fail(HSPMM_ERR_INVALID, "unknown dtype %d", dtype);
    if (max_windows != 1 && max_windows != 2 && max_windows != 4)
        return fail(HSPMM_ERR_INVALID, "max_windows %u: 1, 2 or 4", max_windows);
    const uint32_t cw = dtype == HSPMM_TF32 ? 8u : 16u, elem = dtype == HSPMM_TF32 ? 4u : 2u;
    bool canonical = true;
    const int rc = validate_format(rows, cols, eff_row_windows, total_tiles, cw, rowOffset, tcA2B, data, rowIdx, &canonical);
    if (rc) return rc;
    const uint32_t W = eff_row_windows;
    Unioned un;
    std::vector<uint32_t> first, count;
    const void *d = data;
    try {
        // column lists that do not ascend strictly, or with padding inside a window, are never merged
        group_windows(W, cw, elem, hspmm::kPanelRowsWide, 32u, canonical ? max_windows : 1u, kPanelWideCost, 0, rowOffset, tcA2B, d,
                      rowIdx, un, first, count);
    } catch (const std::bad_alloc &) { return fail(HSPMM_ERR_ALLOC, "out of host memory"); }
    const uint32_t T = W ? rowOffset[W] : 0u;
    if (n_groups) *n_groups = uint32_t(first.size());
    if (new_total_tiles) *new_total_tiles = T;
    for (size_t g = 0; g < first.size(); ++g) {
        if (group_first) group_first[g] = first[g];
        if (group_count) group_count[g] = count[g];
    }
    if (new_rowOffset && W) std::memcpy(new_rowOffset, rowOffset, (size_t(W) + 1) * 4);
    if (new_tcA2B || new_data) {
        if (T > capacity_tiles)
            return fail(HSPMM_ERR_INVALID, "the grouped matrix has %u tiles, the output arrays hold %u", T, capacity_tiles);
        if (new_tcA2B && T) std::memcpy(new_tcA2B, tcA2B, size_t(T) * cw * 4);
        if (new_data && T) std::memcpy(new_data, d, size_t(T) * 8u * cw * elem);
    }
    return HSPMM_OK;
}

namespace {

// The caller's bitmap tiles (HSPMM_BITS_PER_TILE words: two per 8 x 16 tile, one per 8 x 8 tile of fp32 storage):
// reference BTCF_MTX, src/utils/class.h:55-67.
struct BitmapSource { const uint32_t *nnzOffset; const uint64_t *tcBit; const void *data; };
// The ends of the caller's groups (groupOffset of the reference's GBTCF_MTX, src/utils/class.h:93-108), n + 1 of them.
struct GroupCuts { const uint32_t *offsets; uint32_t n_groups; };
constexpr int kNeedsPlainTiles = -1000;     // create_plan with a BitmapSource: this matrix needs the tiles on the host

// Header of the gather kernels' bitmap stream straight from the caller's arrays; returns the first tile whose bit
// count differs from its nnzOffset span (HSPMM_IDX_MAX: none).
uint32_t bitmap_header_from_caller(uint32_t T, uint32_t elem, const BitmapSource &src, hspmm_host::ZeroedBuffer<uint32_t> &header)
{
    header = hspmm_host::ZeroedBuffer<uint32_t>(size_t(T) * (elem == 2u ? 8u : 4u));
    std::atomic<uint32_t> first_bad{HSPMM_IDX_MAX};
    hspmm_host::parallel_blocks(T, 4096, [&](size_t tb, size_t te) {
        for (size_t t = tb; t < te; ++t) {
            if (elem == 4u) {
                // 8 x 8 tiles of 32-bit elements: one 64-bit word per tile; header = rows 0..3, rows 4..7, position, count
                uint32_t *hd = header.data() + t * 4u;
                hd[0] = uint32_t(src.tcBit[t]); hd[1] = uint32_t(src.tcBit[t] >> 32);
                hd[2] = src.nnzOffset[t];
                hd[3] = uint32_t(__builtin_popcount(hd[0])) + uint32_t(__builtin_popcount(hd[1]));
                if (src.nnzOffset[t + 1] < src.nnzOffset[t] || src.nnzOffset[t + 1] - src.nnzOffset[t] != hd[3]) {
                    uint32_t seen = first_bad.load();
                    while (uint32_t(t) < seen && !first_bad.compare_exchange_weak(seen, uint32_t(t))) {}
                }
                continue;
            }
            uint32_t *hd = header.data() + t * 8u;
            hd[0] = uint32_t(src.tcBit[2 * t]); hd[1] = uint32_t(src.tcBit[2 * t] >> 32);
            hd[2] = uint32_t(src.tcBit[2 * t + 1]); hd[3] = uint32_t(src.tcBit[2 * t + 1] >> 32);
            const uint32_t c0 = uint32_t(__builtin_popcount(hd[0])), c1 = c0 + uint32_t(__builtin_popcount(hd[1])),
                           c2 = c1 + uint32_t(__builtin_popcount(hd[2])), c3 = c2 + uint32_t(__builtin_popcount(hd[3]));
            hd[4] = c0 << 8 | c1 << 16 | c2 << 24;
            hd[5] = src.nnzOffset[t];
            if (src.nnzOffset[t + 1] < src.nnzOffset[t] || src.nnzOffset[t + 1] - src.nnzOffset[t] != c3) {
                uint32_t seen = first_bad.load();
                while (uint32_t(t) < seen && !first_bad.compare_exchange_weak(seen, uint32_t(t))) {}
            }
        }
    });
    return first_bad.load();
}

// hspmm_create; with `bitmap` (data == nullptr) the tiles come as the caller's bitmap arrays,
// which are uploaded as they are, kept as the gather kernels' bitmap stream and expanded on the device for the
// kernels that read plain tiles.  Returns kNeedsPlainTiles when the plan would need the tiles on the host
// (windows paired through equal column lists; the caller then expands them).
int create_plan(hspmm_plan **out, int dtype, uint32_t rows, uint32_t cols, uint32_t eff_row_windows,
                uint32_t total_tiles, const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data,
                const uint32_t *rowIdx, const BitmapSource *bitmap, const GroupCuts *cuts = nullptr)
{
    if (!out) return fail(HSPMM_ERR_INVALID, "null plan pointer");
    *out = nullptr;
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16)
        return fail(HSPMM_ERR_INVALID, "unknown dtype %d", dtype);
    const uint32_t cw = dtype == HSPMM_TF32 ? 8u : 16u;
    const uint32_t elem = dtype == HSPMM_TF32 ? 4u : 2u;
    PhaseTimer timer;
    bool canonical = true;
    int rc = validate_format(rows, cols, eff_row_windows, total_tiles, cw, rowOffset, tcA2B, bitmap ? bitmap->data : data, rowIdx,
                             &canonical);
    if (rc) return rc;
    timer.mark("validate");

    hspmm_plan *p = new (std::nothrow) hspmm_plan;
    if (!p) return fail(HSPMM_ERR_ALLOC, "out of host memory");
    p->dtype = dtype; p->rows = rows; p->cols = cols; p->W = eff_row_windows; p->T = total_tiles;
    p->cw = cw; p->elem = elem; p->canonical = canonical;
    { std::lock_guard<std::mutex> lk(g_cfg_mutex); p->cfg = g_cfg; }
    p->cfg.read_environment();                      // tuning overrides, once per plan

    auto bail = [&](int code) { hspmm_destroy(p); return code; };
    hipError_t e = hipGetDevice(&p->device);
    if (e != hipSuccess) return bail(fail(HSPMM_ERR_DEVICE, "hipGetDevice failed: %s", hipGetErrorString(e)));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, p->device);
    if (e != hipSuccess) return bail(fail(HSPMM_ERR_DEVICE, "hipGetDeviceProperties failed: %s", hipGetErrorString(e)));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return bail(fail(HSPMM_ERR_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only", p->device,
                         prop.gcnArchName));
    p->compute_units = p->cfg.sm_num > 0 ? p->cfg.sm_num : prop.multiProcessorCount;
    {
        // the address of this device's fixed scratch array, for hspmm_run_static (which then looks nothing up)
        float *unused = nullptr;
        if ((rc = static_scratch_address(p->device, &unused))) return bail(rc);
    }

    // (a host allocation that fails anywhere below ends the call with HSPMM_ERR_ALLOC)
    if (p->W) try {
        const size_t n_ids = size_t(total_tiles) * cw;
        if ((rc = upload(&p->d_rowOffset, rowOffset, size_t(p->W) + 1, &p->fixed_bytes))) return bail(rc);
        if ((rc = upload(&p->d_rowIdx, rowIdx, size_t(p->W), &p->fixed_bytes))) return bail(rc);
        if ((rc = upload(&p->d_a2b_raw, tcA2B, n_ids, &p->fixed_bytes))) return bail(rc);
        if (!bitmap) {
            uint8_t *dd = nullptr;
            if ((rc = upload(&dd, static_cast<const uint8_t *>(data), size_t(total_tiles) * 8u * cw * elem,
                             &p->fixed_bytes)))
                return bail(rc);
            p->d_data = dd;
        } else {
            // the caller's bitmap tiles: header from tcBit / nnzOffset, the stored elements as they are (and four
            // more: a lane of the gather kernels reads 8 bytes from its first element), plain tiles by a kernel
            hspmm_host::ZeroedBuffer<uint32_t> header;
            const uint32_t bad = bitmap_header_from_caller(total_tiles, elem, *bitmap, header);
            if (bad != HSPMM_IDX_MAX)
                return bail(fail(HSPMM_ERR_INVALID, "tile %u: %s", bad, "the bit count of tcBit differs from the nnzOffset span"));
            const size_t stored = bitmap->nnzOffset[total_tiles], spare = 8u / elem;
            if (stored + spare >= (size_t(1) << 31)) return bail(kNeedsPlainTiles);      // positions are 32-bit
            if ((rc = upload(&p->bm.d_header, header.data(), header.size(), &p->fixed_bytes))) return bail(rc);
            char *dv = nullptr;
            HSPMM_HIP_OR(hipMalloc(reinterpret_cast<void **>(&dv), (stored + spare) * elem), bail);
            p->bm.d_vals = dv; p->bm.stored = stored; p->fixed_bytes += (stored + spare) * elem;
            if (stored) HSPMM_HIP_OR(hipMemcpy(dv, bitmap->data, stored * elem, hipMemcpyHostToDevice), bail);
            HSPMM_HIP_OR(hipMemset(dv + stored * elem, 0, 8), bail);
            uint8_t *dd = nullptr;
            HSPMM_HIP_OR(hipMalloc(reinterpret_cast<void **>(&dd), size_t(total_tiles) * 256u), bail);
            p->d_data = dd; p->fixed_bytes += size_t(total_tiles) * 256u;
            HSPMM_HIP_OR(hspmm::launch_expand_bitmap(int(elem), p->bm.d_header, dv, dd, total_tiles, nullptr), bail);
            HSPMM_HIP_OR(hipStreamSynchronize(nullptr), bail);
            p->bm.from_caller = true;
        }
        timer.mark("upload format arrays");
        // padding ids -> the real id in front of them (the tile column is all zero)
        // (padding trails a window's real ids, of which every window has one at least)
        hspmm_host::ZeroedBuffer<uint32_t> clean_ids;
        try { clean_ids = hspmm_host::ZeroedBuffer<uint32_t>(n_ids); }
        catch (const std::bad_alloc &) { return bail(fail(HSPMM_ERR_ALLOC, "out of host memory")); }
        uint32_t *clean = clean_ids.data();
        hspmm_host::parallel_blocks(p->W, 1024, [&](size_t wb, size_t we) {
            for (size_t i = size_t(rowOffset[wb]) * cw, e = size_t(rowOffset[we]) * cw; i < e; ++i)
                clean[i] = (tcA2B[i] == HSPMM_IDX_MAX && i) ? clean[i - 1] : tcA2B[i];
        });
        timer.mark("ids without padding");
        const StepStream st = build_units(p->W, cw, rowOffset, rowIdx, clean, p->cfg.pairing);
        timer.mark("units");
        if (bitmap && st.G != 1) return bail(kNeedsPlainTiles);         // paired windows: their tiles are re-laid out on the host
        p->G = st.G;
        p->n_units = uint32_t(st.unitRow.size());
        p->n_paired = st.n_paired;
        p->n_steps = st.n_steps;
        if ((rc = upload(&p->d_unitOffset, st.unitOffset.data(), st.unitOffset.size(), &p->fixed_bytes))) return bail(rc);
        if ((rc = upload(&p->d_unitRow, st.unitRow.data(), st.unitRow.size(), &p->fixed_bytes))) return bail(rc);
        if (dtype != HSPMM_TF32 && st.G == 1) {
            // single 16-bit windows: the steps are the caller's tiles in the caller's order, their ids these
            if ((rc = upload(&p->d_ids, clean, n_ids, &p->fixed_bytes))) return bail(rc);
        } else {
            const hspmm_host::ZeroedBuffer<uint32_t> ids = lane_order_ids(st, dtype, rowOffset, clean);
            if ((rc = upload(&p->d_ids, ids.data(), ids.size(), &p->fixed_bytes))) return bail(rc);
        }
        // (single fp32 windows: decided below, once it is known whether the gather kernels of this plan read
        // bitmap tiles - then nothing reads tiles in lane order)
        const bool lane_tiles_later = dtype == HSPMM_TF32 && st.G == 1;
        if (dtype != HSPMM_TF32 && st.G == 1) {
            p->d_tiles = p->d_data;                 // the caller's tile layout already is the lane order
        } else if (!lane_tiles_later) {
            const hspmm_host::ZeroedBuffer<uint32_t> tiles = lane_order_tiles(st, dtype, rowOffset, data);
            uint32_t *dt = nullptr;
            if ((rc = upload(&dt, tiles.data(), tiles.size(), &p->fixed_bytes))) return bail(rc);
            p->d_tiles = dt;
        }
        timer.mark("step stream (ids, tiles)");
        // Single 16-bit windows with few stored elements per tile (graphs: 16 of 128): the gather kernels read the
        // tiles as bitmap + stored elements, 32 + 2 x 16 bytes per tile instead of 256 (power-law graph 2^20 at
        // N = 128, where the stream is read once per XCD half: 0.64 -> 0.19 GB per launch).
        if (bitmap) {
            // (same rule as below, with the exact number of stored elements)
            const size_t stored = size_t(p->bm.stored);
            p->bm.built = total_tiles && p->cfg.gather_bitmap != 0 &&
                          (p->cfg.gather_bitmap > 0 ||
                           (stored * 3u < size_t(total_tiles) * 8u * cw && size_t(total_tiles) * 256u >= (size_t(8) << 20)));
            if (!p->bm.built) {
                (void)hipFree(p->bm.d_header); (void)hipFree(p->bm.d_vals);
                p->bm.d_header = nullptr; p->bm.d_vals = nullptr;
            }
        } else if (st.G == 1 && p->cfg.gather_bitmap != 0 && total_tiles) {
            const size_t n = size_t(total_tiles) * 8u * cw;                 // tile elements
            size_t stored = 0;
            if (p->cfg.gather_bitmap < 0) {
                const size_t sample = std::min<size_t>(n, size_t(1) << 22);
                if (elem == 2u) {
                    const uint16_t *hv = static_cast<const uint16_t *>(data);
                    for (size_t i = 0; i < sample; ++i) stored += hv[i] != 0;
                } else {
                    const uint32_t *wv = static_cast<const uint32_t *>(data);
                    for (size_t i = 0; i < sample; ++i) stored += wv[i] != 0;
                }
                stored = size_t(double(stored) * double(n) / double(sample));
            }
            // 32 + 2 e bytes against 256 per tile with e stored elements (16 + 4 e for fp32): worth it below about a
            // third full, and where the tile stream is large enough to be traffic at all (a matrix whose tiles sit
            // in the L2s only pays the longer dependent chain: 4096 x 4096 at 1 %, 2.7 MB of tiles: 6.8 -> 7.5 us)
            if (p->cfg.gather_bitmap > 0 ||
                (stored * 3u < n && size_t(total_tiles) * 256u >= (size_t(8) << 20))) {
                if ((rc = bitmap_from_uploaded_tiles(p, total_tiles))) return bail(rc);
            }
        }
        if (lane_tiles_later && total_tiles && !(p->bm.built && (p->cfg.kernel_mode == 0 || p->cfg.kernel_mode == 3))) {
            // single fp32 windows: steps are the caller's tiles in the caller's order; a kernel re-orders each for the lanes
            void *dt = nullptr;
            HSPMM_HIP_OR(hipMalloc(&dt, size_t(total_tiles) * 256u), bail);
            p->d_tiles = dt; p->fixed_bytes += size_t(total_tiles) * 256u;
            HSPMM_HIP_OR(hspmm::launch_lane_order32(p->d_data, dt, total_tiles, nullptr), bail);
            HSPMM_HIP_OR(hipStreamSynchronize(nullptr), bail);
        }
        timer.mark("bitmap tiles");
        p->h_unitOffset = st.unitOffset;
        p->h_unitRow = st.unitRow;
        if (st.G != 1) {
            p->h_winOffset.assign(rowOffset, rowOffset + size_t(p->W) + 1u);
            p->h_winRow.assign(rowIdx, rowIdx + size_t(p->W));
        }
        // single windows walked tile by tile: the caller's tile numbers are the stream's, its cuts can be kept
        if (cuts && p->cfg.group_cuts && st.G == 1) p->caller_cuts.assign(cuts->offsets, cuts->offsets + size_t(cuts->n_groups) + 1u);
        if ((rc = build_and_upload_partition(p, 0))) return bail(rc);
        timer.mark("partition");
        {
            // all units long, and so long that the balanced partition cuts each of them several ways:
            // eight ranges per unit where it would cut eight ways or more, four from `four_from` ways on
            uint32_t shortest = 0xFFFFFFFFu;
            for (size_t u = 0; u + 1 < st.unitOffset.size(); ++u)
                shortest = std::min(shortest, st.unitOffset[u + 1] - st.unitOffset[u]);
            const double steps_per_range = double(p->n_steps) / double(p->parts[0].part.ranges.size());
            const double ways = double(p->n_steps) / double(p->n_units) / steps_per_range;
            const double four_from = kAlignedFourFrom;
            const int group = ways >= 8.0 ? hspmm::kAlignedGroupWaves : ways >= four_from ? hspmm::kMaxWavesPerGroup : 0;
            if (group && shortest >= 8u * uint32_t(group) && uint64_t(p->n_units) * group <= (1u << 24)) p->aligned_group = group;
            // A matrix too small to fill the waves of the GPU with ranges of useful length: what its launch takes
            // is one wave walking its range step by step (4096 x 4096 at 1 %: 434 waves of 24 dependent steps).
            // One workgroup per unit, its waves a quarter (an eighth) of the unit's steps each, shortens that walk.
            const uint64_t wave_slots = uint64_t(p->compute_units) * 16u;
            int small_group = 0;
            if (p->cfg.aligned_small < 0) {
                if (!p->aligned_group && p->parts[0].part.ranges.size() * 4u <= wave_slots && uint64_t(p->n_units) * 4u <= wave_slots)
                    small_group = hspmm::kMaxWavesPerGroup;      // (eight waves per unit measured no faster: 7.2 against 6.8 us)
            } else {
                small_group = p->cfg.aligned_small;
            }
            if (small_group && shortest >= 2u * uint32_t(small_group)) p->aligned_group = small_group;
            if (!p->caller_cuts.empty()) p->aligned_group = 0;       // (those partitions cut every unit into equal parts)
        }
        // (the LDS-panel stream re-tiles ascending column lists; a caller's lists in another order stay
        // with the gather and all-shapes kernels)
        if (!bitmap && (p->cfg.kernel_mode == 0 || p->cfg.kernel_mode >= 4) && p->canonical) {
            int prc = HSPMM_OK;
            try { (void)build_panel_stream(p, st, rowOffset, tcA2B, data, rowIdx, p->cfg.kernel_mode >= 4, &prc); }
            catch (const std::bad_alloc &) { return bail(fail(HSPMM_ERR_ALLOC, "out of host memory")); }
            if (prc) return bail(prc);
            timer.mark("LDS-panel stream");
        }
    } catch (const std::bad_alloc &) {
        return bail(fail(HSPMM_ERR_ALLOC, "out of host memory"));
    }
    *out = p;
    return HSPMM_OK;
}

}  // namespace

int hspmm_create(hspmm_plan **out, int dtype, uint32_t rows, uint32_t cols, uint32_t eff_row_windows,
                 uint32_t total_tiles, const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data,
                 const uint32_t *rowIdx)
{
    return create_plan(out, dtype, rows, cols, eff_row_windows, total_tiles, rowOffset, tcA2B, data, rowIdx, nullptr);
}

namespace {
// Widths a tile layout may have for an element type: the default one, and 4 for fp32 storage.
int layout_widths(int dtype, uint32_t col_window, uint32_t &cw, uint32_t &cw_default, uint32_t &elem)
{
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16)
        return fail(HSPMM_ERR_INVALID, "unknown dtype %d", dtype);
    cw_default = dtype == HSPMM_TF32 ? 8u : 16u;
    elem = dtype == HSPMM_TF32 ? 4u : 2u;
    cw = col_window ? col_window : cw_default;
    if (cw != cw_default && !(dtype == HSPMM_TF32 && cw == 4u))
        return fail(HSPMM_ERR_INVALID, "col_window %u: %u, or 4 for HSPMM_TF32", col_window, cw_default);
    return HSPMM_OK;
}
}  // namespace

int hspmm_btcf_relayout_sizes(int dtype, uint32_t col_window, uint32_t eff_row_windows, const uint32_t *rowOffset,
                              const uint32_t *tcA2B, uint32_t *total_tiles)
{
    uint32_t cw, cw_default, elem;
    if (int rc = layout_widths(dtype, col_window, cw, cw_default, elem)) return rc;
    if (!total_tiles) return fail(HSPMM_ERR_INVALID, "null output");
    const uint32_t W = eff_row_windows;
    if (W && (!rowOffset || !tcA2B)) return fail(HSPMM_ERR_INVALID, "null format array");
    if (W && rowOffset[0] != 0) return fail(HSPMM_ERR_INVALID, "rowOffset[0] = %u, expected 0", rowOffset[0]);
    uint64_t tiles = 0;
    for (uint32_t w = 0; w < W; ++w) {
        if (rowOffset[w + 1] <= rowOffset[w])
            return fail(HSPMM_ERR_INVALID, "rowOffset not strictly increasing at window %u", w);
        const uint32_t *ids = tcA2B + size_t(rowOffset[w]) * cw;
        uint32_t real = 0;
        for (size_t i = 0, n = size_t(rowOffset[w + 1] - rowOffset[w]) * cw; i < n; ++i) real += ids[i] != HSPMM_IDX_MAX;
        if (!real) return fail(HSPMM_ERR_INVALID, "window %u has no column", w);
        tiles += (real + cw_default - 1u) / cw_default;
    }
    if (tiles > 0xffffffffull) return fail(HSPMM_ERR_INVALID, "more than 2^32 - 1 tiles");
    *total_tiles = uint32_t(tiles);
    return HSPMM_OK;
}

int hspmm_btcf_relayout_fill(int dtype, uint32_t col_window, int transposed, uint32_t eff_row_windows,
                             const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data,
                             uint32_t *out_rowOffset, uint32_t *out_tcA2B, void *out_data)
{
    uint32_t cw, cw_default, elem, NT = 0;
    if (int rc = hspmm_btcf_relayout_sizes(dtype, col_window, eff_row_windows, rowOffset, tcA2B, &NT)) return rc;
    layout_widths(dtype, col_window, cw, cw_default, elem);
    const uint32_t W = eff_row_windows;
    if (!out_rowOffset || (NT && (!data || !out_tcA2B || !out_data))) return fail(HSPMM_ERR_INVALID, "null array");
    out_rowOffset[0] = 0;
    for (uint32_t w = 0; w < W; ++w) {
        const uint32_t *ids = tcA2B + size_t(rowOffset[w]) * cw;
        uint32_t real = 0;
        for (size_t i = 0, n = size_t(rowOffset[w + 1] - rowOffset[w]) * cw; i < n; ++i) real += ids[i] != HSPMM_IDX_MAX;
        out_rowOffset[w + 1] = out_rowOffset[w] + (real + cw_default - 1u) / cw_default;
    }
    std::fill(out_tcA2B, out_tcA2B + size_t(NT) * cw_default, HSPMM_IDX_MAX);
    std::memset(out_data, 0, size_t(NT) * 8u * cw_default * elem);
    const uint8_t *src = static_cast<const uint8_t *>(data);
    uint8_t *dst = static_cast<uint8_t *>(out_data);
    hspmm_host::parallel_blocks(W, 1024, [&](size_t wb, size_t we) {
        for (size_t w = wb; w < we; ++w) {
            size_t at = size_t(out_rowOffset[w]) * cw_default;                // next column slot of the window
            for (uint32_t t = rowOffset[w]; t < rowOffset[w + 1]; ++t)
                for (uint32_t k = 0; k < cw; ++k) {
                    const uint32_t id = tcA2B[size_t(t) * cw + k];
                    if (id == HSPMM_IDX_MAX) continue;                        // the real columns keep their order
                    const size_t nt = at / cw_default, nk = at % cw_default;
                    out_tcA2B[at] = id;
                    for (uint32_t r = 0; r < 8u; ++r) {
                        const size_t from = size_t(t) * 8u * cw + (transposed ? size_t(k) * 8u + r : size_t(r) * cw + k);
                        std::memcpy(dst + ((nt * 8u + r) * cw_default + nk) * elem, src + from * elem, elem);
                    }
                    ++at;
                }
        }
    });
    return HSPMM_OK;
}

int hspmm_create_layout(hspmm_plan **out, int dtype, uint32_t col_window, int transposed, uint32_t rows, uint32_t cols,
                        uint32_t eff_row_windows, uint32_t total_tiles, const uint32_t *rowOffset, const uint32_t *tcA2B,
                        const void *data, const uint32_t *rowIdx)
{
    if (!out) return fail(HSPMM_ERR_INVALID, "null plan pointer");
    *out = nullptr;
    uint32_t cw, cw_default, elem;
    if (int rc = layout_widths(dtype, col_window, cw, cw_default, elem)) return rc;
    if (cw == cw_default && !transposed)
        return hspmm_create(out, dtype, rows, cols, eff_row_windows, total_tiles, rowOffset, tcA2B, data, rowIdx);
    const uint32_t W = eff_row_windows;
    if (W && (!rowOffset || !tcA2B || !data || !rowIdx)) return fail(HSPMM_ERR_INVALID, "null format array");
    for (uint32_t w = 0; w < W; ++w)
        if (rowOffset[w + 1] > total_tiles)
            return fail(HSPMM_ERR_INVALID, "rowOffset[%u] = %u beyond total_tiles = %u", w + 1, rowOffset[w + 1], total_tiles);
    if (W && rowOffset[W] != total_tiles)
        return fail(HSPMM_ERR_INVALID, "rowOffset[%u] = %u differs from total_tiles = %u", W, rowOffset[W], total_tiles);
    // the same matrix in the layout hspmm_create reads: tiles of the default width, element (r, k) at r * width + k
    try {
        uint32_t NT = 0;
        if (int rc = hspmm_btcf_relayout_sizes(dtype, col_window, W, rowOffset, tcA2B, &NT)) return rc;
        std::vector<uint32_t> n_rowOffset(size_t(W) + 1), n_ids(size_t(NT) * cw_default);
        std::vector<uint8_t> n_data(size_t(NT) * 8u * cw_default * elem);
        if (int rc = hspmm_btcf_relayout_fill(dtype, col_window, transposed, W, rowOffset, tcA2B, data, n_rowOffset.data(),
                                              n_ids.data(), n_data.data()))
            return rc;
        return hspmm_create(out, dtype, rows, cols, W, NT, n_rowOffset.data(), n_ids.data(), n_data.data(), rowIdx);
    } catch (const std::bad_alloc &) { return fail(HSPMM_ERR_ALLOC, "out of host memory"); }
}

static int create_from_bitmap(hspmm_plan **out, int dtype, uint32_t rows, uint32_t cols, uint32_t eff_row_windows,
                              uint32_t total_tiles, const uint32_t *rowOffset, const uint32_t *nnzOffset,
                              const uint32_t *tcA2B, const uint64_t *tcBit, const void *data, const uint32_t *rowIdx,
                              const GroupCuts *cuts)
{
    if (!out) return fail(HSPMM_ERR_INVALID, "null plan pointer");
    *out = nullptr;
    if (dtype != HSPMM_FP16 && dtype != HSPMM_TF32 && dtype != HSPMM_BF16)
        return fail(HSPMM_ERR_INVALID, "unknown dtype %d", dtype);
    if (total_tiles && (!nnzOffset || !tcBit)) return fail(HSPMM_ERR_INVALID, "null nnzOffset or tcBit");
    // Sparse windows (graphs) never need their tiles on the host: the bitmap arrays go to the device as they are -
    // the gather kernels read them (spmm_mfma_kernel.hpp, Fp16TileDWB and Fp32TileB) - and kernels expand them
    // for the kernels that read plain tiles.  Dense windows (the LDS-panel stream re-tiles them on the host) and
    // paired windows are expanded here first.
    if (eff_row_windows && total_tiles && rowOffset && nnzOffset[0] == 0 && (!nnzOffset[total_tiles] || data)) {
        int mode;
        { std::lock_guard<std::mutex> lk(g_cfg_mutex); mode = g_cfg.kernel_mode; }
        const double density = double(total_tiles) / (double(eff_row_windows) * double((uint64_t(cols) + 127u) / 128u));
        if (mode < 4 && density < 1.2) {
            const BitmapSource src{nnzOffset, tcBit, data};
            const int rc = create_plan(out, dtype, rows, cols, eff_row_windows, total_tiles, rowOffset, tcA2B, nullptr, rowIdx, &src,
                                       cuts);
            if (rc != kNeedsPlainTiles) return rc;
        }
    }
    const size_t tile_bytes = size_t(HSPMM_ROW_WINDOW) * (dtype == HSPMM_TF32 ? 8u * 4u : 16u * 2u);
    std::vector<uint8_t> dense;
    try { dense.resize(size_t(total_tiles) * tile_bytes); }
    catch (const std::bad_alloc &) { return fail(HSPMM_ERR_ALLOC, "out of host memory"); }
    // hspmm_bitmap_expand leaves its own message behind on failure
    const int rc = hspmm_bitmap_expand(dtype, total_tiles, nnzOffset, tcBit, data, dense.data());
    if (rc) return rc;
    return create_plan(out, dtype, rows, cols, eff_row_windows, total_tiles, rowOffset, tcA2B, dense.data(), rowIdx, nullptr, cuts);
}

int hspmm_create_bitmap(hspmm_plan **out, int dtype, uint32_t rows, uint32_t cols, uint32_t eff_row_windows,
                        uint32_t total_tiles, const uint32_t *rowOffset, const uint32_t *nnzOffset,
                        const uint32_t *tcA2B, const uint64_t *tcBit, const void *data, const uint32_t *rowIdx)
{
    return create_from_bitmap(out, dtype, rows, cols, eff_row_windows, total_tiles, rowOffset, nnzOffset, tcA2B, tcBit, data,
                              rowIdx, nullptr);
}

int hspmm_create_grouped(hspmm_plan **out, int dtype, uint32_t rows, uint32_t cols, uint32_t total_groups,
                         const uint32_t *groupOffset, const uint32_t *nnzOffset, const uint32_t *tcA2B,
                         const uint64_t *tcBit, const void *data, const uint32_t *groupRowIdx,
                         const uint8_t *atomic)
{
    if (!out) return fail(HSPMM_ERR_INVALID, "null plan pointer");
    *out = nullptr;
    if (total_groups && (!groupOffset || !groupRowIdx || !atomic))
        return fail(HSPMM_ERR_INVALID, "null groupOffset, rowIdx or atomic");
    // consecutive groups with one row index are one window again
    std::vector<uint32_t> rowOffset(1, total_groups ? groupOffset[0] : 0u), rowIdx;
    for (uint32_t g = 0; g < total_groups; ++g) {
        if (groupOffset[g + 1] <= groupOffset[g])
            return fail(HSPMM_ERR_INVALID, "groupOffset does not increase at group %u", g);
        const bool first = g == 0 || groupRowIdx[g] != groupRowIdx[g - 1];
        const bool last = g + 1 == total_groups || groupRowIdx[g + 1] != groupRowIdx[g];
        const bool shared = !(first && last);
        if ((atomic[g] != 0) != shared)
            return fail(HSPMM_ERR_INVALID, "atomic[%u] = %u but the group %s its rows with a neighbour", g,
                        unsigned(atomic[g]), shared ? "shares" : "does not share");
        if (first) rowIdx.push_back(groupRowIdx[g]);
        if (last) rowOffset.push_back(groupOffset[g + 1]);
    }
    // groups of one window that are not adjacent show up as a row index that does
    // not increase, which the checks of hspmm_create reject
    const uint32_t W = uint32_t(rowIdx.size());
    const GroupCuts cuts{groupOffset, total_groups};
    return create_from_bitmap(out, dtype, rows, cols, W, rowOffset.back(), rowOffset.data(), nnzOffset, tcA2B, tcBit, data,
                              rowIdx.data(), total_groups && groupOffset[0] == 0 ? &cuts : nullptr);
}

void hspmm_destroy(hspmm_plan *p)
{
    if (!p) return;
    (void)hipFree(p->d_rowOffset); (void)hipFree(p->d_rowIdx); (void)hipFree(p->d_a2b_raw);
    if (p->d_tiles != p->d_data) (void)hipFree(p->d_tiles);
    (void)hipFree(p->d_data); (void)hipFree(p->d_unitOffset); (void)hipFree(p->d_unitRow); (void)hipFree(p->d_ids);
    for (auto &dp : p->parts) { (void)hipFree(dp.d_ranges); (void)hipFree(dp.d_split); (void)hipFree(dp.d_fix_slots); }
    (void)hipFree(p->panel.d_poff); (void)hipFree(p->panel.d_ids); (void)hipFree(p->panel.d_tiles);
    (void)hipFree(p->panel.d_unitRow);
    (void)hipFree(p->panel.d_step_panel);
    (void)hipFree(p->panel.d_masks); (void)hipFree(p->panel.d_vals); (void)hipFree(p->panel.d_step_voff);
    (void)hipFree(p->bm.d_header); (void)hipFree(p->bm.d_vals);
    for (auto &b : p->buffers) { (void)hipFree(b.d_scratch); (void)hipFree(b.d_arrive); (void)hipFree(b.d_vector); }
    for (void *old : p->retired) (void)hipFree(old);
    delete p;
}

int hspmm_run(hspmm_plan *p, const void *dB, void *dC, uint32_t N, void *stream)
{
    return run_impl(p, dB, dC, N, stream, nullptr, RunMode::kLaunch);
}

int hspmm_run_static(hspmm_plan *p, const void *dB, void *dC, uint32_t N, void *stream)
{
    return run_impl(p, dB, dC, N, stream, nullptr, RunMode::kStatic);
}

int hspmm_prepare(hspmm_plan *p, uint32_t N)
{
    // B and C at the alignments that select different load widths (and so different partitions and amounts of
    // partial sums; 2: a 16-bit B or C that starts on an odd half); nothing is launched and the pointers are
    // never dereferenced
    if (!p) return fail(HSPMM_ERR_INVALID, "null plan");
    for (uintptr_t align : {uintptr_t(16), uintptr_t(8), uintptr_t(4), uintptr_t(2)}) {
        if (align < p->elem) continue;
        const int rc = run_impl(p, reinterpret_cast<const void *>(align), reinterpret_cast<void *>(align), N, nullptr,
                                nullptr, RunMode::kPrepare);
        if (rc) return rc;
    }
    return HSPMM_OK;
}

}  // extern "C"

// ---------------------------------------------------------------------------
// A launch in three steps: choose (a function of the plan, N and the pointers' alignment alone: kernel
// family, load layout, launch shape), acquire (what the choice needs beyond the plan's fixed arrays - a work
// partition, partial sums, arrival counters - under the plan's mutex), launch.  hspmm_prepare stops after the
// second step; hspmm_run_static fails in the second when something would have to be built.
// ---------------------------------------------------------------------------

// Shape of a launch of the LDS-panel kernels: grid = row blocks x feature blocks x chunks of panels.
struct PanelShape {
    int units = 0;                      // workgroup shape code (launch_spmm_panel)
    uint32_t units_per_group = 0;       // consumer waves of a workgroup that get a unit
    uint32_t n_feat_blocks = 0, n_chunks = 0, panels_per_chunk = 0;
    size_t acc_per_unit = 0;            // accumulator registers (of four floats per lane) a unit's chunk sums take
    uint32_t mfma_kind = 0;
    uint64_t mfma_count = 0;
};

static int choose_panel_shape(const hspmm_plan *p, uint32_t N, PanelShape *out)
{
    const hspmm_plan::Panel &pl = p->panel;
    PanelShape sh;
    const uint32_t block = hspmm::kPanelRowBytes / p->elem;
    sh.n_feat_blocks = (N + block - 1u) / block;                   // (the last block may end inside: panel_serves says when)
    // The workgroup shape: code 14 / 12 = that many consumer waves and two producers, 13 = 12 consumers and
    // four producers (few enough registers for two workgroups per compute unit, which the 4x4x1 fp32 kernel
    // needs to keep its short MFMAs fed).  Of the consumer waves any number may be given a unit.
    const bool wide = p->dtype != HSPMM_TF32 || pl.split;          // panels of 256 rows: always 12 + 4 waves
    int units = (pl.quad || wide) ? 13 : pl.G == 2 ? 14 : 12;
    int forced_units = 0;
    if (p->cfg.panel_units) {                                                                    // tuning overrides
        units = p->cfg.panel_units;
        forced_units = units == 13 ? 12 : units;
        if (wide) { units = 13; forced_units = std::min(forced_units, 12); }
    }
    if (p->cfg.panel_units_per_group)          // fewer units than the shape has consumer waves
        forced_units = std::min(p->cfg.panel_units_per_group, units == 13 ? 12 : units);
    // (units of up to four windows: eight consumer waves with twice the accumulators)
    // (two 16-bit units per wave: eight larger consumer waves as well)
    const int max_units = (pl.G == 4 || (pl.tall && p->dtype != HSPMM_TF32)) ? 8 : units == 13 ? 12 : units;
    // what one consumer wave takes: a unit, or (tall streams) two
    const uint32_t wave_units = pl.tall ? (pl.n_units + 1u) / 2u : pl.n_units;
    if (forced_units) forced_units = std::min(forced_units, max_units);
    const uint64_t slots = uint64_t(p->compute_units) * (pl.quad ? 2u : 1u);     // workgroups resident at a time
    // Units per workgroup and chunks of panels: the workgroups should fill the compute units in whole
    // rounds.  Cost of a shape = rounds x panels per chunk x (units + 3: a panel costs its LDS reads and
    // MFMAs, which go with the units, plus its copy and barrier), plus what chunk sums cost.
    uint64_t chunks = 1;
    int best_units = max_units;
    double best_cost = 0.0;
    for (int nc = forced_units ? forced_units : std::max(4, max_units / 2); nc <= (forced_units ? forced_units : max_units); ++nc) {
        const uint64_t rbs = (uint64_t(wave_units) + nc - 1) / nc, base = rbs * sh.n_feat_blocks;
        uint64_t ch = base >= slots ? 1 : std::min<uint64_t>(slots / base, pl.n_panels);
        const uint64_t ppc = (pl.n_panels + ch - 1) / ch;
        ch = (pl.n_panels + ppc - 1) / ppc;
        const uint64_t rounds = (base * ch + slots - 1) / slots;
        // (streams with two units per wave: the same in 128-byte lines - per panel its copy and every unit's
        // tiles and ids - which is what those streams were measured with)
        const double cost = pl.tall ? double(rounds) * double(ppc) * (512.0 + 2.0 * double(nc) * pl.unit_lines) +
                                          (ch > 1 ? 2500.0 + 300.0 * double(ch) : 0.0)
                                    : double(rounds) * double(ppc) * (double(nc) + 3.0) + (ch > 1 ? 80.0 : 0.0);
        if (best_cost == 0.0 || cost < best_cost) { best_cost = cost; best_units = nc; chunks = ch; }
    }
    sh.units = units;
    sh.units_per_group = uint32_t(best_units);
    const uint64_t row_blocks = (uint64_t(wave_units) + best_units - 1) / best_units;
    const uint64_t base = row_blocks * sh.n_feat_blocks;
    if (p->cfg.panel_chunks) chunks = uint64_t(p->cfg.panel_chunks);
    if (chunks < 1) chunks = 1;
    if (chunks > pl.n_panels) chunks = pl.n_panels;
    sh.panels_per_chunk = uint32_t((pl.n_panels + chunks - 1) / chunks);
    sh.n_chunks = (pl.n_panels + sh.panels_per_chunk - 1) / sh.panels_per_chunk;
    if (base * sh.n_chunks > 0x7FFFFFFFull)
        return fail(HSPMM_ERR_UNSUPPORTED, "feature dimension %u needs too many workgroups", N);
    if (uint64_t(pl.n_units) * sh.n_chunks > 0xFFFFFFFFull)
        return fail(HSPMM_ERR_UNSUPPORTED, "feature dimension %u needs too many partial sums", N);
    const size_t wide_rows = pl.G == 4 ? 2u : 1u;
    sh.acc_per_unit = pl.quad ? 2u : pl.split ? 4u * wide_rows : p->dtype != HSPMM_TF32 ? 8u * wide_rows : 4u * size_t(pl.G);
    // matrix instructions per step and feature block (PanelOps<...>::mma_half in spmm_panel_kernel.hpp)
    sh.mfma_kind = pl.quad ? 4u : (p->dtype == HSPMM_TF32 && !pl.split) ? 3u : (p->dtype == HSPMM_FP16 ? 1u : 2u);
    const uint64_t per_step = pl.quad ? 16u : pl.split ? 12u * wide_rows : p->dtype != HSPMM_TF32 ? 8u * wide_rows : 8u * uint64_t(pl.G);
    sh.mfma_count = uint64_t(pl.n_steps) * sh.n_feat_blocks * per_step;
    *out = sh;
    return HSPMM_OK;
}

// Launch through the LDS-panel kernels.  The launch shape is a function of the plan and N alone.
static int run_panel(hspmm_plan *p, const void *dB, void *dC, uint32_t N, hipStream_t s, hipEvent_t mid, RunMode mode)
{
    PanelShape sh;
    if (int rc = choose_panel_shape(p, N, &sh)) return rc;
    const hspmm_plan::Panel &pl = p->panel;
    hspmm::PanelArgs pa{};
    pa.unitRow = pl.d_unitRow; pa.poff = pl.d_poff; pa.step_panel = pl.d_step_panel; pa.ids = pl.d_ids;
    pa.tiles = pl.d_tiles; pa.n_steps = pl.n_steps;
    pa.masks = pl.d_masks; pa.vals = pl.d_vals; pa.step_voff = pl.d_step_voff;
    pa.B = dB; pa.C = dC;
    pa.n_units = pl.n_units; pa.rows = p->rows; pa.cols = p->cols; pa.N = N;
    pa.n_feat_blocks = sh.n_feat_blocks; pa.n_panels = pl.n_panels;
    pa.units_per_group = sh.units_per_group; pa.n_chunks = sh.n_chunks; pa.panels_per_chunk = sh.panels_per_chunk;
    hspmm::KernelArgs ka{};
    if (sh.n_chunks > 1) {
        // acquire: the chunk sums and, where the last wave to arrive adds them, the arrival counters
        const size_t need = size_t(pl.n_units) * sh.n_chunks * sh.n_feat_blocks * sh.acc_per_unit * 64u * 16u;
        {
            std::lock_guard<std::mutex> lk(p->mu);
            int rc = scratch_for(p, s, need, mode, &pa.scratch);
            if (rc) return rc;
            // As in the gather kernels, the wave that brings a unit's last chunk adds the chunk sums itself
            // (16-byte device-scope accesses; block-clustered configuration at N = 512: 56.0 + 8.1 us in two
            // launches, 60.3 us in one).  It addresses a unit's chunk sums with 32-bit offsets.
            if (p->cfg.fused_fixup != 0 && mode != RunMode::kStatic &&
                uint64_t(sh.n_chunks) * sh.n_feat_blocks * sh.acc_per_unit * 1024u < (1ull << 31) &&
                (rc = ensure_arrive(p, s, size_t(pl.n_units) * sh.n_feat_blocks, mode, &pa.arrive)))
                return rc;
        }
        // the chunk sums of unit u are slots u * chunks .. + chunks - 1: no table
        ka.unitRow = pl.d_unitRow; ka.ids = pl.d_ids; ka.tiles = pl.d_tiles;
        ka.scratch = pa.scratch;
        ka.C = dC; ka.B = dB;
        ka.n_split = pl.n_units; ka.n_units = pl.n_units; ka.rows = p->rows; ka.N = N; ka.ld = N;
        ka.n_feat_blocks = sh.n_feat_blocks;
        ka.uniform_chunks = sh.n_chunks;
    }
    if (mode == RunMode::kPrepare) return HSPMM_OK;
    p->note_launch(3, sh.mfma_kind, sh.mfma_count);
    HSPMM_HIP(hspmm::launch_spmm_panel(p->dtype, pl.quad ? 0 : pl.G, pl.split, pl.tall, pl.packed, pa, ka, sh.units, s, mid));
    return HSPMM_OK;
}

// Whether the LDS-panel kernels serve feature dimension N (a workgroup covers 256 bytes of every B row with
// 16-byte accesses).
static bool panel_serves(const hspmm_plan *p, uint32_t N)
{
    if (!p->panel.built || !(p->cfg.kernel_mode == 0 || p->cfg.kernel_mode >= 4)) return false;
    const uint32_t block_feat = hspmm::kPanelRowBytes / p->elem;
    // (a 16-bit matrix near the break-even is served as fast or faster by the gather kernels while
    // one wave of theirs covers all of N)
    const bool pays = p->cfg.kernel_mode >= 4 || p->cw != 16 || p->panel.density >= 2.2 || N >= 256u;
    // (the producers address a panel of B - up to 256 rows - with 32-bit offsets)
    const bool offsets_fit = uint64_t(N) * p->elem < (uint64_t(1) << 24);
    // Whole blocks of features; or any N of one block at least - the last block then moves back to end with
    // the row (panel_block_first_feature in spmm_mfma_kernel.hpp) -; or, fp32 storage in bf16 parts, whose
    // gather kernels multiply at a sixteenth of the rate, one partly empty block from 16 features on when the
    // rows are whole 16-byte pieces (the lanes of that kernel own one feature per accumulator: what the block
    // lacks is read from the row's first piece and not stored).
    const bool ragged_ok = N >= block_feat || (p->panel.split && (uint64_t(N) * p->elem) % 16u == 0 && N >= 16u);
    // (B and C wherever they start: the producers' 16-byte loads need no alignment, C is stored element by element)
    return pays && offsets_fit && (N % block_feat == 0 || ragged_ok);
}

static int run_gather(hspmm_plan *p, const void *dB, void *dC, uint32_t N, uint32_t ld, hipStream_t s, hipEvent_t mid, RunMode mode);

// One launch (or, kPrepare, everything a launch with this N and these pointer alignments would build): which
// kernel family serves N, and in how many pieces.
// mid: when not null, an event recorded between the main kernel and the kernel that adds the partial
// sums of split windows.
static int run_impl(hspmm_plan *p, const void *dB, void *dC, uint32_t N, void *stream, hipEvent_t mid, RunMode mode)
{
    if (!p) return fail(HSPMM_ERR_INVALID, "null plan");
    if (N == 0) return fail(HSPMM_ERR_INVALID, "feature dimension N = 0");
    if (p->rows == 0) return HSPMM_OK;
    if (!dC) return fail(HSPMM_ERR_INVALID, "null C");
    if (!dB && p->W) return fail(HSPMM_ERR_INVALID, "null B");
    if (reinterpret_cast<uintptr_t>(dC) % p->elem || reinterpret_cast<uintptr_t>(dB) % p->elem)
        return fail(HSPMM_ERR_INVALID, "B and C must be aligned to the element size");
    {
        // the plan's arrays live on the device that was current in hspmm_create
        int dev = -1;
        HSPMM_HIP(hipGetDevice(&dev));
        if (dev != p->device)
            return fail(HSPMM_ERR_INVALID, "the plan was created on device %d, the current device is %d", p->device, dev);
    }
    const bool launch = mode != RunMode::kPrepare;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (p->W == 0) {
        if (!launch) return HSPMM_OK;
        p->note_launch(4, 0, 0);
        HSPMM_HIP(hspmm::launch_fill_zero(dC, size_t(p->rows) * N * p->elem, s));
        return HSPMM_OK;
    }
    if (panel_serves(p, N)) return run_panel(p, dB, dC, N, s, mid, mode);
    // A feature dimension that no wide load divides (16-bit types: N not a multiple of 8, fp32 storage: of 4) would
    // run in blocks of 32 resp. 16 features, each block a pass over the tiles and another gather of every row
    // (power-law graph 2^20, fp16: N = 130 in five passes, 1404 us against 481 us at N = 128).  Two launches
    // instead: the features up to the last multiple with the wide loads, the few behind it in one narrow block.
    // (An odd N of a 16-bit type: the narrow block gets nine features rather than one, its last lane reads one half
    // in front of its feature.)
    // (Cutting at the last multiple of 64 as well, so that those features run with word loads and bitmap tiles,
    // measured 1027 -> 895 us at N = 136 and 1175 -> 1259 us at N = 200: not done.)
    // A single feature of a 16-bit type (matrix times vector): B and C widened to words - the element and a zero -
    // in a buffer of the plan's, two features through the MFMA kernels, the low halves back (power-law graph 2^20:
    // 21 ms on the all-shapes kernel).  hspmm_run_static, which allocates nothing, wants the buffer made already.
    if (p->elem == 2u && N == 1u && p->cfg.kernel_mode != 1) {
        uint32_t *b2 = nullptr;
        {
            std::lock_guard<std::mutex> lk(p->mu);
            if (mode == RunMode::kStatic) {
                hspmm_plan::StreamBuffers *b = buffers_for(p, s, false);
                if (!b || !b->d_vector)
                    return fail(HSPMM_ERR_UNSUPPORTED, "hspmm_run_static: a single feature of a 16-bit type goes through a buffer "
                                "of the plan's that does not exist yet (call hspmm_prepare(plan, 1) or hspmm_run with N = 1 first)");
                b2 = b->d_vector;
            } else {
                for (hspmm_plan::StreamBuffers *b : sets_for(p, s, mode)) {
                    if (!b->d_vector) {
                        HSPMM_HIP(hipMalloc(reinterpret_cast<void **>(&b->d_vector), (size_t(p->cols) + p->rows) * 4u));
                        p->fixed_bytes += (size_t(p->cols) + p->rows) * 4u;
                    }
                    b2 = b->d_vector;
                }
            }
        }
        uint32_t *c2 = b2 + p->cols;
        if (launch) HSPMM_HIP(hspmm::launch_widen_halves(dB, b2, p->cols, s));
        const int rc = run_gather(p, b2, c2, 2u, 2u, s, mid, mode);
        if (rc) return rc;
        if (launch) HSPMM_HIP(hspmm::launch_narrow_words(c2, dC, p->rows, s));
        return HSPMM_OK;
    }
    const uint32_t wide = p->elem == 2u ? 8u : 4u;
    const uintptr_t align = reinterpret_cast<uintptr_t>(dB) | reinterpret_cast<uintptr_t>(dC);
    // (not where one block of the narrower loads covers all of N anyway)
    bool one_block = false;
    if (p->cfg.kernel_mode != 1) {
        const Choice whole = choose_kernel(p, dB, dC, N, N);
        one_block = !whole.scalar && N <= uint32_t(whole.block_feat);
    }
    if (p->cfg.kernel_mode != 1 && !one_block && N > wide && N % wide != 0 && !(align & 3u)) {
        const uint32_t first = N - N % wide - ((p->elem == 2u && N % wide == 1u) ? wide : 0u);
        const int rc = run_gather(p, dB, dC, first, N, s, mid, mode);
        if (rc) return rc;
        return run_gather(p, static_cast<const char *>(dB) + size_t(first) * p->elem, static_cast<char *>(dC) + size_t(first) * p->elem,
                          N - first, N, s, nullptr, mode);
    }
    return run_gather(p, dB, dC, N, N, s, mid, mode);
}

// What a launch of the gather kernels (or of the all-shapes kernel) over N features looks like: a function of the
// plan, N, the row pitch and the alignment of B and C.
struct GatherShape {
    Choice c{};
    int layout = 0;                     // c.layout, or the bitmap form of it
    uint32_t n_feat_blocks = 0, xcd_split = 0;
    int level = 0;                      // which partition: fewer, longer ranges for more feature blocks
    int wpg = 0;                        // waves per workgroup
    bool combine = false;               // the waves of a workgroup add the sums of one unit among themselves
    bool aligned = false;               // every unit is cut into the ranges of one workgroup, which stores it
    int prefetch = 0;
    int partition_index() const { return aligned ? 4 : combine ? 3 : level; }
};

static GatherShape choose_gather_shape(const hspmm_plan *p, const void *dB, const void *dC, uint32_t N, uint32_t ld)
{
    GatherShape g;
    // Feature blocks with XCDs of their own (see spmm_mfma_kernel): pays when B is far larger than an
    // XCD's 4 MB L2, so that what an L2 can keep of it decides the hit rate of the gathers (power-law
    // graph 2^20, N = 128: 575 -> 535 us; uniform 65536^2: 39.7 -> 35.5 us), and costs a second pass over
    // the tile stream.  Requests below a 128-byte line lose (N = 64 as two blocks of 32: 280 -> 510 us).
    const bool want_split = p->cfg.xcd_split > 0 ||
                             (p->cfg.xcd_split < 0 && uint64_t(p->cols) * N * p->elem >= (uint64_t(8) << 20));
    g.c = choose_kernel(p, dB, dC, N, ld, want_split);
    if (g.c.scalar) return g;
    const Choice &c = g.c;
    g.layout = c.layout;
    if (p->bm.built && (p->cfg.kernel_mode == 0 || p->cfg.kernel_mode == 3) &&
        (p->dtype == HSPMM_TF32 || (c.layout == hspmm::kLayoutDW && (c.V == 2 || c.V == 4))))
        g.layout = hspmm::kLayoutDWB;                 // tiles as bitmap + stored elements
    g.n_feat_blocks = (N + uint32_t(c.block_feat) - 1u) / uint32_t(c.block_feat);
    g.xcd_split = (want_split && (g.n_feat_blocks == 2u || g.n_feat_blocks == 4u || g.n_feat_blocks == 8u)) ? 1u : 0u;
    // Several feature blocks give several waves per range; fewer, longer ranges then keep
    // the number of waves, and pay off where units are long enough to be cut into many
    // pieces (each piece of a cut unit costs a partial sum).
    const double steps_per_unit = double(p->n_steps) / double(p->n_units);
    const double steps_per_range = double(p->n_steps) / double(p->parts[0].part.ranges.size());
    if (steps_per_unit >= 8.0 * steps_per_range) g.level = g.n_feat_blocks >= 4 ? 2 : g.n_feat_blocks >= 2 ? 1 : 0;
    // One feature block: the waves of a workgroup walk consecutive ranges and add the partial sums of
    // one unit among themselves.
    g.wpg = p->cfg.consumer_warp_num > 0 ? p->cfg.consumer_warp_num : hspmm::kMaxWavesPerGroup;
    g.combine = g.level == 0 && g.n_feat_blocks == 1 && g.wpg > 1 && p->cfg.fused_fixup <= 0;
    // Units that are all long (block-clustered, pruned or dense-ish random matrices at a small N): every
    // unit is cut into the ranges of one workgroup of four or eight waves, which stores it itself - no
    // partial sums leave the chip and there is no second launch (block-clustered 4096 x 14336, N = 16:
    // 18.9 + 6.4 us -> 19 us; random 8192 x 8192 at 2 %, N = 128: 26.8 + 7.1 -> 22.8 us).  With the default
    // knobs only: the eight-wave kernels exist for the default depth.
    g.aligned = g.combine && p->aligned_group && c.narrow && p->cfg.consumer_warp_num == 0 &&
                (p->cfg.buffer_stage == 0 || p->aligned_group == hspmm::kMaxWavesPerGroup) &&
                p->cfg.producer_warp_group_num == 0;
    if (g.aligned) g.wpg = p->aligned_group;
    const int default_depth = hspmm::default_prefetch(int(p->elem), p->G, c.V);
    g.prefetch = p->cfg.buffer_stage > 0 ? p->cfg.buffer_stage : default_depth;
#ifndef HSPMM_EXPERIMENTAL
    if (!c.narrow) g.prefetch = default_depth;    // (64-bit gather offsets are built for the default depth only)
#endif
    return g;
}

// One launch of the gather kernels (or of the all-shapes kernel) over N features of rows that are ld elements apart.
static int run_gather(hspmm_plan *p, const void *dB, void *dC, uint32_t N, uint32_t ld, hipStream_t s, hipEvent_t mid, RunMode mode)
{
    const bool launch = mode != RunMode::kPrepare;
    const GatherShape g = choose_gather_shape(p, dB, dC, N, ld);
    const Choice &c = g.c;
    hspmm::KernelArgs ka{};
    ka.rowOffset = p->d_rowOffset; ka.data = p->d_data; ka.rowIdx = p->d_rowIdx; ka.tcA2B = p->d_a2b_raw;
    ka.B = dB; ka.C = dC;
    ka.eff_windows = p->W; ka.rows = p->rows; ka.N = N; ka.ld = ld;
    if (c.scalar) {
        if (ld != N) return fail(HSPMM_ERR_UNSUPPORTED, "the all-shapes kernel takes whole rows");
        if (!launch) return HSPMM_OK;
        p->note_launch(1, 0, 0);
        HSPMM_HIP(hspmm::launch_spmm_scalar(p->dtype, ka, s));
        return HSPMM_OK;
    }
    ka.unitOffset = p->d_unitOffset; ka.unitRow = p->d_unitRow; ka.ids = p->d_ids; ka.tiles = p->d_tiles;
    if (g.layout == hspmm::kLayoutDWB) { ka.tiles = p->bm.d_vals; ka.bm_header = p->bm.d_header; }
    ka.n_units = p->n_units;
    ka.n_feat_blocks = g.n_feat_blocks;
    ka.xcd_split = g.xcd_split;
    // acquire: the partition this shape walks, the partial sums of its cut units, their arrival counters
    hspmm_plan::DevPartition &dp = p->parts[g.partition_index()];
    {
        std::lock_guard<std::mutex> lk(p->mu);
        if (!dp.built) {
            if (mode == RunMode::kStatic)
                return fail(HSPMM_ERR_UNSUPPORTED,
                            "hspmm_run_static: the work partition for N = %u is not built yet; call hspmm_prepare(plan, N) "
                            "or hspmm_run once with this N first", N);
            const int rc = build_and_upload_partition(p, g.level, g.combine ? uint32_t(g.wpg) : 1u, g.aligned);
            if (rc) return rc;
        }
        ka.n_ranges = uint32_t(dp.part.ranges.size());
        ka.n_split = uint32_t(dp.part.split.size());
        // The wave that brings a cut unit's last partial sum adds them itself (in range order, as the second
        // kernel would): worth it where few units are cut and the second launch is most of what they cost
        // (power-law graph, 382 of 110 746 units: 540.6 + 9.4 -> 541.1 us); where every unit is cut the
        // device-scope traffic costs more than the launch (block-clustered: 30 -> 129 us).
        const bool fused = mode != RunMode::kStatic && !g.combine &&
                           (p->cfg.fused_fixup > 0 || (p->cfg.fused_fixup < 0 && ka.n_split && uint64_t(ka.n_split) * 32u <= p->n_units));
        if (uint64_t(ka.n_ranges) * ka.n_feat_blocks > 0x7FFFFFFFull)
            return fail(HSPMM_ERR_UNSUPPORTED, "feature dimension %u needs too many work items", N);
        const size_t need = size_t(dp.part.n_slots) * ka.n_feat_blocks * size_t(c.V) * size_t(p->G) * 64u * 16u;
        int rc = scratch_for(p, s, need, mode, &ka.scratch);
        if (rc) return rc;
        if (fused && ka.n_split && (rc = ensure_arrive(p, s, size_t(ka.n_split) * ka.n_feat_blocks, mode, &ka.arrive))) return rc;
    }
    ka.ranges = dp.d_ranges; ka.split = dp.d_split; ka.fix_slots = dp.d_fix_slots;
    if (!launch) return HSPMM_OK;
    // (per step and feature block: G * V instructions of 16 x 16 x 32, or 2 G V of 16 x 16 x 4 for 32-bit elements)
    p->note_launch(2, p->dtype == HSPMM_TF32 ? 3u : p->dtype == HSPMM_FP16 ? 1u : 2u,
                   uint64_t(p->n_steps) * ka.n_feat_blocks * uint64_t(p->G) * uint64_t(c.V) * (p->dtype == HSPMM_TF32 ? 2u : 1u));
    HSPMM_HIP(hspmm::launch_spmm_mfma(p->dtype, g.layout, p->G, ka, c.V, g.prefetch, c.narrow, g.wpg, s, mid));
    return HSPMM_OK;
}

extern "C" {

int hspmm_profile(hspmm_plan *p, const void *dB, void *dC, uint32_t N, int runs, void *stream,
                  float *main_ms, float *fixup_ms)
{
    if (!main_ms || !fixup_ms) return fail(HSPMM_ERR_INVALID, "null output");
    if (runs < 1 || runs > 1000) return fail(HSPMM_ERR_INVALID, "runs %d outside 1..1000", runs);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the events are destroyed on every way out
    struct Events {
        std::vector<hipEvent_t> ev;
        ~Events() { for (hipEvent_t e : ev) (void)hipEventDestroy(e); }
    } events;
    events.ev.reserve(size_t(runs) * 3);
    for (int i = 0; i < runs * 3; ++i) {
        hipEvent_t e;
        HSPMM_HIP(hipEventCreate(&e));
        events.ev.push_back(e);
    }
    const std::vector<hipEvent_t> &ev = events.ev;
    for (int i = 0; i < runs; ++i) {
        HSPMM_HIP(hipEventRecord(ev[3 * i], s));
        const int rc = run_impl(p, dB, dC, N, stream, ev[3 * i + 1], RunMode::kLaunch);
        if (rc) return rc;
        HSPMM_HIP(hipEventRecord(ev[3 * i + 2], s));
    }
    HSPMM_HIP(hipStreamSynchronize(s));
    *main_ms = 0.f; *fixup_ms = 0.f;
    for (int i = 0; i < runs; ++i) {
        float a = 0.f, b = 0.f;
        if (hipEventQuery(ev[3 * i + 1]) == hipSuccess && hipEventElapsedTime(&a, ev[3 * i], ev[3 * i + 1]) == hipSuccess) {
            HSPMM_HIP(hipEventElapsedTime(&b, ev[3 * i + 1], ev[3 * i + 2]));
        } else {                          // no split windows (or scalar kernel): one kernel only
            (void)hipGetLastError();
            HSPMM_HIP(hipEventElapsedTime(&a, ev[3 * i], ev[3 * i + 2]));
        }
        *main_ms += a; *fixup_ms += b;
    }
    return HSPMM_OK;
}

int hspmm_bench(hspmm_plan *p, const void *dB, void *dC, uint32_t N, int warmup, int runs, void *stream,
                float *total_ms)
{
    if (!total_ms) return fail(HSPMM_ERR_INVALID, "null total_ms");
    if (warmup < 0 || runs < 1) return fail(HSPMM_ERR_INVALID, "warmup %d / runs %d", warmup, runs);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc;
    for (int i = 0; i < warmup; ++i)
        if ((rc = hspmm_run(p, dB, dC, N, stream))) return rc;
    struct Pair {
        hipEvent_t a = nullptr, b = nullptr;
        ~Pair() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
    } ev;
    HSPMM_HIP(hipEventCreate(&ev.a));
    HSPMM_HIP(hipEventCreate(&ev.b));
    HSPMM_HIP(hipEventRecord(ev.a, s));
    for (int i = 0; i < runs; ++i)
        if ((rc = hspmm_run(p, dB, dC, N, stream))) return rc;
    HSPMM_HIP(hipEventRecord(ev.b, s));
    HSPMM_HIP(hipEventSynchronize(ev.b));
    HSPMM_HIP(hipEventElapsedTime(total_ms, ev.a, ev.b));
    return HSPMM_OK;
}

int hspmm_measure_gather(hspmm_plan *p, const void *dB, uint32_t N, int runs, void *stream, float *ms,
                         uint64_t *bytes_per_run)
{
    if (!p || !dB || !ms) return fail(HSPMM_ERR_INVALID, "null argument");
    if (runs < 1 || runs > 1000) return fail(HSPMM_ERR_INVALID, "runs %d outside 1..1000", runs);
    if (p->W == 0) return fail(HSPMM_ERR_INVALID, "the matrix has no stored entries");
    const uint64_t row_bytes = uint64_t(N) * p->elem;
    if (row_bytes % 128u || row_bytes > (1u << 24) || reinterpret_cast<uintptr_t>(dB) % 16u)
        return fail(HSPMM_ERR_UNSUPPORTED, "rows of %llu bytes: a multiple of 128 bytes and a B aligned to 16 is needed",
                    (unsigned long long)row_bytes);
    int dev = -1;
    HSPMM_HIP(hipGetDevice(&dev));
    if (dev != p->device) return fail(HSPMM_ERR_INVALID, "the plan was created on device %d, the current device is %d", p->device, dev);
    // the parts the gather kernels would read the rows in: one 128-byte line per XCD group where they deal
    // feature blocks out by XCD (same rule as run_impl), else 256 bytes at a time
    const bool split = p->cfg.xcd_split > 0 ||
                       (p->cfg.xcd_split < 0 && uint64_t(p->cols) * row_bytes >= (uint64_t(8) << 20));
    uint32_t part_bytes = 256u, parts = 1u, passes = uint32_t(row_bytes / 256u);
    if (row_bytes % 256u) { part_bytes = 128u; passes = uint32_t(row_bytes / 128u); }
    if (split && (row_bytes == 256u || row_bytes == 512u || row_bytes == 1024u)) {
        part_bytes = 128u; parts = uint32_t(row_bytes / 128u); passes = 1u;
    }
    const uint64_t n_ids = uint64_t(p->n_steps) * p->cw;
    hipStream_t s = static_cast<hipStream_t>(stream);
    struct Pair {
        hipEvent_t a = nullptr, b = nullptr;
        ~Pair() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
    } ev;
    HSPMM_HIP(hipEventCreate(&ev.a));
    HSPMM_HIP(hipEventCreate(&ev.b));
    for (int i = -1; i < runs; ++i) {                      // one untimed run first
        if (i == 0) HSPMM_HIP(hipEventRecord(ev.a, s));
        for (uint32_t pass = 0; pass < passes; ++pass)
            HSPMM_HIP(hspmm::launch_gather_rate(p->d_ids, n_ids, static_cast<const char *>(dB) + size_t(pass) * part_bytes,
                                                uint32_t(row_bytes), part_bytes, parts, p->compute_units, nullptr, s));
    }
    HSPMM_HIP(hipEventRecord(ev.b, s));
    HSPMM_HIP(hipEventSynchronize(ev.b));
    HSPMM_HIP(hipEventElapsedTime(ms, ev.a, ev.b));
    *ms /= float(runs);
    if (bytes_per_run) *bytes_per_run = n_ids * row_bytes;
    return HSPMM_OK;
}

int hspmm_get_plan_info(const hspmm_plan *p, hspmm_plan_info *info)
{
    if (!p || !info) return fail(HSPMM_ERR_INVALID, "null argument");
    info->rows = p->rows; info->cols = p->cols; info->eff_row_windows = p->W; info->total_tiles = p->T;
    info->dtype = p->dtype;
    info->n_ranges = uint32_t(p->parts[0].part.ranges.size());
    info->n_split_windows = uint32_t(p->parts[0].part.split.size());
    info->n_partial_slots = p->parts[0].part.n_slots;
    info->compute_units = uint32_t(p->compute_units);
    info->n_units = p->n_units;
    info->n_paired_units = p->n_paired;
    {
        // everything the plan holds on the device: its arrays, the buffers of every stream, superseded buffers
        std::lock_guard<std::mutex> lk(const_cast<hspmm_plan *>(p)->mu);
        info->device_bytes = uint64_t(p->fixed_bytes) + uint64_t(p->retired_bytes);
        for (const auto &b : p->buffers) info->device_bytes += uint64_t(b.scratch_bytes);
    }
    info->n_panels = p->panel.built ? p->panel.n_panels : 0u;
    info->n_panel_steps = p->panel.built ? p->panel.n_steps : 0u;
    info->n_panel_units = p->panel.built ? p->panel.n_units : 0u;
    info->n_panel_paired_units = p->panel.built ? p->panel.n_paired : 0u;
    info->n_panel_wide_units = p->panel.built ? p->panel.n_wide : 0u;
    info->last_kernel_family = p->last_family.load(std::memory_order_relaxed);
    info->last_mfma_kind = p->last_mfma_kind.load(std::memory_order_relaxed);
    static const uint32_t kMfmaFlops[5] = {0u, 16384u, 16384u, 2048u, 512u};
    info->last_mfma_flops = kMfmaFlops[info->last_mfma_kind];
    info->last_mfma_instructions = p->last_mfma_count.load(std::memory_order_relaxed);
    info->gather_bitmap = p->bm.built ? 1u : 0u;
    info->bitmap_from_caller = p->bm.from_caller ? 1u : 0u;
    info->group_cuts_kept = p->caller_cuts.empty() ? 0u : 1u;
    info->panel_stream_mode = !p->panel.built ? 0u : p->panel.packed ? 2u : p->panel.tall ? 1u : 0u;
    return HSPMM_OK;
}

int hspmm_get_partition(const hspmm_plan *p, uint32_t *ranges, uint32_t capacity_ranges)
{
    if (!p || !ranges) return fail(HSPMM_ERR_INVALID, "null argument");
    const size_t n = p->parts[0].part.ranges.size() < capacity_ranges ? p->parts[0].part.ranges.size() : capacity_ranges;
    for (size_t i = 0; i < n; ++i) {
        ranges[5 * i + 0] = p->parts[0].part.ranges[i].tile_begin; ranges[5 * i + 1] = p->parts[0].part.ranges[i].tile_end;
        ranges[5 * i + 2] = p->parts[0].part.ranges[i].first_window;
        ranges[5 * i + 3] = p->parts[0].part.ranges[i].head_slot; ranges[5 * i + 4] = p->parts[0].part.ranges[i].tail_slot;
    }
    return HSPMM_OK;
}

int hspmm_partition_as_groups(const hspmm_plan *p, uint32_t capacity_groups, uint32_t *total_groups, uint32_t *groupOffset,
                              uint32_t *groupRowIdx, uint8_t *atomic)
{
    if (!p || !total_groups) return fail(HSPMM_ERR_INVALID, "null argument");
    // A plan that walks pairs of windows has steps the caller never had: the groups then come from the balanced
    // partition of the caller's single windows, built here with the plan's cost model.
    hspmm::Partition own;
    if (p->W && p->G != 1) {
        const uint64_t waves = uint64_t(p->compute_units) * 4u * uint64_t(p->cfg.producer_warp_group_num > 0 ? p->cfg.producer_warp_group_num : 4);
        const uint64_t cap = (uint64_t(p->T) + kMinTilesPerRange - 1) / kMinTilesPerRange;
        const uint32_t target = uint32_t(std::max<uint64_t>(1, std::min(waves, cap)));
        try {
            own = hspmm::build_partition(p->W, p->h_winOffset.data(), target, kWindowCost, kSlack, kWholeWindowMargin, 1, nullptr);
        } catch (const std::bad_alloc &) { return fail(HSPMM_ERR_ALLOC, "out of host memory"); }
    }
    const bool merged = p->W && p->G != 1;
    const std::vector<hspmm::Range> &ranges = merged ? own.ranges : p->parts[0].part.ranges;
    const std::vector<uint32_t> &first_tile = merged ? p->h_winOffset : p->h_unitOffset;     // single windows: a step is a tile
    const std::vector<uint32_t> &first_row = merged ? p->h_winRow : p->h_unitRow;
    const bool write = groupOffset && groupRowIdx && atomic;
    uint32_t n = 0;
    for (const hspmm::Range &r : ranges) {
        uint32_t w = r.first_window;
        for (uint32_t t = r.tile_begin; t < r.tile_end; ++w) {
            const uint32_t end = std::min(r.tile_end, first_tile[w + 1]);
            if (write && n < capacity_groups) {
                groupOffset[n] = t;
                groupRowIdx[n] = first_row[w] & ~7u;
                atomic[n] = (t > first_tile[w] || end < first_tile[w + 1]) ? 1 : 0;     // the window continues in another group
            }
            ++n;
            t = end;
        }
    }
    if (write && n <= capacity_groups) groupOffset[n] = p->T;
    *total_groups = n;
    if (write && n > capacity_groups) return fail(HSPMM_ERR_INVALID, "%u groups, room for %u", n, capacity_groups);
    return HSPMM_OK;
}

}  // extern "C"
