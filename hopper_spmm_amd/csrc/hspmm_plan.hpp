// Internal header of the library's host code: what hspmm_capi.hip (settings, queries), hspmm_create.hip
// (plan creation) and hspmm_run.hip (launches) share - the plan, the process-wide settings, error reporting.
#pragma once
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

namespace hspmm_host {

// Stores the message hspmm_last_error returns on this thread and returns `code` (hspmm_capi.hip).
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

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
extern std::mutex g_cfg_mutex;          // guards g_cfg (hspmm_capi.hip)
extern Config g_cfg;

constexpr uint32_t kMinTilesPerRange = 24;

}  // namespace hspmm_host

struct hspmm_plan {
    int dtype = 0;
    int device = 0;
    uint32_t rows = 0, cols = 0, W = 0, T = 0;
    uint32_t cw = 16, elem = 2;
    int compute_units = 0;
    hspmm_host::Config cfg;
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

namespace hspmm_host {

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

// How a launch gets the memory it needs beyond the plan's fixed arrays.
//   kLaunch:  hspmm_run - may build a partition and grow the plan's scratch buffer (under the plan's mutex)
//   kPrepare: hspmm_prepare - builds and grows exactly like kLaunch and launches nothing
//   kStatic:  hspmm_run_static - partial sums go to the library's fixed device array; builds and allocates nothing
enum class RunMode { kLaunch, kPrepare, kStatic };

// hspmm_create.hip
int validate_format(uint32_t rows, uint32_t cols, uint32_t W, uint32_t T, uint32_t cw,
                    const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data, const uint32_t *rowIdx,
                    bool *canonical = nullptr);
int choose_ranges(const hspmm_plan *p);
int build_and_upload_partition(hspmm_plan *p, int level, uint32_t group = 1, bool aligned = false);

// hspmm_run.hip: the address of the device's fixed scratch array (hspmm_run_static); `device` must be current
int static_scratch_address(int device, float **out);

}  // namespace hspmm_host
