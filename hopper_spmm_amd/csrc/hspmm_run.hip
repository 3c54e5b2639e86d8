// C ABI of the SpMM operator (include/hspmm.h), part 3 of 3: launches - hspmm_run, hspmm_run_static,
// hspmm_prepare, and the timing entry points (hspmm_bench follows the reference's convention of warm-up and
// timed launches, reference src/fp16.cu:255-268, src/common.h:48-49).
#include "hspmm_plan.hpp"

using namespace hspmm_host;

// The fixed scratch array of hspmm_run_static (see static_scratch_address below): device memory the
// library holds on every device it is loaded on, for callers that must not allocate.
constexpr size_t kStaticScratchBytes = HSPMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char hspmm_static_scratch[kStaticScratchBytes];

namespace hspmm_host {

// The fixed scratch array of hspmm_run_static: one copy per device, held from the moment the library is
// loaded on that device until the process ends.  Host code never passes the array's name to a kernel (on
// the host it names a stand-in, not device memory): the device address is looked up once per device with
// hipGetSymbolAddress and that pointer is what launches carry.
constexpr int kMaxDevices = 64;
static std::mutex g_static_mutex;
static void *g_static_scratch_ptr[kMaxDevices] = {};

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

}  // namespace hspmm_host

namespace {

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

}  // extern "C"
