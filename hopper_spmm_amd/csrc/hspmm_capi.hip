// C ABI of the SpMM operator (include/hspmm.h), part 1 of 3: error reporting, the process-wide settings
// (the knobs of the reference's Scheduler singleton, reference src/scheduler.h:7-41), previews of the work
// partition, queries on a plan, hspmm_destroy.  Plans are made in hspmm_create.hip and launched in
// hspmm_run.hip; the kernels live in hspmm_kernels.hip.  Together they mirror the host half of the
// reference's fp16_spmm (reference src/fp16.cu:221-281) split into create / run / bench / destroy so
// that a caller can keep A on the device across launches.
#include "hspmm_plan.hpp"

namespace hspmm_host {

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

void set_error(const std::string &msg) { g_last_error = msg; }

std::mutex g_cfg_mutex;
Config g_cfg;

}  // namespace hspmm_host

using namespace hspmm_host;

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
