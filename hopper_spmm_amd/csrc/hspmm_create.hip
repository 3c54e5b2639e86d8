// C ABI of the SpMM operator (include/hspmm.h), part 2 of 3: plan creation - validation of the caller's
// arrays (reference src/utils/class.h:55-108), upload, the step streams of the two kernel families, the
// work partition.  Everything the reference's fp16_spmm does before its first launch (reference
// src/fp16.cu:221-254), done once per matrix.
#include "hspmm_plan.hpp"

using namespace hspmm_host;

namespace hspmm_host {

// canonical (optional): whether every window's real column ids ascend strictly with padding only behind
// the window's last column, as the reference's converter writes them (src/utils/convert.h:166-181).
int validate_format(uint32_t rows, uint32_t cols, uint32_t W, uint32_t T, uint32_t cw,
                    const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data, const uint32_t *rowIdx,
                    bool *canonical)
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
    // every tile's ids: real columns below `cols`, padding only behind them.  Checked on all cores; the message
    // names the first tile that fails.
    auto tile_error = [&](uint32_t t, bool report) -> bool {
        const uint32_t *ids = tcA2B + size_t(t) * cw;
        if (ids[0] == HSPMM_IDX_MAX) { if (report) fail(HSPMM_ERR_INVALID, "tile %u starts with a padding column", t); return true; }
        bool pad = false;
        for (uint32_t k = 0; k < cw; ++k) {
            if (ids[k] == HSPMM_IDX_MAX) { pad = true; continue; }
            if (pad) { if (report) fail(HSPMM_ERR_INVALID, "tile %u: column id after padding", t); return true; }
            if (ids[k] >= cols) { if (report) fail(HSPMM_ERR_INVALID, "tile %u: column id %u >= cols %u", t, ids[k], cols); return true; }
        }
        return false;
    };
    std::atomic<uint32_t> first_bad{T};
    hspmm_host::parallel_blocks(T, 65536, [&](size_t tb, size_t te) {
        if (tb >= first_bad.load(std::memory_order_relaxed)) return;
        for (size_t t = tb; t < te; ++t)
            if (tile_error(uint32_t(t), false)) {
                uint32_t seen = first_bad.load(std::memory_order_relaxed);
                while (uint32_t(t) < seen && !first_bad.compare_exchange_weak(seen, uint32_t(t), std::memory_order_relaxed)) {}
                return;
            }
    });
    if (first_bad.load() < T) { tile_error(first_bad.load(), true); return HSPMM_ERR_INVALID; }
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

int build_and_upload_partition(hspmm_plan *p, int level, uint32_t group, bool aligned)
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

}  // namespace hspmm_host

namespace {

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
    // (hspmm_set_panel_stream, libraries built with EXPERIMENTAL=1).
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

extern "C" {

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

}  // extern "C"
