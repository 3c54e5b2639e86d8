// Host-side work partition for the persistent SpMM waves.
//
// The reference walks effective row windows round-robin over its thread blocks
// (reference src/fp16.cu:86, 138) and each window's tiles in order
// (src/fp16.cu:90, 140).  Here the flat tile sequence 0..T-1 (windows are
// contiguous in it) is cut into ranges of about equal cost; one wave walks one
// range.  A cut that falls near a window boundary snaps to it; a window that is
// still cut (a heavy window) has its per-range partial sums kept in fp32 slots
// and added in range order by a second small kernel, so the result does not
// depend on timing.
#pragma once
#include <cstdint>
#include <vector>
#include <algorithm>

namespace hspmm {

constexpr uint32_t kNoSlot = 0xFFFFFFFFu;



struct Range {
    uint32_t tile_begin, tile_end;    // [begin, end) in the flat tile sequence
    uint32_t first_window;            // effective window holding tile_begin
    uint32_t head_slot, tail_slot;    // partial-sum slots (kNoSlot = none)
    uint32_t head_split, tail_split;  // index of the cut window's entry in Partition::split
    uint32_t combine;                 // 1: the ranges of this range's group add their sums before they leave the chip;
                                      // 2: they are a whole window, which the group stores itself
};

struct SplitWindow {
    uint32_t window;                  // effective window index
    uint32_t slot_begin, slot_count;  // into Partition::fix_slots, in range order
};

struct Partition {
    std::vector<Range> ranges;
    std::vector<SplitWindow> split;
    std::vector<uint32_t> fix_slots;
    uint32_t n_slots = 0;
};

// rowOffset has W+1 entries, rowOffset[0] == 0, strictly increasing.
// target_ranges: wanted number of ranges (>= 1).
// window_cost: cost of finishing one window, in units of one tile.
// slack: a cut closer than slack * (mean tiles per range) to a window boundary
// moves onto the boundary.
// whole_window_margin: when no window costs more than a mean range plus this many
// tiles, every cut moves onto a boundary and no window is cut: halving so short a
// window saves less time than the second launch that adds its partial sums costs
// (measured: about 6 us against 0.4 us per tile of one wave).
// group: ranges group * k .. group * k + group - 1 are walked by the waves of one workgroup.  Where all
// of them lie inside one window, the workgroup adds their partial sums itself (in range order) and
// the group takes one slot, that of its first range, instead of one per range.
// allowed_cuts (optional; ascending, holds every window boundary): a cut inside a window moves to the
// nearest of these positions - the ends of the caller's groups (reference GBTCF_MTX,
// src/utils/class.h:93-108), so that a window is cut only where the caller cut it.
inline Partition build_partition(uint32_t W, const uint32_t *rowOffset, uint32_t target_ranges,
                                 double window_cost = 1.5, double slack = 0.35, double whole_window_margin = 32.0,
                                 uint32_t group = 1, const std::vector<uint32_t> *allowed_cuts = nullptr)
{
    Partition P;
    if (W == 0) return P;
    const uint32_t T = rowOffset[W];
    if (T == 0) return P;
    if (target_ranges < 1) target_ranges = 1;
    const double total = double(T) + window_cost * double(W);
    const double per = total / double(target_ranges);
    double snap = slack * double(T) / double(target_ranges);
    {
        uint32_t longest = 0;
        for (uint32_t i = 0; i < W; ++i) longest = std::max(longest, rowOffset[i + 1] - rowOffset[i]);
        if (double(longest) + window_cost <= per + whole_window_margin) snap = double(T);
    }

    std::vector<uint32_t> cuts;
    cuts.reserve(target_ranges + 1);
    cuts.push_back(0);
    uint32_t w = 0;                    // window holding the current cut (monotone)
    for (uint32_t i = 1; i < target_ranges; ++i) {
        const double c = per * double(i);
        // advance to the last window boundary whose prefix cost is <= c
        while (w + 1 <= W && double(rowOffset[w + 1]) + window_cost * double(w + 1) <= c) ++w;
        if (w >= W) break;
        const double base = double(rowOffset[w]) + window_cost * double(w);
        const uint32_t ws = rowOffset[w], we = rowOffset[w + 1];
        double into = c - base;
        if (into < 0) into = 0;
        uint32_t tau = ws + uint32_t(into);
        if (tau > we) tau = we;
        if (double(tau - ws) <= snap) tau = ws;
        else if (double(we - tau) <= snap) tau = we;
        if (allowed_cuts && tau > ws && tau < we) {
            auto hi = std::lower_bound(allowed_cuts->begin(), allowed_cuts->end(), tau);     // <= we: boundaries are in the list
            const uint32_t above = hi == allowed_cuts->end() ? we : *hi;
            const uint32_t below = hi == allowed_cuts->begin() ? ws : *(hi - 1);
            tau = above - tau < tau - below ? above : below;
            if (tau < ws) tau = ws;
            if (tau > we) tau = we;
        }
        if (tau > cuts.back() && tau < T) cuts.push_back(tau);
    }
    cuts.push_back(T);

    const size_t R = cuts.size() - 1;
    P.ranges.resize(R);
    uint32_t win = 0;
    for (size_t r = 0; r < R; ++r) {
        Range &g = P.ranges[r];
        g.tile_begin = cuts[r];
        g.tile_end = cuts[r + 1];
        while (rowOffset[win + 1] <= g.tile_begin) ++win;
        g.first_window = win;
        g.head_slot = g.tail_slot = kNoSlot;
        g.head_split = g.tail_split = kNoSlot;
        g.combine = 0;
    }
    if (group > 1)
        for (size_t r0 = 0; r0 + group <= R; r0 += group) {
            const uint32_t w = P.ranges[r0].first_window;
            bool inside = true;
            for (uint32_t k = 0; k < group; ++k)
                inside = inside && P.ranges[r0 + k].first_window == w && P.ranges[r0 + k].tile_end <= rowOffset[w + 1];
            // two or more ranges inside one window: none of them is the whole window
            if (inside) for (uint32_t k = 0; k < group; ++k) P.ranges[r0 + k].combine = 1;
        }
    // Partial segments: only the first and the last window segment of a range can
    // be incomplete.  The kernel's rule: an incomplete segment that starts at the
    // range's first tile uses head_slot, any other incomplete segment tail_slot.
    uint32_t cur_split = kNoSlot;     // window of the open split entry
    for (size_t r = 0; r < R; ++r) {
        Range &g = P.ranges[r];
        uint32_t wv = g.first_window;
        uint32_t t = g.tile_begin;
        while (t < g.tile_end) {
            const uint32_t ws = rowOffset[wv], we = rowOffset[wv + 1];
            const uint32_t se = std::min(we, g.tile_end);
            const bool complete = (t == ws) && (se == we);
            if (!complete && g.combine && r % group != 0) {
                // the group's first range, in front of this one in the same window, holds the slot
            } else if (!complete) {
                const uint32_t slot = P.n_slots++;
                if (cur_split != wv) {
                    P.split.push_back(SplitWindow{wv, uint32_t(P.fix_slots.size()), 0});
                    cur_split = wv;
                }
                const uint32_t entry = uint32_t(P.split.size()) - 1u;
                if (t == g.tile_begin) { g.head_slot = slot; g.head_split = entry; }
                else { g.tail_slot = slot; g.tail_split = entry; }
                P.fix_slots.push_back(slot);
                P.split.back().slot_count++;
            }
            // jump over the complete windows in the middle of the range
            if (se == we) {
                ++wv;
                t = se;
                if (t < g.tile_end) {
                    // skip whole windows until the last one of the range
                    const uint32_t *lo = rowOffset + wv;
                    const uint32_t *hi = std::upper_bound(lo, rowOffset + W + 1, g.tile_end);
                    // windows wv .. (hi - rowOffset - 2) end at or before tile_end
                    const uint32_t last_full = uint32_t(hi - rowOffset) - 1;   // rowOffset[last_full] <= tile_end
                    if (last_full > wv) { wv = last_full; t = rowOffset[wv]; }
                }
            } else {
                t = se;
            }
        }
    }
    return P;
}

// Every window cut into `group` ranges of (almost) equal length, walked by the waves of one workgroup,
// which add their sums among themselves and store the window: no slot and no second kernel.  For
// matrices whose windows are all long; the caller makes sure every window has at least `group` tiles.
inline Partition build_aligned_partition(uint32_t W, const uint32_t *rowOffset, uint32_t group)
{
    Partition P;
    P.ranges.resize(size_t(W) * group);
    for (uint32_t w = 0; w < W; ++w) {
        const uint64_t ws = rowOffset[w], n = rowOffset[w + 1] - rowOffset[w];
        for (uint32_t k = 0; k < group; ++k) {
            Range &g = P.ranges[size_t(w) * group + k];
            g.tile_begin = uint32_t(ws + n * k / group);
            g.tile_end = uint32_t(ws + n * (k + 1) / group);
            g.first_window = w;
            g.head_slot = g.tail_slot = kNoSlot;
            g.head_split = g.tail_split = kNoSlot;
            g.combine = 2;
        }
    }
    return P;
}

}  // namespace hspmm
