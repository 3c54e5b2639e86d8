// The step streams a plan is built from: units (windows, or groups of adjacent windows) and, per step, the column
// ids and tiles in the order the lanes of the MFMA kernels read them; groups of windows that carry the union of
// their column lists for the LDS-panel kernels; steps stored without their zeros.  Host code only, no device
// calls: hspmm_create.hip uploads what these functions return.
#pragma once
#include <stdint.h>
#include <stddef.h>
#include <cstring>
#include <vector>
#include <algorithm>
#include "hspmm_device.h"
#include "host_parallel.hpp"

namespace hspmm_host {

// The step stream: units (single windows, or pairs of vertically adjacent windows
// with one column list) and, per step, the ids and tiles in the order the lanes
// of the MFMA kernels read them.
struct StepStream {
    int G = 1;
    std::vector<uint32_t> unitOffset, unitRow, unitWindow;   // unitWindow: first effective window of the unit
    uint32_t n_paired = 0, n_steps = 0;
    uint32_t n_wide = 0;                                     // units of three or four windows (LDS-panel stream only)
};

inline StepStream build_units(uint32_t W, uint32_t cw, const uint32_t *rowOffset, const uint32_t *rowIdx,
                       const uint32_t *ids_clean, int pairing)
{
    StepStream st;
    // which windows could pair with their successor
    std::vector<uint8_t> can(W, 0);
    uint64_t paired_tiles = 0;
    if (pairing != 1) {
        for (uint32_t w = 0; w + 1 < W; ++w) {
            const uint32_t n = rowOffset[w + 1] - rowOffset[w];
            if (rowIdx[w + 1] != rowIdx[w] + HSPMM_ROW_WINDOW || rowOffset[w + 2] - rowOffset[w + 1] != n) continue;
            const uint32_t *a = ids_clean + size_t(rowOffset[w]) * cw;
            const uint32_t *b = ids_clean + size_t(rowOffset[w + 1]) * cw;
            if (std::memcmp(a, b, size_t(n) * cw * 4) == 0) can[w] = 1;
        }
        for (uint32_t w = 0; w + 1 < W;) {
            if (can[w]) { paired_tiles += 2ull * (rowOffset[w + 1] - rowOffset[w]); w += 2; } else ++w;
        }
    }
    // pairs pay off when a fair share of the tiles is in them: an unpaired window in a
    // paired stream costs a zero tile and an idle MFMA
    const bool use_pairs = pairing == 2 ? paired_tiles > 0 : (pairing == 0 && paired_tiles * 4ull >= uint64_t(rowOffset[W]));
    st.G = use_pairs ? 2 : 1;
    st.unitOffset.push_back(0);
    for (uint32_t w = 0; w < W;) {
        const uint32_t n = rowOffset[w + 1] - rowOffset[w];
        const bool pair = use_pairs && w + 1 < W && can[w];
        st.unitWindow.push_back(w);
        st.unitRow.push_back(rowIdx[w] | (pair ? 1u : 0u));
        st.unitOffset.push_back(st.unitOffset.back() + n);
        st.n_paired += pair;
        w += pair ? 2 : 1;
    }
    st.n_steps = st.unitOffset.back();
    return st;
}

// ids per step in lane order.  fp16: the 16 ids of the step's tile.  fp32: [g][2] = (id g, id g + 4).
inline hspmm_host::ZeroedBuffer<uint32_t> lane_order_ids(const StepStream &st, int dtype, const uint32_t *rowOffset, const uint32_t *ids_clean)
{
    const uint32_t cw = dtype == HSPMM_TF32 ? 8u : 16u;
    hspmm_host::ZeroedBuffer<uint32_t> out(size_t(st.n_steps) * cw);
    hspmm_host::parallel_blocks(st.unitRow.size(), 256, [&](size_t ub, size_t ue) {
        for (size_t u = ub; u < ue; ++u) {
            const uint32_t t0 = rowOffset[st.unitWindow[u]];
            for (uint32_t i = 0, n = st.unitOffset[u + 1] - st.unitOffset[u]; i < n; ++i) {
                const uint32_t *src = ids_clean + size_t(t0 + i) * cw;
                uint32_t *dst = out.data() + size_t(st.unitOffset[u] + i) * cw;
                if (dtype != HSPMM_TF32) std::memcpy(dst, src, 64);
                else for (uint32_t g = 0; g < 4; ++g) { dst[2 * g] = src[g]; dst[2 * g + 1] = src[g + 4]; }
            }
        }
    });
    return out;
}

// tiles per step in lane order, as 32-bit words.
//   fp16: [row r][g][window][2 words = halves 4g..4g+3 of row r]
//   fp32: [row r][g][window][2 words = a[r][g], a[r][g+4]]
inline hspmm_host::ZeroedBuffer<uint32_t> lane_order_tiles(const StepStream &st, int dtype, const uint32_t *rowOffset, const void *data)
{
    const int G = st.G;
    const uint32_t *words = static_cast<const uint32_t *>(data);     // a tile is 64 words in both formats
    hspmm_host::ZeroedBuffer<uint32_t> out(size_t(st.n_steps) * 64u * G);
    hspmm_host::parallel_blocks(st.unitRow.size(), 64, [&](size_t ub, size_t ue) {
        for (size_t u = ub; u < ue; ++u) {
            const uint32_t w0 = st.unitWindow[u];
            const int nwin = (st.unitRow[u] & 1u) ? 2 : 1;
            for (uint32_t i = 0, n = st.unitOffset[u + 1] - st.unitOffset[u]; i < n; ++i) {
                uint32_t *dst = out.data() + size_t(st.unitOffset[u] + i) * 64u * G;
                for (int w = 0; w < nwin; ++w) {
                    const uint32_t *src = words + size_t(rowOffset[w0 + w] + i) * 64u;
                    for (uint32_t r = 0; r < 8; ++r)
                        for (uint32_t g = 0; g < 4; ++g) {
                            uint32_t *d = dst + ((r * 4 + g) * G + w) * 2;
                            if (dtype != HSPMM_TF32) { d[0] = src[r * 8 + 2 * g]; d[1] = src[r * 8 + 2 * g + 1]; }
                            else { d[0] = src[r * 8 + g]; d[1] = src[r * 8 + g + 4]; }
                        }
                }
            }
        }
    });
    return out;
}

// 16-bit steps of 32 columns for the LDS-panel kernels (Fp16Tr in spmm_panel_kernel.hpp): a re-tiled
// step of a window is [row r][32 halves]; lane l = (g, m) of the step's 1 KB gets the 16 bytes
// a[m][8g .. 8g + 7], m = row of the unit's 16 rows (rows 8..15: the second window of a pair, else zero).
// A stream with units of up to four windows (G = 4) has a second KB per step for windows 2 and 3.
inline hspmm_host::ZeroedBuffer<uint32_t> lane_order_wide_steps(const StepStream &st, const uint32_t *rowOffset, const void *data)
{
    const uint16_t *halves = static_cast<const uint16_t *>(data);   // a step of a window is 8 x 32 halves
    const size_t step_words = st.G == 4 ? 512u : 256u;
    hspmm_host::ZeroedBuffer<uint32_t> out(size_t(st.n_steps) * step_words);
    hspmm_host::parallel_blocks(st.unitRow.size(), 16, [&](size_t ub, size_t ue) {
        for (size_t u = ub; u < ue; ++u) {
            const uint32_t w0 = st.unitWindow[u];
            const uint32_t nwin = (st.unitRow[u] & 3u) + 1u;
            for (uint32_t i = 0, n = st.unitOffset[u + 1] - st.unitOffset[u]; i < n; ++i) {
                uint16_t *dst = reinterpret_cast<uint16_t *>(out.data() + size_t(st.unitOffset[u] + i) * step_words);
                for (uint32_t w = 0; w < nwin; ++w) {
                    const uint16_t *src = halves + size_t(rowOffset[w0 + w] + i) * 256u;
                    uint16_t *half = dst + (w >> 1) * 512u;
                    for (uint32_t r = 0; r < 8; ++r)
                        for (uint32_t g = 0; g < 4; ++g)
                            std::memcpy(half + ((g * 16u + 8u * (w & 1u) + r) * 8u), src + r * 32u + 8u * g, 16);
                }
            }
        }
    });
    return out;
}

// fp32 value -> its upper 16 bits (bf16, cut) in the low half, bf16(value - that) (nearest even) in the
// high half; the same split the producer waves apply to B (write_piece of Fp32Split in spmm_panel_kernel.hpp).
inline uint32_t split_bf16_host(float v)
{
    uint32_t bits;
    std::memcpy(&bits, &v, 4);
    const uint32_t hi = bits & 0xFFFF0000u;
    if ((bits & 0x7F800000u) == 0x7F800000u) return hi >> 16;            // infinite or NaN: hi carries it
    float hf;
    std::memcpy(&hf, &hi, 4);
    const float rest = v - hf;                                            // exact
    uint32_t rb;
    std::memcpy(&rb, &rest, 4);
    rb += 0x7FFFu + ((rb >> 16) & 1u);                                    // nearest even (rest is finite and small)
    return (hi >> 16) | (rb & 0xFFFF0000u);
}

// fp32 steps of 32 columns in the split form (Fp32Split): a re-tiled step of a window is [row r][32 floats];
// lane l = (g, m) gets 32 bytes: the 8 hi halves, then the 8 lo halves of a[m][8g .. 8g + 7].  A stream with
// units of up to four windows (G = 4) has a second 2 KB per step for windows 2 and 3.
inline hspmm_host::ZeroedBuffer<uint32_t> lane_order_split_steps(const StepStream &st, const uint32_t *rowOffset, const void *data)
{
    const float *vals = static_cast<const float *>(data);            // a step of a window is 8 x 32 floats
    const size_t step_words = st.G == 4 ? 1024u : 512u;
    hspmm_host::ZeroedBuffer<uint32_t> out(size_t(st.n_steps) * step_words);
    hspmm_host::parallel_blocks(st.unitRow.size(), 16, [&](size_t ub, size_t ue) {
        for (size_t u = ub; u < ue; ++u) {
            const uint32_t w0 = st.unitWindow[u];
            const uint32_t nwin = (st.unitRow[u] & 3u) + 1u;
            for (uint32_t i = 0, n = st.unitOffset[u + 1] - st.unitOffset[u]; i < n; ++i) {
                uint16_t *dst = reinterpret_cast<uint16_t *>(out.data() + size_t(st.unitOffset[u] + i) * step_words);
                for (uint32_t w = 0; w < nwin; ++w) {
                    const float *src = vals + size_t(rowOffset[w0 + w] + i) * 256u;
                    uint16_t *half = dst + (w >> 1) * 1024u;
                    for (uint32_t r = 0; r < 8; ++r)
                        for (uint32_t g = 0; g < 4; ++g)
                            for (uint32_t c = 0; c < 8; ++c) {
                                const uint32_t sp = split_bf16_host(src[r * 32u + 8u * g + c]);
                                uint16_t *lane = half + (g * 16u + 8u * (w & 1u) + r) * 16u;
                                lane[c] = uint16_t(sp & 0xFFFFu);
                                lane[8 + c] = uint16_t(sp >> 16);
                            }
                }
            }
        }
    });
    return out;
}

// For the LDS-panel kernels built on the 16-bit MFMA a step multiplies 16 rows, and a wave can run one
// second operand (the gathered rows of B, read from LDS - what binds these kernels) against two first
// operands, 32 rows.  So vertically adjacent windows should share their steps: groups of up to four
// windows are rewritten to carry the union of their column lists (absent entries become stored zeros)
// and run as one unit.  merge_groups is one pass over neighbouring groups: two groups whose windows
// number at most max_windows are merged when cost x steps(union) < steps(a) + steps(b), steps counted
// in panels of panel_cols columns and steps of step_cols (no step straddles a panel); cost = 1 for a
// pair (its step costs what a single window's costs), wide_cost for three and four windows (the same
// LDS reads, twice the MFMAs).  Pruned dense weights at 10 % density: 4.6 steps per 256 columns for a
// window, 6.5 for a pair, 7.7 for four; sparser matrices still save the half-empty last step of every
// panel.  Returns false (outputs unused) when no two groups merge.
struct Unioned {
    std::vector<uint32_t> rowOffset, tcA2B;
    hspmm_host::ZeroedBuffer<uint8_t> data;
    uint32_t T = 0;
};

inline bool merge_groups(uint32_t W, uint32_t cw, uint32_t elem, uint32_t panel_cols, uint32_t step_cols, uint32_t max_windows,
                  double wide_cost, const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data,
                  const uint32_t *rowIdx, const std::vector<uint32_t> &first, const std::vector<uint32_t> &count,
                  Unioned &out, std::vector<uint32_t> &out_first, std::vector<uint32_t> &out_count)
{
    // steps of step_cols columns an ascending list needs when no step straddles a panel of panel_cols
    auto panel_steps = [&](const uint32_t *c, uint32_t n) {
        uint32_t steps = 0;
        for (uint32_t i = 0; i < n;) {
            const uint32_t pn = c[i] / panel_cols, a = i;
            while (i < n && c[i] / panel_cols == pn) ++i;
            steps += (i - a + step_cols - 1) / step_cols;
        }
        return steps;
    };
    const size_t tile_bytes = size_t(8) * cw * elem;
    const uint8_t *src = static_cast<const uint8_t *>(data);
    auto real_ids = [&](uint32_t w) {
        uint32_t n = (rowOffset[w + 1] - rowOffset[w]) * cw;
        const uint32_t *c = tcA2B + size_t(rowOffset[w]) * cw;
        while (n && c[n - 1] == HSPMM_IDX_MAX) --n;
        return n;
    };
    // (the converters write ascending lists; a caller's list in another order is only merged with an equal one)
    auto ascending = [](const uint32_t *c, uint32_t n) {
        for (uint32_t i = 1; i < n; ++i) if (c[i] <= c[i - 1]) return false;
        return true;
    };
    // the column list of the merged group (all windows of a group carry their group's list)
    auto merged_list = [&](uint32_t wa, uint32_t wb, std::vector<uint32_t> &merged) {
        const uint32_t *a = tcA2B + size_t(rowOffset[wa]) * cw, *b = tcA2B + size_t(rowOffset[wb]) * cw;
        const uint32_t na = real_ids(wa), nb = real_ids(wb);
        if (na == nb && std::memcmp(a, b, size_t(na) * 4) == 0) { merged.assign(a, a + na); return; }
        merged.resize(size_t(na) + nb);
        merged.resize(size_t(std::set_union(a, a + na, b, b + nb, merged.begin()) - merged.begin()));
    };
    // first pass: which groups could join their successor (all candidates, in parallel), then the
    // greedy choice from the top, and the new tile counts
    const size_t NG = first.size();
    std::vector<uint8_t> can(NG, 0), join(NG, 0);
    std::vector<uint32_t> union_tiles(NG, 0u), tiles(W);
    // (as many groups per worker as make a few thousand tiles)
    const size_t groups_per_worker = std::max<size_t>(1, (size_t(1) << 12) / std::max<uint32_t>(1u, rowOffset[W] / W));
    hspmm_host::parallel_blocks(NG - 1, groups_per_worker, [&](size_t gb, size_t ge) {
        std::vector<uint32_t> merged;
        for (size_t g = gb; g < ge; ++g) {
            const uint32_t wa = first[g], wb = first[g + 1], nw = count[g] + count[g + 1];
            if (rowIdx[wb] != rowIdx[wa] + HSPMM_ROW_WINDOW * count[g] || nw > max_windows) continue;
            const uint32_t *a = tcA2B + size_t(rowOffset[wa]) * cw, *b = tcA2B + size_t(rowOffset[wb]) * cw;
            const uint32_t na = real_ids(wa), nb = real_ids(wb);
            const bool same = na == nb && std::memcmp(a, b, size_t(na) * 4) == 0;
            if (!same && (!ascending(a, na) || !ascending(b, nb))) continue;
            merged_list(wa, wb, merged);
            const uint32_t nu = uint32_t(merged.size());
            const double cost = nw > 2 ? wide_cost : 1.0;
            if (same || cost * double(panel_steps(merged.data(), nu)) < double(panel_steps(a, na) + panel_steps(b, nb))) {
                can[g] = 1;
                union_tiles[g] = (nu + cw - 1) / cw;
            }
        }
    });
    bool any = false;
    for (uint32_t w = 0; w < W; ++w) tiles[w] = rowOffset[w + 1] - rowOffset[w];
    for (size_t g = 0; g + 1 < NG;) {
        if (!can[g]) { ++g; continue; }
        join[g] = 1; any = true;
        for (uint32_t w = first[g]; w < first[g] + count[g] + count[g + 1]; ++w) tiles[w] = union_tiles[g];
        g += 2;
    }
    if (!any) return false;
    out.rowOffset.assign(size_t(W) + 1, 0u);
    for (uint32_t w = 0; w < W; ++w) out.rowOffset[w + 1] = out.rowOffset[w] + tiles[w];
    out.T = out.rowOffset[W];
    out.tcA2B.assign(size_t(out.T) * cw, HSPMM_IDX_MAX);
    out.data = hspmm_host::ZeroedBuffer<uint8_t>(size_t(out.T) * tile_bytes);
    // second pass: copy, or spread a window's tile columns over the merged list's columns
    auto spread = [&](uint32_t w, const uint32_t *ids, uint32_t n_ids) {
        const uint32_t *c = tcA2B + size_t(rowOffset[w]) * cw;
        const uint32_t n = real_ids(w);
        uint32_t *dst_ids = out.tcA2B.data() + size_t(out.rowOffset[w]) * cw;
        std::memcpy(dst_ids, ids, size_t(n_ids) * 4);
        uint32_t j = 0;                                         // position in the merged list (same order)
        for (uint32_t i = 0; i < n; ++i) {
            while (ids[j] != c[i]) ++j;
            const uint8_t *st = src + size_t(rowOffset[w] + i / cw) * tile_bytes;
            uint8_t *dt = out.data.data() + size_t(out.rowOffset[w] + j / cw) * tile_bytes;
            for (uint32_t r = 0; r < 8; ++r)
                std::memcpy(dt + (size_t(r) * cw + j % cw) * elem, st + (size_t(r) * cw + i % cw) * elem, elem);
        }
    };
    out_first.clear(); out_count.clear();
    std::vector<uint32_t> second;                               // first window of the group that joined, or IDX_MAX
    for (size_t g = 0; g < NG; ++g) {
        out_first.push_back(first[g]);
        out_count.push_back(join[g] ? count[g] + count[g + 1] : count[g]);
        second.push_back(join[g] ? first[g + 1] : HSPMM_IDX_MAX);
        if (join[g]) ++g;
    }
    hspmm_host::parallel_blocks(out_first.size(), groups_per_worker, [&](size_t gb, size_t ge) {
        std::vector<uint32_t> merged;
        for (size_t g = gb; g < ge; ++g) {
            const uint32_t wa = out_first[g], nw = out_count[g];
            if (second[g] != HSPMM_IDX_MAX) {
                merged_list(wa, second[g], merged);
                for (uint32_t w = wa; w < wa + nw; ++w) spread(w, merged.data(), uint32_t(merged.size()));
            } else {
                for (uint32_t w = wa; w < wa + nw; ++w) {
                    std::memcpy(out.tcA2B.data() + size_t(out.rowOffset[w]) * cw, tcA2B + size_t(rowOffset[w]) * cw,
                                size_t(tiles[w]) * cw * 4);
                    std::memcpy(out.data.data() + size_t(out.rowOffset[w]) * tile_bytes,
                                src + size_t(rowOffset[w]) * tile_bytes, size_t(tiles[w]) * tile_bytes);
                }
            }
        }
    });
    return true;
}

// The two passes of merge_groups: windows into pairs, then neighbouring groups into units of up to
// max_windows (2 or 4) windows, the second pass only when it leaves at least min_wide_units units.
// On return rowOffset / tcA2B / data point to the arrays the groups refer to: the caller's, or those
// of `un` when anything was merged.
inline void group_windows(uint32_t W, uint32_t cw, uint32_t elem, uint32_t panel_cols, uint32_t step_cols, uint32_t max_windows,
                   double wide_cost, size_t min_wide_units, const uint32_t *&rowOffset, const uint32_t *&tcA2B,
                   const void *&data, const uint32_t *rowIdx, Unioned &un, std::vector<uint32_t> &first,
                   std::vector<uint32_t> &count)
{
    first.resize(W); count.assign(W, 1u);
    for (uint32_t w = 0; w < W; ++w) first[w] = w;
    if (max_windows < 2 || W < 2) return;
    std::vector<uint32_t> f2, c2;
    if (merge_groups(W, cw, elem, panel_cols, step_cols, 2, 1.0, rowOffset, tcA2B, data, rowIdx, first, count, un, f2, c2)) {
        rowOffset = un.rowOffset.data(); tcA2B = un.tcA2B.data(); data = un.data.data();
        first.swap(f2); count.swap(c2);
    }
    Unioned un2;
    if (max_windows > 2 && first.size() / 2u >= min_wide_units &&
        merge_groups(W, cw, elem, panel_cols, step_cols, max_windows, wide_cost, rowOffset, tcA2B, data, rowIdx, first,
                     count, un2, f2, c2) &&
        f2.size() >= min_wide_units) {
        un = std::move(un2);
        rowOffset = un.rowOffset.data(); tcA2B = un.tcA2B.data(); data = un.data.data();
        first.swap(f2); count.swap(c2);
    }
}

// Two units per consumer wave of the LDS-panel kernels ("tall" streams): units 2q and 2q + 1 become one
// sequence of steps, panel by panel the steps of the first, then those of the second (marked with bit 28 of
// their id words; the panel counts in bits 0..3 are those of the merged sequence).  One image of a panel in
// LDS then serves twice as many rows.  ids: 16 words per step; tiles: tile_words per step.
inline void merge_unit_pairs(uint32_t U, uint32_t NP, size_t tile_words, const std::vector<uint32_t> &unitOffset,
                      std::vector<uint32_t> &poff, std::vector<uint32_t> &step_panel, std::vector<uint32_t> &ids,
                      hspmm_host::ZeroedBuffer<uint32_t> &tiles)
{
    const uint32_t Q = (U + 1u) / 2u;
    const size_t n_steps = step_panel.size();
    std::vector<uint32_t> n_poff(size_t(Q) * (NP + 1)), n_panel(n_steps), n_ids(ids.size());
    hspmm_host::ZeroedBuffer<uint32_t> n_tiles(tiles.size());
    hspmm_host::parallel_blocks(Q, 8, [&](size_t qb, size_t qe) {
        for (size_t q = qb; q < qe; ++q) {
            const uint32_t a = uint32_t(2 * q), b = a + 1u;
            const bool two = b < U;
            const uint32_t *pa = poff.data() + size_t(a) * (NP + 1);
            const uint32_t *pb = two ? poff.data() + size_t(b) * (NP + 1) : nullptr;
            uint32_t at = unitOffset[a];                          // the pair's steps start where its first unit's did
            uint32_t *po = n_poff.data() + q * (NP + 1);
            uint32_t prev_panel = 0;
            bool first = true;
            for (uint32_t pn = 0; pn <= NP; ++pn) {
                po[pn] = at;
                if (pn == NP) break;
                for (int which = 0; which < (two ? 2 : 1); ++which) {
                    const uint32_t *src_off = which ? pb : pa;
                    for (uint32_t t = src_off[pn]; t < src_off[pn + 1]; ++t, ++at) {
                        const uint32_t jump = first ? 0u : pn - prev_panel;
                        first = false;
                        prev_panel = pn;
                        n_panel[at] = pn;
                        for (uint32_t w = 0; w < 16; ++w)
                            n_ids[size_t(at) * 16 + w] = (ids[size_t(t) * 16 + w] & 0x0FFFFFF0u) | jump | (which ? 1u << 28 : 0u);
                        std::memcpy(n_tiles.data() + size_t(at) * tile_words, tiles.data() + size_t(t) * tile_words,
                                    tile_words * 4);
                    }
                }
            }
        }
    });
    poff.swap(n_poff); step_panel.swap(n_panel); ids.swap(n_ids); tiles.swap(n_tiles);
}

// The tiles of a stream of 16 x 32 steps without their zeros.  A lane-order step is [lane l][8 values] (16-bit
// types: halves; fp32 in bf16 parts: 8 hi halves then 8 lo halves).  masks[8 s + i] has bit l set when lane l's
// i-th value of step s is stored (any bit pattern but +0); the stored values follow in the order (i, l), one
// half each (fp32 in parts: one word, hi | lo << 16), those of step s from position step_voff[s] on.  Position
// 0 holds a zero, and a step's worth of zeros follows the last value.  This is the bitmap layout of the
// reference's BTCF_MTX (nnzOffset / tcBit / packed data, reference src/utils/class.h:55-67 and
// src/utils/convert.h:83-101) with one bitmap per step and the bits in the order the lanes need them.
inline void pack_steps(size_t n_steps, bool split, const hspmm_host::ZeroedBuffer<uint32_t> &tiles, std::vector<uint64_t> &masks,
                std::vector<uint8_t> &vals, std::vector<uint32_t> &step_voff)
{
    const size_t lane_halves = split ? 16 : 8, es = split ? 4 : 2;
    const uint16_t *h = reinterpret_cast<const uint16_t *>(tiles.data());
    masks.assign(n_steps * 8, 0);
    step_voff.assign(n_steps + 1, 0);
    auto stored = [&](size_t s, uint32_t l, uint32_t i) {
        const uint16_t *lane = h + (s * 64 + l) * lane_halves;
        return split ? (lane[i] | lane[8 + i]) != 0 : lane[i] != 0;
    };
    hspmm_host::parallel_blocks(n_steps, 1024, [&](size_t sb, size_t se) {
        for (size_t s = sb; s < se; ++s) {
            uint32_t count = 0;
            for (uint32_t i = 0; i < 8; ++i) {
                uint64_t m = 0;
                for (uint32_t l = 0; l < 64; ++l) if (stored(s, l, i)) m |= uint64_t(1) << l;
                masks[s * 8 + i] = m;
                count += uint32_t(__builtin_popcountll(m));
            }
            step_voff[s + 1] = count;
        }
    });
    step_voff[0] = 1;                                             // position 0: the zero
    for (size_t s = 0; s < n_steps; ++s) step_voff[s + 1] += step_voff[s];
    vals.assign((size_t(step_voff[n_steps]) + 512) * es, 0);
    hspmm_host::parallel_blocks(n_steps, 1024, [&](size_t sb, size_t se) {
        for (size_t s = sb; s < se; ++s) {
            size_t at = step_voff[s];
            for (uint32_t i = 0; i < 8; ++i)
                for (uint32_t l = 0; l < 64; ++l) {
                    if (!(masks[s * 8 + i] >> l & 1u)) continue;
                    const uint16_t *lane = h + (s * 64 + l) * lane_halves;
                    if (split) {
                        const uint32_t w = uint32_t(lane[i]) | uint32_t(lane[8 + i]) << 16;
                        std::memcpy(vals.data() + at * 4, &w, 4);
                    } else {
                        std::memcpy(vals.data() + at * 2, &lane[i], 2);
                    }
                    ++at;
                }
        }
    });
}

}  // namespace hspmm_host
