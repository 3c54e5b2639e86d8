// Shared between the kernels and the C ABI layer: kernel argument block and
// launch entry points.  Internal; the public interface is include/hspmm.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

namespace hspmm {

constexpr uint32_t kIdxMax = 0xFFFFFFFFu;      // reference src/common.h:47
constexpr uint32_t kRowWindow = 8u;            // reference src/common.h:17
constexpr uint32_t kRangeWordsDev = 8u;
constexpr uint32_t kRangeWords = kRangeWordsDev;
constexpr uint32_t kFixWords = 4u;
constexpr int kMaxWavesPerGroup = 4;
constexpr int kAlignedGroupWaves = 8;          // waves of a workgroup that walks one whole unit (aligned partition)

struct KernelArgs {
    // the four format arrays exactly as given (device copies), reference
    // src/fp16.cu:38-41: read by the scalar kernel
    const uint32_t *rowOffset;
    const uint32_t *tcA2B;
    const void     *data;
    const uint32_t *rowIdx;
    // the step stream the MFMA kernels walk
    const uint32_t *unitOffset;  // n_units + 1: first step of every unit
    const uint32_t *unitRow;     // n_units: first matrix row of the unit | its windows less one (1: a pair)
    const uint32_t *ids;         // per step, lane order, padding ids renamed
    const void     *tiles;       // per step, lane order; bitmap stream: the stored elements, tile after tile
    const uint32_t *bm_header;   // bitmap stream (kLayoutDWB): per step 8 words - the tile's four bitmap words, the bit
                                 // counts of words 0, 0..1, 0..2 (bytes 1..3), the position of its first stored element
    // partition
    const uint32_t *ranges;      // n_ranges x kRangeWords
    const uint32_t *split;       // n_split x kFixWords {unit, slot_begin, slot_count, 0}
    const uint32_t *fix_slots;
    float          *scratch;     // partial sums: [slot][feature block][acc reg][lane] x 4 floats
    uint32_t       *arrive;      // [split unit][feature block] arrival counters (all zero between launches);
                                 // null: the partial sums are added by a second kernel
    const void     *B;           // cols x N
    void           *C;           // rows x N
    uint32_t n_ranges, n_split, eff_windows, n_units, rows, N, n_feat_blocks;
    uint32_t ld;                 // elements from one row of B (and of C) to the next: N, or more when the launch
                                 // covers a range of the features only (MFMA kernels; the scalar kernel takes whole rows)
    uint32_t xcd_split;          // != 0 (gather kernels; 2, 4 or 8 feature blocks): every feature block has XCDs of its own
    uint32_t uniform_chunks;     // != 0 (LDS-panel kernels): no split table - entry e is unit e, whose partial sums
                                 // are slots e * uniform_chunks .. + uniform_chunks - 1, in that order
};

// dtype: 0 = fp16 tiles 8x16, 1 = fp32 tiles 8x8, 2 = bf16 tiles 8x16.  V = 32-bit words a lane loads
// per B row (1, 2 or 4).
// layout (fp16 only): kLayoutX4 = wide loads, contiguous features per lane, N % (2V) == 0;
// kLayoutDW = word loads, features strided by 32 per lane, N % (32V) == 0.
constexpr int kLayoutX4 = 0, kLayoutDW = 1, kLayoutDWB = 2;   // DWB: word loads, tiles as bitmap + stored elements (16-bit, G = 1)
// element types, numbered as HSPMM_FP16 / HSPMM_TF32 / HSPMM_BF16 of the public header
constexpr int kDtypeF16 = 0, kDtypeF32 = 1, kDtypeBf16 = 2;
// The gather kernels' prefetch depth (steps of loads in flight per wave) when the caller sets none: what fits 128
// registers per lane without spilling.  Workgroups of eight waves and 64-bit gather offsets are built for this depth
// only; depths 2, 3 and 4 exist for the rest (1, 6 and 8 in builds with HSPMM_EXPERIMENTAL).
constexpr int default_prefetch(int elem_bytes, int G, int V)
{
    return elem_bytes == 4 ? (G == 2 && V == 4 ? 3 : 4) : (G == 2 && V == 4 ? 2 : 3);
}
// narrow: B < 4 GiB and cols < 2^24 (32-bit gather offsets).
// mid: optional event recorded between the main kernel and the partial-sum kernel.
// G: windows per unit in the step stream (1, or 2 when the plan paired windows).
hipError_t launch_spmm_mfma(int dtype, int layout, int G, const KernelArgs &ka, int V, int prefetch, bool narrow,
                            int waves_per_group, hipStream_t s, hipEvent_t mid);
hipError_t launch_spmm_scalar(int dtype, const KernelArgs &ka, hipStream_t s);

// LDS-panel kernels (spmm_panel_kernel.hpp).
constexpr uint32_t kPanelRowBytes = 256;       // bytes of a B row one workgroup covers (128 halves / 64 floats)
// B rows per panel: 256 for the kernels built on the transposing LDS read (16-bit types, fp32 in bf16
// parts), 128 for the fp32 MFMA forms
constexpr uint32_t kPanelRowsWide = 256, kPanelRowsFp32 = 128;

struct PanelArgs {
    const uint32_t *unitRow;     // n_units: first matrix row of the unit | its windows less one (0..3)
    const uint32_t *poff;        // n_units x (n_panels + 1): first step of the unit at or behind every panel
    const uint32_t *step_panel;  // per step: its panel
    const uint32_t *ids;         // per step: the rows (inside the panel) each quarter-wave reads and the panels
                                 // between the step and the one in front of it; the format depends on the element
                                 // type (PanelOps in spmm_panel_kernel.hpp)
    const void     *tiles;       // per step, lane order (null when the stream is packed)
    // packed streams (tiles without their zeros): per step eight lane masks; the stored values, (mask, lane)
    // order, values[0] = 0; per step the position of its first value
    const uint64_t *masks;
    const void     *vals;
    const uint32_t *step_voff;
    float          *scratch;     // partial sums [unit * n_chunks + chunk][feature block][acc reg][lane]
    uint32_t       *arrive;      // per (unit, feature block): chunks that have left their sums (zero between launches);
                                 // null: a second kernel adds the sums
    const void     *B;
    void           *C;
    uint32_t n_units, n_steps, rows, cols, N, n_feat_blocks, n_panels, n_chunks, panels_per_chunk;
    uint32_t units_per_group;    // consumer waves of a workgroup that get a unit (<= those the kernel has); the
                                 // others only keep the barriers company
};

// units: 12 or 14 units (consumer waves) per workgroup, 2 more waves copy B to LDS; 13 = 12 units and 4 such waves.
// G: windows per unit at most (1, 2, 4); 0 = fp32 single windows with ids in the format of the 4x4x1 tile.  split (fp32): the plan's
// stream is in the bf16 hi / lo form.  ka: arguments of the kernel that adds the chunk sums (split table with one
// entry per unit), used when pa.n_chunks > 1.
// tall: the stream gives every consumer wave two units (poff per pair of units, steps of the second unit marked);
// packed: its tiles are stored without their zeros (tall streams only).
hipError_t launch_spmm_panel(int dtype, int G, bool split, bool tall, bool packed, const PanelArgs &pa, const KernelArgs &ka,
                             int units, hipStream_t s, hipEvent_t mid);
hipError_t launch_fill_zero(void *dst, size_t bytes, hipStream_t s);
// bitmap tiles (header, stored elements: see KernelArgs::bm_header and, for 32-bit elements, launch_bitmap_header
// below) -> plain tiles (8 x 16 of 16-bit elements, 8 x 8 of 32-bit elements)
hipError_t launch_expand_bitmap(int elem_bytes, const uint32_t *header, const void *vals, void *tiles, uint32_t n_tiles,
                                hipStream_t s);
// n 16-bit elements -> n words with the element in the low half (launch_widen_halves), and back (launch_narrow_words):
// a single feature of a 16-bit type runs as two features, the second all zero
hipError_t launch_widen_halves(const void *src, void *dst, size_t n, hipStream_t s);
hipError_t launch_narrow_words(const void *src, void *dst, size_t n, hipStream_t s);
// plain 8 x 8 tiles of 32-bit elements, single windows -> the order the lanes of the fp32 gather kernels read them in
hipError_t launch_lane_order32(const void *tiles, void *out, uint32_t n_tiles, hipStream_t s);
// plain tiles -> bitmap tiles (8 x 16 tiles of 16-bit elements, elem_bytes = 2: 8 header words per tile, see
// KernelArgs::bm_header; 8 x 8 tiles of 32-bit elements, elem_bytes = 4: 4 header words - rows 0..3, rows 4..7,
// position of the first stored element, number of stored elements), in two steps with the host in between (it
// sizes `vals`): launch_bitmap_header writes the masks and the tiles' counts, and leaves in block_sums
// (bitmap_scan_blocks(n_tiles) + 1 words of 64 bits) the exclusive sums per 2048 tiles and, last, the number of
// stored elements; launch_bitmap_pack writes the positions and the stored elements.
uint32_t bitmap_scan_blocks(uint32_t n_tiles);
hipError_t launch_bitmap_header(int elem_bytes, const void *tiles, uint32_t *header, uint32_t n_tiles, uint64_t *block_sums,
                                hipStream_t s);
hipError_t launch_bitmap_pack(int elem_bytes, const void *tiles, uint32_t *header, void *vals, uint32_t n_tiles,
                              const uint64_t *block_sums, hipStream_t s);
// Measurement only (gather_rate_kernel in hspmm_kernels.hip): loads part_bytes (128 or 256) of row ids[i] of B for
// every i < n_ids; parts > 1: `parts` parts of part_bytes each, dealt out by XCD, every part walking all ids.
hipError_t launch_gather_rate(const uint32_t *ids, uint64_t n_ids, const void *B, uint32_t row_bytes, uint32_t part_bytes,
                              uint32_t parts, int compute_units, uint32_t *sink, hipStream_t s);

}  // namespace hspmm
