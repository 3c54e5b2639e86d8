/*
 * hspmm.h - C ABI of the MI355X (gfx950) SpMM operator  C = A * B
 *
 * A is sparse in the condensed row-window tile format without bitmap
 * (BTCF_MTX_NO_BITMAP, reference src/utils/class.h:74-85, produced by
 * CSR2BTCFNOBITMAP, reference src/utils/convert.h:146-225):
 *   rowOffset[W+1]  first tile of each effective 8-row window
 *   tcA2B[T*CW]     column id of every tile column, IDX_MAX (0xFFFFFFFF) = padding
 *   data[T*8*CW]    dense 8 x CW tiles, row-major inside a tile
 *   rowIdx[W]       first matrix row of each effective window (multiple of 8)
 * with CW = 16 and 2-byte values for HSPMM_FP16 (IEEE half) and HSPMM_BF16
 * (bfloat16), CW = 8 and 4-byte float values for HSPMM_TF32 (reference
 * src/common.h:14-43).
 * B is dense cols x N, C is dense rows x N, both row-major, same element type
 * as `data` (reference src/fp16.cu:36-46, 163-170).  Accumulation is fp32; the
 * 16-bit paths round once to nearest-even on store.
 *
 * All functions return 0 (HSPMM_OK) or a positive error code; the text of the
 * last error on the calling thread is available from hspmm_last_error().
 * Nothing here calls exit() or throws across the boundary.
 */
#ifndef HSPMM_H
#define HSPMM_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HSPMM_FP16 0            /* reference -DUSE_FP16 build, src/common.h:14-19 */
#define HSPMM_TF32 1            /* reference -DUSE_TF32 build, src/common.h:26-43 (fp32 storage) */
#define HSPMM_BF16 2            /* reference -DUSE_BF16 build, src/common.h:20-25 (the reference has no bf16 program) */
#define HSPMM_IDX_MAX 0xFFFFFFFFu   /* reference src/common.h:47 */
#define HSPMM_ROW_WINDOW 8u         /* reference src/common.h:17 */

enum {
    HSPMM_OK = 0,
    HSPMM_ERR_INVALID = 1,      /* bad argument or malformed format arrays */
    HSPMM_ERR_DEVICE = 2,       /* a HIP runtime call failed */
    HSPMM_ERR_ALLOC = 3,        /* host or device allocation failed */
    HSPMM_ERR_IO = 4,           /* file cannot be opened / parsed */
    HSPMM_ERR_UNSUPPORTED = 5
};

typedef struct hspmm_plan hspmm_plan;

/* ---- device operator ---------------------------------------------------- */

/* Replaces the allocation + host-to-device part of fp16_spmm (reference
 * src/fp16.cu:228-249) and create_tma_desc_A (src/fp16.cu:177-219): validates
 * the four format arrays (host pointers), copies them to the current HIP
 * device and builds the work partition the kernels walk.  `dtype` is
 * HSPMM_FP16, HSPMM_TF32 or HSPMM_BF16.
 * Column lists: the reference's converter writes every window's real column
 * ids strictly ascending, with padding only behind the window's last column
 * (src/utils/convert.h:166-181).  Other orders are accepted (ids < cols,
 * padding only at the end of a tile) and give the same product, but such a plan
 * runs the gather and all-shapes kernels only: the LDS-staging kernels, and the
 * merging of adjacent windows, need the ascending order.
 * Tuning variables of the environment (HSPMM_*) are read here, once per plan. */
int hspmm_create(hspmm_plan **plan, int dtype, uint32_t rows, uint32_t cols,
                 uint32_t eff_row_windows, uint32_t total_tiles,
                 const uint32_t *rowOffset, const uint32_t *tcA2B,
                 const void *data, const uint32_t *rowIdx);

/* Replaces one launch of fp16_spmm_kernel (reference src/fp16.cu:256): computes
 * all of C = A*B for feature dimension N.  dB (cols x N) and dC (rows x N) are
 * DEVICE pointers, row-major, aligned to the element size (the LDS-staging kernels
 * want one block of features - 256 bytes of a row - and take B and C wherever they start, the widest loads
 * of the other MFMA kernels want 16 bytes and N a multiple of 8 - of 4 for fp32 storage -; everything else
 * takes narrower loads or two launches; a single feature of a 16-bit type goes
 * through a buffer of cols + rows words that the plan allocates at the first such
 * launch or at hspmm_prepare(plan, 1)); every element of C is
 * written (rows without nonzeros become 0).  Asynchronous on `stream` (a
 * hipStream_t, NULL = default stream).
 * Host side: a plan is immutable after hspmm_create except for what the first
 * launch with a new N, or on a new stream, may add under the plan's own mutex -
 * a work partition for that width and buffers for what a launch writes besides C
 * (partial sums of cut windows, their arrival counters; older buffers stay
 * allocated until hspmm_destroy, so launches recorded earlier, e.g. in a HIP
 * graph, stay valid whatever N is run afterwards).  hspmm_run may therefore be
 * called from several threads; after one earlier call with that N on that
 * stream it only launches kernels (no allocation, memset or copy) and can be
 * captured in a HIP graph.
 * Device side: every stream that launches a plan gets buffers of its own at its
 * first launch, so launches of one plan on different streams may overlap in time
 * (as may different plans); launches on one stream are ordered anyway.  Two
 * exceptions share the buffers of the first stream the plan saw, and must then
 * not overlap with its launches: a stream that is being captured when it first
 * launches the plan (nothing is allocated under capture: launch once on that
 * stream before the capture, or call hspmm_prepare(plan, N) first and keep the
 * graph's replays apart from launches on the plan's first stream), and streams
 * beyond the sixteenth. */
int hspmm_run(hspmm_plan *plan, const void *dB, void *dC, uint32_t N, void *stream);

/* No reference counterpart (the reference allocates inside every call,
 * src/fp16.cu:236-249): builds now what the first hspmm_run with feature
 * dimension N would build - the work partition for that width and, for every
 * stream that has launched the plan so far (for the set that the first stream
 * and streams under capture use, if none has; the first stream that launches
 * the plan afterwards takes that set over), the buffers a launch writes
 * besides C, for every alignment of B and C - and launches nothing. */
int hspmm_prepare(hspmm_plan *plan, uint32_t N);

/* No reference counterpart; for callers that must not allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): hspmm_run with the partial sums of cut windows kept in a fixed
 * array of device memory that the library holds on every device it is loaded
 * on (HSPMM_STATIC_SCRATCH_BYTES, from library load until the process ends)
 * instead of the plan's own buffer.  It calls no hipMalloc / hipFree and builds
 * nothing: the work partition for this N (and, for a single feature of a 16-bit
 * type, the plan's buffer of cols + rows words) must exist already (hspmm_prepare, or
 * one hspmm_run with this N), else HSPMM_ERR_UNSUPPORTED; so does a launch whose
 * partial sums exceed the array (the message says how much it needs).  Results
 * are bit-identical to hspmm_run.  All calls on one device share the one array
 * whatever their plan: two calls that overlap in time on one device race. */
#define HSPMM_STATIC_SCRATCH_BYTES (32u << 20)
int hspmm_run_static(hspmm_plan *plan, const void *dB, void *dC, uint32_t N, void *stream);

/* Replaces the warm-up + timed loop of fp16_spmm (reference src/fp16.cu:254-268,
 * WARMUP_RUNS / RUNS of src/common.h:48-49): `warmup` untimed launches, then
 * `runs` back-to-back launches between two device events on `stream`;
 * *total_ms receives the time of the `runs` launches together. */
int hspmm_bench(hspmm_plan *plan, const void *dB, void *dC, uint32_t N,
                int warmup, int runs, void *stream, float *total_ms);

/* No reference counterpart (the reference times whole launches only): `runs`
 * launches with an event between the two kernels of a launch; *main_ms is the
 * total time of the main kernel, *fixup_ms of the kernel that adds the partial
 * sums of windows split across waves (0 when no window is split). */
int hspmm_profile(hspmm_plan *plan, const void *dB, void *dC, uint32_t N, int runs, void *stream,
                  float *main_ms, float *fixup_ms);

/* No reference counterpart.  Measurement only: launches, `runs` times, a kernel that
 * loads every row of B the plan's step stream gathers (each (window, column) pair
 * once, in the stream's order, N elements per row, in the same parts and with the
 * same assignment to XCDs as the gather kernels use) and does nothing else.  *ms
 * receives the mean time of one run, *bytes_per_run (optional) the bytes its lanes
 * load.  That time is a floor for any kernel that gathers these rows: bench.py
 * reports it next to the SpMM kernel's time.  N * element size must be a multiple
 * of 128 bytes and dB aligned to 16. */
int hspmm_measure_gather(hspmm_plan *plan, const void *dB, uint32_t N, int runs, void *stream, float *ms,
                         uint64_t *bytes_per_run);

/* Replaces the cudaFree block of fp16_spmm (reference src/fp16.cu:274-279). */
void hspmm_destroy(hspmm_plan *plan);

/* Replaces checkCudaErrors' message (reference src/utils/utils.h:9-21) without
 * exiting: text of the last failure on this thread ("" if none). */
const char *hspmm_last_error(void);

/* Replaces Scheduler::configure (reference src/scheduler.h:33-38).  Values are
 * read by the next hspmm_create on any thread; 0 keeps the built-in default.
 *   buffer_stage             tiles each wave keeps in flight (prefetch depth): 2, 3 or 4 (builds with
 *                            EXPERIMENTAL=1 also 1, 6 and 8); launches with 64-bit gather offsets (a B of
 *                            4 GiB or more) and workgroups of eight waves use the default depth
 *   consumer_warp_num        waves per workgroup, 1..4
 *   producer_warp_group_num  tile ranges (waves) per SIMD the partition aims at, 1..16
 *   sm_num                   compute units to balance over (default: the device's) */
int hspmm_configure(int buffer_stage, int consumer_warp_num,
                    int producer_warp_group_num, int sm_num);
/* Getter side of the same singleton (reference src/scheduler.h:26-30, 41). */
void hspmm_get_config(int *buffer_stage, int *consumer_warp_num,
                      int *producer_warp_group_num, int *sm_num);

/* No reference counterpart.  1 when the library was built with EXPERIMENTAL=1 (csrc/Makefile): it then also
 * holds the kernel variants that no automatic plan selects - prefetch depths 1, 6 and 8, the stream modes 1 and 2
 * of hspmm_set_panel_stream, units of four windows for fp32 storage in bf16 parts, the other workgroup shapes of
 * the fp32-MFMA LDS-staging kernels - which were measured against the defaults and lost.  0: those requests fail
 * with HSPMM_ERR_INVALID / HSPMM_ERR_UNSUPPORTED. */
int hspmm_has_experimental(void);

/* Kernel selection, read by the next hspmm_create: 0 = automatic (MFMA kernels
 * whenever the feature dimension allows; the kernels that stage B through LDS
 * for matrices whose windows touch a large share of the columns), 1 = always the
 * scalar all-shapes kernel, 2 = 16-bit MFMA kernel with wide loads only, 3 =
 * 16-bit MFMA kernel with word loads whenever N is a multiple of 32, 4 = the
 * LDS-staging kernels for every matrix (whenever N is 128 at least - 64 for fp32
 * storage, or 16 with rows of whole 16-byte pieces), 5 = the same
 * with fp32 products in the HSPMM_TF32 LDS-staging kernels (N 64 at least).  (By default those
 * kernels multiply the bf16 parts hi + lo of every fp32 factor, which keeps 16
 * mantissa bits per factor; the reference's tf32 instruction keeps 10,
 * src/ptx/wgmma.h:42-58.  The other HSPMM_TF32 kernels always multiply in fp32.) */
int hspmm_set_kernel_mode(int mode);

/* No reference counterpart.  Two vertically adjacent windows with the same
 * column list (block-clustered weights) can share one gather of B.  Read by the
 * next hspmm_create: 0 = pair when at least a quarter of the tiles would be in
 * pairs, 1 = never, 2 = whenever any two windows qualify.  The LDS-staging
 * kernels built on the 16-bit MFMA (a step of theirs multiplies 16 or 32 rows)
 * go further unless the mode is 1: in their copy of the matrix groups of up to
 * four adjacent windows carry the union of their column lists, absent entries
 * as zeros, wherever that saves work. */
int hspmm_set_window_pairing(int mode);

/* Bitmap tiles on the device (the reference's CSR2BTCF format, src/utils/convert.h:22-139
 * and BTCF_MTX of src/utils/class.h:55-67, which its kernel never reads).  Read by the
 * next hspmm_create / hspmm_create_bitmap / hspmm_create_grouped.  mode 0 (default): the
 * LDS-staging kernels stream their steps as uncompressed tiles.  mode 1: every consumer
 * wave of theirs takes two units (one copy of a panel of B in LDS then serves twice the
 * rows).  mode 2: as 1, and the tiles of the steps are kept on the device without their
 * zeros - per step of 16 rows x 32 columns a 512-bit mask and the stored values - and
 * expanded in registers (a lane finds its values by counting mask bits below it).
 * Modes 1 and 2 apply to streams built on the 16-bit MFMA (fp16, bf16, fp32 in bf16
 * parts) whose units have at most two windows; other plans ignore them.  Results are
 * bit-identical in all three modes.  Both cut the bytes a launch moves (measured: a
 * third and 60 % fewer 128-byte lines into the compute units) and neither makes it
 * faster on the configurations measured: these kernels are bound by the LDS reads and
 * MFMAs of a step, not by their traffic; hence the default.  Modes 1 and 2 exist in builds with
 * EXPERIMENTAL=1 only (hspmm_has_experimental); elsewhere they return HSPMM_ERR_UNSUPPORTED. */
int hspmm_set_panel_stream(int mode);

/* No reference counterpart (the reference defines the grouped format, src/utils/class.h:93-108
 * and src/utils/convert.h:232-276, but no kernel that walks it): process-wide like
 * hspmm_configure, read by the next hspmm_create_grouped.  mode 0 (default): consecutive groups
 * with one row index are one window again and the plan cuts heavy windows where its own cost
 * model puts the cuts.  mode 1: the plan's waves walk whole groups - a window given as several
 * groups (atomic = 1) is cut only where one of its groups ends, a window given as one group is
 * never cut; partial sums of a cut window are added in group order, not with atomics.  Kept by
 * plans whose units are the caller's single windows walked by the gather kernels
 * (hspmm_plan_info.group_cuts_kept = 1); plans that merge windows with one column list, the
 * LDS-staging kernels (they walk a re-tiled stream) and the all-shapes kernel (one wave per
 * window, nothing cut) have no use for the cuts.  The product is the same up to the order of the
 * fp32 additions of a cut window. */
int hspmm_set_group_cuts(int mode);

/* No reference counterpart; host only (no device needed).  The grouping that the
 * LDS-staging kernels built on the 16-bit MFMA apply to their copy of the
 * matrix, for tests and for sizing: adjacent windows are merged into units of up
 * to max_windows (1, 2 or 4) windows that carry the union of their column lists
 * wherever that saves steps of 32 columns inside panels of 256 columns (a step of
 * three or four windows counted as 1.25).  Outputs, each optional: the groups
 * (first window and window count; at most eff_row_windows of them), the tile
 * offsets of the rewritten matrix (eff_row_windows + 1 words), its tile count,
 * and its tcA2B / data arrays when they fit capacity_tiles tiles
 * (HSPMM_ERR_INVALID otherwise; *new_total_tiles then says how many are needed).
 * All windows of a group carry the same column list; added entries are zeros. */
int hspmm_panel_units_preview(int dtype, uint32_t rows, uint32_t cols, uint32_t eff_row_windows, uint32_t total_tiles,
                              const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data,
                              const uint32_t *rowIdx, uint32_t max_windows, uint32_t *n_groups,
                              uint32_t *group_first, uint32_t *group_count, uint32_t *new_rowOffset,
                              uint32_t *new_total_tiles, uint32_t capacity_tiles, uint32_t *new_tcA2B,
                              void *new_data);

typedef struct {
    uint32_t rows, cols, eff_row_windows, total_tiles;
    int32_t  dtype;
    uint32_t n_ranges;          /* tile ranges (one wave each per feature block) */
    uint32_t n_split_windows;   /* windows whose tiles span more than one range */
    uint32_t n_partial_slots;   /* fp32 partial accumulators the split windows use */
    uint32_t compute_units;
    uint32_t n_units;           /* units of the step stream: single windows and pairs */
    uint32_t n_paired_units;    /* units made of two adjacent windows with one column list */
    uint64_t device_bytes;      /* bytes of device memory the plan holds right now */
    uint32_t n_panels;          /* column panels of the LDS-staging kernels; 0: the plan does not use them */
    uint32_t n_panel_steps;     /* steps of the unit stream re-tiled panel by panel */
    uint32_t n_panel_units;     /* units of that stream: groups of up to four adjacent windows that share, or were given, one column list */
    uint32_t n_panel_paired_units;  /* of those: units of two or more windows */
    uint32_t n_panel_wide_units;    /* of those: units of three or four windows */
    uint32_t last_kernel_family;    /* what the last hspmm_run launched: 0 nothing yet, 1 all-shapes kernel, 2 gather (MFMA) kernels,
                                       3 LDS-staging kernels, 4 clear only (matrix without entries) */
    uint32_t gather_bitmap;         /* 1: the gather kernels read this plan's tiles as bitmap + stored elements (single
                                     * windows with few stored elements per tile), 0: as uncompressed tiles */
    uint32_t bitmap_from_caller;    /* 1: the plan was made from bitmap tiles (hspmm_create_bitmap / _grouped) and uploaded them as they
                                     * came - header words from tcBit and nnzOffset, the stored elements untouched; the plain tiles
                                     * that some kernels read were written by a kernel on the device */
    uint32_t panel_stream_mode;     /* the LDS-staging stream as built (hspmm_set_panel_stream): 0 uncompressed tiles, 1 two units
                                     * per consumer wave, 2 also tiles without their zeros; 0 when the plan has no such stream */
    uint32_t group_cuts_kept;       /* 1: the plan cuts a window only where the caller's groups end (hspmm_set_group_cuts) */
    uint32_t last_mfma_kind;        /* matrix instruction of the last hspmm_run's main kernel: 0 none (all-shapes kernel, clear),
                                     * 1 v_mfma_f32_16x16x32_f16, 2 v_mfma_f32_16x16x32_bf16, 3 v_mfma_f32_16x16x4_f32,
                                     * 4 v_mfma_f32_4x4x1_16B_f32 */
    uint32_t last_mfma_flops;       /* floating-point operations of one such instruction (16384, 16384, 2048, 512) */
    uint64_t last_mfma_instructions;    /* how many of them that launch issued (zero padding of tiles and rows included) */
} hspmm_plan_info;

/* No reference counterpart (the reference prints its statistics from main,
 * src/fp16.cu:295-301): reports the shape of the plan and of its partition. */
int hspmm_get_plan_info(const hspmm_plan *plan, hspmm_plan_info *info);

/* No reference counterpart: copies the partition for inspection (tests).
 * ranges: n_ranges x 5 words {tile_begin, tile_end, first_window, head_slot,
 * tail_slot} (slot 0xFFFFFFFF = none). */
int hspmm_get_partition(const hspmm_plan *plan, uint32_t *ranges, uint32_t capacity_ranges);

/* The plan's own balanced partition in the form of the reference's grouped format (GBTCF_MTX, reference
 * src/utils/class.h:93-108; BTCF2GBTCF, src/utils/convert.h:232-276, cuts every window into groups of a fixed
 * length instead): one group per piece of a window that one wave walks, groupOffset[g] its first tile in the
 * caller's tile arrays (groupOffset[total] = total_tiles), groupRowIdx[g] the window's first row, atomic[g] = 1
 * where the window continues in another group.  Together with the tile arrays the plan was made from this is a
 * GBTCF_MTX that hspmm_create_grouped takes back.  First call with the arrays NULL for *total_groups.  A plan
 * that walks pairs of windows (equal column lists merged: its steps are not the caller's tiles) writes the balanced
 * partition of the caller's single windows instead, built with the same cost model.  Host only. */
int hspmm_partition_as_groups(const hspmm_plan *plan, uint32_t capacity_groups, uint32_t *total_groups,
                              uint32_t *groupOffset, uint32_t *groupRowIdx, uint8_t *atomic);

/* No reference counterpart: the partition hspmm_create would build for a
 * rowOffset array and a wanted number of ranges, computed on the host alone
 * (no device needed).  ranges as in hspmm_get_partition; any output may be NULL. */
int hspmm_partition_preview(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                            uint32_t *ranges, uint32_t capacity_ranges, uint32_t *n_ranges,
                            uint32_t *n_split_windows, uint32_t *n_partial_slots);

/* No reference counterpart: the same for the case that the waves of a workgroup
 * walk `group` consecutive ranges (1..4) and add the partial sums of one window
 * among themselves before one sum leaves the chip (what hspmm_run does when one
 * wave covers the whole feature dimension).  ranges: n_ranges x 6 words, the five
 * above and {combine}: 1 for the ranges of a group that lies inside one window;
 * only the group's first range then has a slot. */
int hspmm_partition_preview_grouped(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                                    uint32_t group, uint32_t *ranges, uint32_t capacity_ranges,
                                    uint32_t *n_ranges, uint32_t *n_split_windows, uint32_t *n_partial_slots);

/* No reference counterpart; host only.  The partition of a plan that keeps the caller's
 * group cuts (hspmm_set_group_cuts(1), hspmm_create_grouped): as hspmm_partition_preview,
 * but a cut inside a window moves to the nearest end of one of the caller's groups
 * (groupOffset of the reference's GBTCF_MTX, src/utils/class.h:93-108; total_groups + 1
 * entries, every window boundary among them). */
int hspmm_partition_preview_group_cuts(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t target_ranges,
                                       uint32_t total_groups, const uint32_t *groupOffset, uint32_t *ranges,
                                       uint32_t capacity_ranges, uint32_t *n_ranges, uint32_t *n_split_windows,
                                       uint32_t *n_partial_slots);

/* No reference counterpart; host only.  The partition used where every unit is
 * long (the balanced partition would cut each of them 2.5 ways or more, and one
 * wave covers the feature dimension): every window is cut into `group` (4 or 8)
 * ranges of about equal length, walked by the waves of one workgroup, which adds
 * their sums itself and stores the window - no slots and no second kernel.
 * Ranges as in hspmm_partition_preview_grouped (six words; the sixth is 2). */
int hspmm_partition_preview_aligned(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t group,
                                    uint32_t *ranges, uint32_t capacity_ranges, uint32_t *n_ranges);

/* ---- host format functions ---------------------------------------------- */

typedef struct {
    uint32_t rows, cols, nnzs;  /* CSR_MTX, reference src/utils/class.h:30-37 */
    uint32_t *row_ptr;          /* rows + 1 */
    uint32_t *col_idx;          /* nnzs */
    void     *values;           /* nnzs halves (HSPMM_FP16) or floats (HSPMM_TF32) */
} hspmm_csr;

/* Replaces load_matrix (reference src/utils/load.h:152-322): MatrixMarket
 * coordinate text -> CSR sorted by (row, column), 1-based -> 0-based, values
 * rounded to half for HSPMM_FP16.  Arrays are owned by the library until
 * hspmm_csr_free.  Returns HSPMM_ERR_IO where the reference prints an error
 * and returns an empty matrix. */
int hspmm_mtx_load(const char *path, int dtype, hspmm_csr *out);
/* Replaces free_csr_matrix (reference src/utils/load.h:337-355). */
void hspmm_csr_free(hspmm_csr *m);

/* Replaces CSR2BTCFNOBITMAP (reference src/utils/convert.h:146-225) in two
 * calls so that the caller owns the arrays: first the sizes, then the fill.
 * `transpose` != 0 gives the SPARSE_A_TRANSPOSE tile order (convert.h:207-209),
 * which the device operator takes through hspmm_create_layout. */
int hspmm_btcf_sizes(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                     uint32_t *eff_row_windows, uint32_t *total_tiles);
int hspmm_btcf_fill(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                    const void *values, int transpose,
                    uint32_t *rowOffset, uint32_t *tcA2B, void *data, uint32_t *rowIdx);

/* The same converter with the tile width given: col_window 0 or the element type's default (16 / 8), or 4 for
 * HSPMM_TF32 - the 8 x 4 tiles of the reference's -DMMA_M16N8K4 build (src/common.h:28-35: COL_WINDOW 4), which
 * hspmm_create_layout takes. */
int hspmm_btcf_sizes_cw(int dtype, uint32_t col_window, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                        uint32_t *eff_row_windows, uint32_t *total_tiles);
int hspmm_btcf_fill_cw(int dtype, uint32_t col_window, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                       const void *values, int transpose,
                       uint32_t *rowOffset, uint32_t *tcA2B, void *data, uint32_t *rowIdx);

/* ---- bitmap-compressed and grouped formats ------------------------------ */

/* Words of tcBit per tile: one 64-bit word for 8 x 8 tiles (HSPMM_TF32), two
 * for 8 x 16 tiles (reference src/utils/convert.h:61-66). */
#define HSPMM_BITMAP_WORDS(dtype) ((dtype) == HSPMM_TF32 ? 1u : 2u)

/* Where the bit of element (r, k) of tile t goes for 8 x 16 tiles.
 * HSPMM_BITS_PER_TILE: word 2t + bit/64, so every tile owns its two words; this
 * is the layout the plan functions below read.
 * HSPMM_BITS_AS_REFERENCE: word t + bit/64 in an array of 2 x tiles words, as
 * the reference indexes it (src/utils/convert.h:83,96-101): the high word of
 * tile t is also the low word of tile t + 1, which cannot be decoded; kept so
 * that the converter's output can be compared bit for bit.  Both layouts are
 * the same thing for 8 x 8 tiles. */
#define HSPMM_BITS_PER_TILE 0
#define HSPMM_BITS_AS_REFERENCE 1

/* Replaces CSR2BTCF (reference src/utils/convert.h:22-139; struct BTCF_MTX,
 * src/utils/class.h:55-67) in two calls.  Besides rowOffset, tcA2B and rowIdx
 * of the uncompressed format it gives nnzOffset (total_tiles + 1 prefix sums of
 * the stored entries per tile), tcBit (HSPMM_BITMAP_WORDS x total_tiles words,
 * bit r * COL_WINDOW + k set for a stored element, or k * 8 + r with
 * `transpose`) and `data` with the stored entries only, tile after tile in
 * ascending bit order.  *stored = entries of `data` = row_ptr[rows]. */
int hspmm_bitmap_sizes(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                       uint32_t *eff_row_windows, uint32_t *total_tiles, uint32_t *stored);
int hspmm_bitmap_fill(int dtype, uint32_t rows, const uint32_t *row_ptr, const uint32_t *col_idx,
                      const void *values, int transpose, int bit_layout,
                      uint32_t *rowOffset, uint32_t *nnzOffset, uint32_t *tcA2B, uint64_t *tcBit,
                      void *data, uint32_t *rowIdx);

/* No reference counterpart (the reference never decodes its bitmaps): expands
 * bitmap tiles (HSPMM_BITS_PER_TILE layout) to the dense 8 x COL_WINDOW tiles
 * of the uncompressed format; the k-th stored entry of a tile goes to the
 * offset of its k-th set bit.  Fails when a tile's bit count differs from its
 * nnzOffset span. */
int hspmm_bitmap_expand(int dtype, uint32_t total_tiles, const uint32_t *nnzOffset, const uint64_t *tcBit,
                        const void *data, void *dense_tiles);

/* hspmm_create for the two tile layouts behind the reference's optional build switches:
 *   col_window 4 (HSPMM_TF32 only): 8 x 4 tiles, the format of -DMMA_M16N8K4 (reference
 *     src/common.h:28-35: COL_WINDOW 4); 0 or the element type's default (16 / 8) otherwise;
 *   transposed != 0: element (r, k) of a tile at k * 8 + r, as the converters write it with
 *     -DSPARSE_A_TRANSPOSE (reference src/utils/convert.h:207-209).
 * The plan re-lays the tiles out once on the host (the real columns of every window keep their
 * order and are re-tiled with the default width); everything else is hspmm_create. */
int hspmm_create_layout(hspmm_plan **plan, int dtype, uint32_t col_window, int transposed, uint32_t rows, uint32_t cols,
                        uint32_t eff_row_windows, uint32_t total_tiles, const uint32_t *rowOffset, const uint32_t *tcA2B,
                        const void *data, const uint32_t *rowIdx);
/* The re-layout hspmm_create_layout does, for callers that keep the arrays (host only, no GPU):
 * tiles of width `col_window` (0 = default), column-major inside a tile if `transposed`, to tiles of
 * the default width in the order hspmm_create reads.  First the number of tiles, then the fill:
 * out_rowOffset[eff_row_windows + 1], out_tcA2B[total_tiles * width], out_data[total_tiles * 8 * width];
 * rowIdx does not change.  For tiles the reference's converter wrote (convert.h:146-225: every window's
 * sorted columns cut into tiles), the output is what that converter writes without the switches. */
int hspmm_btcf_relayout_sizes(int dtype, uint32_t col_window, uint32_t eff_row_windows, const uint32_t *rowOffset,
                              const uint32_t *tcA2B, uint32_t *total_tiles);
int hspmm_btcf_relayout_fill(int dtype, uint32_t col_window, int transposed, uint32_t eff_row_windows,
                             const uint32_t *rowOffset, const uint32_t *tcA2B, const void *data,
                             uint32_t *out_rowOffset, uint32_t *out_tcA2B, void *out_data);

/* Same as hspmm_create for a matrix held as bitmap tiles (row-major bit order,
 * HSPMM_BITS_PER_TILE).  Results are those of hspmm_create on the expanded arrays, bit for bit.
 * Sparse windows go to the device as they are: the gather kernels read the caller's tcBit words
 * and stored elements, and a kernel writes the plain tiles other kernels read
 * (hspmm_plan_info.bitmap_from_caller = 1).  Dense windows and windows paired through equal column
 * lists are expanded on the host first. */
int hspmm_create_bitmap(hspmm_plan **plan, int dtype, uint32_t rows, uint32_t cols,
                        uint32_t eff_row_windows, uint32_t total_tiles,
                        const uint32_t *rowOffset, const uint32_t *nnzOffset, const uint32_t *tcA2B,
                        const uint64_t *tcBit, const void *data, const uint32_t *rowIdx);

/* Replaces BTCF2GBTCF (reference src/utils/convert.h:232-276; struct GBTCF_MTX,
 * src/utils/class.h:93-108) in two calls: windows are cut into groups of at
 * most tgl tiles, tgl = max(floor(mean tiles per window), min_len) with the
 * reference's min_len = 32 (convert.h:242-243); a window of n tiles gets
 * g = ceil(n / tgl) groups starting ceil(n / g) tiles apart (convert.h:249-252).
 * groupOffset has total_groups + 1 entries, groupRowIdx and atomic one per
 * group (atomic = 1 where a window has more than one group, convert.h:254-257).
 * The tile arrays (nnzOffset, tcA2B, tcBit, data) are shared with the bitmap
 * format unchanged (convert.h:271-274). */
int hspmm_group_sizes(uint32_t eff_row_windows, const uint32_t *rowOffset, uint32_t min_len,
                      uint32_t *tgl, uint32_t *total_groups);
int hspmm_group_fill(uint32_t eff_row_windows, const uint32_t *rowOffset, const uint32_t *rowIdx,
                     uint32_t tgl, uint32_t *groupOffset, uint32_t *groupRowIdx, uint8_t *atomic);

/* Same as hspmm_create_bitmap for the grouped format: consecutive groups with
 * one row index are one window again (their partial results are summed in a
 * fixed order by the plan's own partition, not with atomics).  Fails when
 * groupOffset does not increase strictly, when groups of one window are not
 * adjacent, or when an atomic flag contradicts the grouping. */
int hspmm_create_grouped(hspmm_plan **plan, int dtype, uint32_t rows, uint32_t cols,
                         uint32_t total_groups, const uint32_t *groupOffset, const uint32_t *nnzOffset,
                         const uint32_t *tcA2B, const uint64_t *tcBit, const void *data,
                         const uint32_t *groupRowIdx, const uint8_t *atomic);

#ifdef __cplusplus
}
#endif
#endif /* HSPMM_H */
