// C++ host interface with the names and argument meaning of the reference's
// host code, implemented on the C ABI of libhspmm.so (include/hspmm.h):
//
//   compile-time element type   -DUSE_FP16 / -DUSE_BF16 / -DUSE_TF32   reference src/common.h:14-43
//   CSR_MTX, DENSE_MTX, BTCF_MTX_NO_BITMAP, PERF_RESULT      reference src/utils/class.h:30-48, 74-85; src/common.h:51-59
//   load_matrix, free_csr_matrix                             reference src/utils/load.h:152-355
//   CSR2BTCFNOBITMAP                                         reference src/utils/convert.h:146-225
//   fp16_spmm / tf32_spmm                                    reference src/fp16.cu:221-281
//   Scheduler                                                reference src/scheduler.h:5-42
//   verify_dense_matrix                                      reference src/utils/verify.h:18-42
//
// Differences from the reference, all deliberate: errors are reported (message on
// stderr, exit code 1) from this layer only, the library below never exits; the
// operator copies C back to the host (the reference stops after the timing loop,
// src/fp16.cu:269); tf32_spmm and bf16_spmm exist (the reference has no such entry points).
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include <hip/hip_runtime.h>
#include "../../include/hspmm.h"

#if !defined(USE_FP16) && !defined(USE_TF32) && !defined(USE_BF16)
#error "define USE_FP16, USE_BF16 or USE_TF32 (as the reference's Makefile does)"
#endif

#define MAT_PTR_TYPE uint32_t
#define MAT_IDX_TYPE uint32_t
#define vint uint32_t
#define ROW_WINDOW 8
#define IDX_MAX UINT32_MAX
#define WARMUP_RUNS 3
#define RUNS 5
#if defined(USE_FP16)
#define MAT_VAL_TYPE _Float16
#define COL_WINDOW 16
#define HSPMM_BUILD_DTYPE HSPMM_FP16
#elif defined(USE_BF16)
#define MAT_VAL_TYPE __bf16
#define COL_WINDOW 16
#define HSPMM_BUILD_DTYPE HSPMM_BF16
#else
#define MAT_VAL_TYPE float
#ifdef MMA_M16N8K4
#define COL_WINDOW 4            // reference src/common.h:28-35: 8 x 4 tiles
#else
#define COL_WINDOW 8
#endif
#define HSPMM_BUILD_DTYPE HSPMM_TF32
#endif

struct PERF_RESULT {
    float time;      // total milliseconds of `runs` launches
    int runs;
    void print() const
    {
        std::printf("SpMM total time: %.3f ms\n", time);
        std::printf("SpMM timed runs: %d\n", runs);
        std::printf("SpMM mean time: %.3f ms\n", time / static_cast<float>(runs));
    }
};

struct CSR_MTX {
    vint rows, cols, nnzs;
    MAT_PTR_TYPE *row_ptr;
    MAT_IDX_TYPE *col_idx;
    MAT_VAL_TYPE *values;
};

struct DENSE_MTX {
    vint rows, cols;
    MAT_VAL_TYPE *values;      // row-major
};

struct BTCF_MTX_NO_BITMAP {
    vint rows, cols, nnzs;
    vint total_row_windows, eff_row_windows;
    std::vector<MAT_PTR_TYPE> rowOffset;
    std::vector<MAT_IDX_TYPE> tcA2B;
    std::vector<MAT_VAL_TYPE> data;
    std::vector<MAT_IDX_TYPE> rowIdx;
    uint32_t total_tiles;
};

// Bitmap-compressed tiles (reference src/utils/class.h:55-67).  For 8 x 16 tiles
// tcBit holds two words per tile, tile t in words 2t and 2t + 1.
#define MAT_MAP_TYPE uint64_t
#define ATOMIC_TYPE uint8_t
struct BTCF_MTX {
    vint rows, cols, nnzs;
    vint total_row_windows, eff_row_windows;
    std::vector<MAT_PTR_TYPE> rowOffset;
    std::vector<MAT_PTR_TYPE> nnzOffset;
    std::vector<MAT_IDX_TYPE> tcA2B;
    std::vector<MAT_MAP_TYPE> tcBit;
    std::vector<MAT_VAL_TYPE> data;       // stored entries only, indexed through nnzOffset
    std::vector<MAT_IDX_TYPE> rowIdx;
};

// Grouped tiles (reference src/utils/class.h:93-108).
struct GBTCF_MTX {
    vint rows, cols, nnzs;
    vint total_row_windows, total_groups, eff_row_windows;
    std::vector<MAT_PTR_TYPE> groupOffset;
    std::vector<MAT_PTR_TYPE> nnzOffset;
    std::vector<MAT_IDX_TYPE> tcA2B;
    std::vector<MAT_MAP_TYPE> tcBit;
    std::vector<MAT_VAL_TYPE> data;
    std::vector<MAT_IDX_TYPE> rowIdx;     // one per group
    std::vector<ATOMIC_TYPE> atomic;      // 1 where a window was cut into several groups
};

namespace hspmm_cpp {
[[noreturn]] inline void die(const char *what)
{
    std::fprintf(stderr, "%s: %s\n", what, hspmm_last_error());
    std::exit(EXIT_FAILURE);
}
inline void check_hip(hipError_t e, const char *what)
{
    if (e != hipSuccess) {
        std::fprintf(stderr, "%s: %s\n", what, hipGetErrorString(e));
        std::exit(EXIT_FAILURE);
    }
}
}  // namespace hspmm_cpp

// An unreadable file gives an empty matrix and a message, as in the reference
// (src/utils/load.h:176-180, 190-194).  enable_validation re-checks the CSR
// structure (the checks of src/utils/load.h:44-73).
inline CSR_MTX load_matrix(const char *filename, int enable_validation = 0)
{
    CSR_MTX m{0, 0, 0, nullptr, nullptr, nullptr};
    hspmm_csr c;
    if (hspmm_mtx_load(filename, HSPMM_BUILD_DTYPE, &c) != HSPMM_OK) {
        std::printf("error: %s\n", hspmm_last_error());
        return m;
    }
    m.rows = c.rows; m.cols = c.cols; m.nnzs = c.nnzs;
    m.row_ptr = c.row_ptr; m.col_idx = c.col_idx; m.values = static_cast<MAT_VAL_TYPE *>(c.values);
    if (enable_validation) {
        int bad = (m.row_ptr[0] != 0) + (m.row_ptr[m.rows] != m.nnzs);
        for (vint i = 0; i < m.rows; ++i) bad += m.row_ptr[i] > m.row_ptr[i + 1];
        for (vint i = 0; i < m.nnzs; ++i) bad += m.col_idx[i] >= m.cols;
        std::printf(bad ? "CSR validation failed: %d violations\n" : "CSR validation passed\n", bad);
    }
    std::printf("loaded matrix: %u x %u, %u stored entries\n", m.rows, m.cols, m.nnzs);
    return m;
}

inline void free_csr_matrix(CSR_MTX *m)
{
    if (!m) return;
    hspmm_csr c{m->rows, m->cols, m->nnzs, m->row_ptr, m->col_idx, m->values};
    hspmm_csr_free(&c);
    *m = CSR_MTX{0, 0, 0, nullptr, nullptr, nullptr};
}

inline void CSR2BTCFNOBITMAP(const CSR_MTX &csr, BTCF_MTX_NO_BITMAP &btcf)
{
    btcf.rows = csr.rows; btcf.cols = csr.cols; btcf.nnzs = csr.nnzs;
    btcf.total_row_windows = (csr.rows + ROW_WINDOW - 1) / ROW_WINDOW;
    uint32_t W = 0, T = 0;
    static const MAT_PTR_TYPE zero_ptr[1] = {0};
    const MAT_PTR_TYPE *rp = csr.row_ptr ? csr.row_ptr : zero_ptr;
    if (hspmm_btcf_sizes_cw(HSPMM_BUILD_DTYPE, COL_WINDOW, csr.rows, rp, csr.col_idx, &W, &T) != HSPMM_OK)
        hspmm_cpp::die("CSR2BTCFNOBITMAP");
    btcf.rowOffset.assign(size_t(W) + 1, 0);
    btcf.tcA2B.assign(size_t(T) * COL_WINDOW, 0);
    btcf.data.assign(size_t(T) * ROW_WINDOW * COL_WINDOW, MAT_VAL_TYPE(0.0f));
    btcf.rowIdx.assign(W, 0);
#ifdef SPARSE_A_TRANSPOSE
    const int transpose = 1;
#else
    const int transpose = 0;
#endif
    if (hspmm_btcf_fill_cw(HSPMM_BUILD_DTYPE, COL_WINDOW, csr.rows, rp, csr.col_idx, csr.values, transpose,
                           btcf.rowOffset.data(), btcf.tcA2B.data(), btcf.data.data(), btcf.rowIdx.data()) != HSPMM_OK)
        hspmm_cpp::die("CSR2BTCFNOBITMAP");
    btcf.eff_row_windows = W;
    btcf.total_tiles = T;
    std::printf("CSR -> condensed tiles: %u effective row windows, %u tiles of %d x %d\n", W, T, ROW_WINDOW, COL_WINDOW);
}

// CSR2BTCF of the reference (src/utils/convert.h:22-139).
inline void CSR2BTCF(const CSR_MTX &csr, BTCF_MTX &btcf)
{
#ifdef MMA_M16N8K4
    // (the library's bitmap tiles are 8 x 8 words of 64 bits; the 32-bit words of 8 x 4 tiles have no kernel)
    std::fprintf(stderr, "CSR2BTCF: bitmap tiles of 8 x 4 (-DMMA_M16N8K4) are not supported; use CSR2BTCFNOBITMAP\n");
    std::exit(EXIT_FAILURE);
#endif
    btcf.rows = csr.rows; btcf.cols = csr.cols; btcf.nnzs = csr.nnzs;
    btcf.total_row_windows = (csr.rows + ROW_WINDOW - 1) / ROW_WINDOW;
    uint32_t W = 0, T = 0, S = 0;
    static const MAT_PTR_TYPE zero_ptr[1] = {0};
    const MAT_PTR_TYPE *rp = csr.row_ptr ? csr.row_ptr : zero_ptr;
    if (hspmm_bitmap_sizes(HSPMM_BUILD_DTYPE, csr.rows, rp, csr.col_idx, &W, &T, &S) != HSPMM_OK)
        hspmm_cpp::die("CSR2BTCF");
    btcf.rowOffset.assign(size_t(W) + 1, 0);
    btcf.nnzOffset.assign(size_t(T) + 1, 0);
    btcf.tcA2B.assign(size_t(T) * COL_WINDOW, 0);
    btcf.tcBit.assign(size_t(T) * HSPMM_BITMAP_WORDS(HSPMM_BUILD_DTYPE), 0);
    btcf.data.assign(S, MAT_VAL_TYPE(0.0f));
    btcf.rowIdx.assign(W, 0);
#ifdef SPARSE_A_TRANSPOSE
    const int transpose = 1;
#else
    const int transpose = 0;
#endif
    if (hspmm_bitmap_fill(HSPMM_BUILD_DTYPE, csr.rows, rp, csr.col_idx, csr.values, transpose, HSPMM_BITS_PER_TILE,
                          btcf.rowOffset.data(), btcf.nnzOffset.data(), btcf.tcA2B.data(), btcf.tcBit.data(),
                          btcf.data.data(), btcf.rowIdx.data()) != HSPMM_OK)
        hspmm_cpp::die("CSR2BTCF");
    btcf.eff_row_windows = W;
    std::printf("CSR -> bitmap tiles: %u effective row windows, %u tiles, %u stored entries\n", W, T, S);
}

// BTCF2GBTCF of the reference (src/utils/convert.h:232-276).
inline void BTCF2GBTCF(BTCF_MTX &btcf, GBTCF_MTX &gbtcf)
{
    uint32_t tgl = 0, groups = 0;
    if (hspmm_group_sizes(btcf.eff_row_windows, btcf.rowOffset.data(), 32, &tgl, &groups) != HSPMM_OK)
        hspmm_cpp::die("BTCF2GBTCF");
    std::printf("tgl : %u\n", tgl);
    gbtcf.groupOffset.assign(size_t(groups) + 1, 0);
    gbtcf.rowIdx.assign(groups, 0);
    gbtcf.atomic.assign(groups, 0);
    if (hspmm_group_fill(btcf.eff_row_windows, btcf.rowOffset.data(), btcf.rowIdx.data(), tgl, gbtcf.groupOffset.data(),
                         gbtcf.rowIdx.data(), gbtcf.atomic.data()) != HSPMM_OK)
        hspmm_cpp::die("BTCF2GBTCF");
    std::printf("total groups : %u\n", groups);
    gbtcf.total_groups = groups;
    gbtcf.rows = btcf.rows; gbtcf.cols = btcf.cols; gbtcf.nnzs = btcf.nnzs;
    gbtcf.total_row_windows = groups + 1;          // groupOffset.size(), as the reference sets both (convert.h:267-268)
    gbtcf.eff_row_windows = groups + 1;
    gbtcf.nnzOffset = btcf.nnzOffset; gbtcf.tcA2B = btcf.tcA2B; gbtcf.tcBit = btcf.tcBit; gbtcf.data = btcf.data;
}

// The groups of the library's own balanced partition instead of the reference's
// fixed group length (src/utils/convert.h:242-258): a plan is made from the bitmap
// tiles, every piece of a window that one wave of its kernels walks becomes a group
// (GBTCF_MTX, src/utils/class.h:93-108), windows cut across waves are marked atomic.
// Needs the GPU the plan is made for; the result is a matrix like BTCF2GBTCF's.
inline void BTCF2GBTCF_balanced(BTCF_MTX &btcf, GBTCF_MTX &gbtcf)
{
#ifdef SPARSE_A_TRANSPOSE
    hspmm_cpp::die("BTCF2GBTCF_balanced with -DSPARSE_A_TRANSPOSE");
#endif
    const uint32_t tiles = btcf.rowOffset.empty() ? 0u : btcf.rowOffset.back();
    hspmm_plan *plan = nullptr;
    if (hspmm_create_bitmap(&plan, HSPMM_BUILD_DTYPE, btcf.rows, btcf.cols, btcf.eff_row_windows, tiles, btcf.rowOffset.data(),
                            btcf.nnzOffset.data(), btcf.tcA2B.data(), btcf.tcBit.data(), btcf.data.data(),
                            btcf.rowIdx.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_create_bitmap");
    uint32_t groups = 0;
    if (hspmm_partition_as_groups(plan, 0, &groups, nullptr, nullptr, nullptr) != HSPMM_OK)
        hspmm_cpp::die("hspmm_partition_as_groups");
    gbtcf.groupOffset.assign(size_t(groups) + 1, 0);
    gbtcf.rowIdx.assign(groups, 0);
    gbtcf.atomic.assign(groups, 0);
    if (hspmm_partition_as_groups(plan, groups, &groups, gbtcf.groupOffset.data(), gbtcf.rowIdx.data(),
                                  gbtcf.atomic.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_partition_as_groups");
    hspmm_destroy(plan);
    std::printf("total groups : %u\n", groups);
    gbtcf.total_groups = groups;
    gbtcf.rows = btcf.rows; gbtcf.cols = btcf.cols; gbtcf.nnzs = btcf.nnzs;
    gbtcf.total_row_windows = groups + 1;
    gbtcf.eff_row_windows = groups + 1;
    gbtcf.nnzOffset = btcf.nnzOffset; gbtcf.tcA2B = btcf.tcA2B; gbtcf.tcBit = btcf.tcBit; gbtcf.data = btcf.data;
}

// The checks of the reference's validateBTCF2GBTCFConversion (src/utils/convert.h:283-402)
// with the group count of every window derived from the converter's own group
// length; the reference's check still assumes a fixed length of 4 tiles
// (convert.h:317-318) and rejects every real conversion.
inline bool validateBTCF2GBTCFConversion(const BTCF_MTX &btcf, const GBTCF_MTX &gbtcf)
{
    if (btcf.rows != gbtcf.rows || btcf.cols != gbtcf.cols || btcf.nnzs != gbtcf.nnzs) return false;
    if (gbtcf.groupOffset.size() != size_t(gbtcf.total_groups) + 1) return false;
    if (gbtcf.atomic.size() != gbtcf.total_groups || gbtcf.rowIdx.size() != gbtcf.total_groups) return false;
    for (size_t i = 0; i + 1 < gbtcf.groupOffset.size(); ++i)
        if (gbtcf.groupOffset[i] >= gbtcf.groupOffset[i + 1]) return false;
    uint32_t tgl = 0, groups = 0;
    if (hspmm_group_sizes(btcf.eff_row_windows, btcf.rowOffset.data(), 32, &tgl, &groups) != HSPMM_OK) return false;
    if (groups != gbtcf.total_groups) return false;
    size_t g = 0;
    for (vint w = 0; w < btcf.eff_row_windows; ++w) {
        const vint n = btcf.rowOffset[w + 1] - btcf.rowOffset[w];
        const vint expected = (n + tgl - 1) / tgl;
        if (gbtcf.groupOffset[g] != btcf.rowOffset[w]) return false;
        for (vint j = 0; j < expected; ++j, ++g) {
            if (gbtcf.rowIdx[g] != btcf.rowIdx[w] || gbtcf.atomic[g] != (expected > 1)) return false;
            if (gbtcf.groupOffset[g + 1] > btcf.rowOffset[w + 1]) return false;
        }
        if (gbtcf.groupOffset[g] != btcf.rowOffset[w + 1]) return false;
    }
    return gbtcf.nnzOffset == btcf.nnzOffset && gbtcf.tcA2B == btcf.tcA2B && gbtcf.tcBit == btcf.tcBit &&
           gbtcf.data.size() == btcf.data.size() &&
           std::memcmp(gbtcf.data.data(), btcf.data.data(), btcf.data.size() * sizeof(MAT_VAL_TYPE)) == 0;
}

// The reference's singleton of launch knobs; here they reach the library.
class Scheduler {
    int BUFFER_STAGE = 0, CONSUMER_WARP_NUM = 0, PRODUCER_WARP_GROUP_NUM = 0, SM_NUM = 0;
    Scheduler() = default;
    Scheduler(const Scheduler &) = delete;
    Scheduler &operator=(const Scheduler &) = delete;
    void push() const
    {
        if (hspmm_configure(BUFFER_STAGE, CONSUMER_WARP_NUM, PRODUCER_WARP_GROUP_NUM, SM_NUM) != HSPMM_OK)
            hspmm_cpp::die("Scheduler");
    }

public:
    static Scheduler &getInstance()
    {
        static Scheduler instance;
        return instance;
    }
    void setBufferStage(int v) { BUFFER_STAGE = v; push(); }
    int getBufferStage() const { return BUFFER_STAGE; }
    void setConsumerWarpNum(int v) { CONSUMER_WARP_NUM = v; push(); }
    int getConsumerWarpNum() const { return CONSUMER_WARP_NUM; }
    void configure(int buffer_stage, int consumer_warp_num, int producer_warp_group_num, int sm_num)
    {
        BUFFER_STAGE = buffer_stage; CONSUMER_WARP_NUM = consumer_warp_num;
        PRODUCER_WARP_GROUP_NUM = producer_warp_group_num; SM_NUM = sm_num;
        push();
    }
    int getSMNum() const { return SM_NUM; }
};

// C = A * B on the GPU: uploads, WARMUP_RUNS untimed and RUNS timed launches
// (src/common.h:48-49), downloads C into dense_c.values.
namespace hspmm_cpp {
inline void check_shapes(vint a_rows, vint a_cols, const DENSE_MTX &dense_b, const DENSE_MTX &dense_c)
{
    if (dense_b.rows != a_cols || dense_c.rows != a_rows || dense_c.cols != dense_b.cols) {
        std::fprintf(stderr, "spmm: shapes do not match: A %u x %u, B %u x %u, C %u x %u\n", a_rows, a_cols,
                     dense_b.rows, dense_b.cols, dense_c.rows, dense_c.cols);
        std::exit(EXIT_FAILURE);
    }
}
inline PERF_RESULT run_plan(hspmm_plan *plan, DENSE_MTX &dense_b, DENSE_MTX &dense_c);
class PageToucher;
}  // namespace hspmm_cpp

inline PERF_RESULT hspmm_cpp_spmm(BTCF_MTX_NO_BITMAP &a, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    hspmm_cpp::check_shapes(a.rows, a.cols, dense_b, dense_c);
    hspmm_plan *plan = nullptr;
    // (the tile order of -DSPARSE_A_TRANSPOSE, which the converters above honour, goes through the layout entry)
#ifdef SPARSE_A_TRANSPOSE
    constexpr int transposed = 1;
#else
    constexpr int transposed = 0;
#endif
    if (hspmm_create_layout(&plan, HSPMM_BUILD_DTYPE, COL_WINDOW, transposed, a.rows, a.cols, a.eff_row_windows, a.total_tiles,
                            a.rowOffset.data(), a.tcA2B.data(), a.data.data(), a.rowIdx.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_create_layout");
    return hspmm_cpp::run_plan(plan, dense_b, dense_c);
}

// The same operator for a matrix held as bitmap tiles or as groups; the
// reference has no kernel for either format.
inline PERF_RESULT hspmm_cpp_spmm(BTCF_MTX &a, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    hspmm_cpp::check_shapes(a.rows, a.cols, dense_b, dense_c);
    hspmm_plan *plan = nullptr;
    const uint32_t tiles = a.rowOffset.empty() ? 0u : a.rowOffset.back();
#ifdef SPARSE_A_TRANSPOSE
    // bit k * 8 + r, stored entries column by column (convert.h:88-90, 120-126): expanded, these are transposed tiles
    std::vector<MAT_VAL_TYPE> dense(size_t(tiles) * ROW_WINDOW * COL_WINDOW);
    if (hspmm_bitmap_expand(HSPMM_BUILD_DTYPE, tiles, a.nnzOffset.data(), a.tcBit.data(), a.data.data(), dense.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_bitmap_expand");
    if (hspmm_create_layout(&plan, HSPMM_BUILD_DTYPE, COL_WINDOW, 1, a.rows, a.cols, a.eff_row_windows, tiles, a.rowOffset.data(),
                            a.tcA2B.data(), dense.data(), a.rowIdx.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_create_layout");
    return hspmm_cpp::run_plan(plan, dense_b, dense_c);
#endif
    if (hspmm_create_bitmap(&plan, HSPMM_BUILD_DTYPE, a.rows, a.cols, a.eff_row_windows, tiles, a.rowOffset.data(),
                            a.nnzOffset.data(), a.tcA2B.data(), a.tcBit.data(), a.data.data(),
                            a.rowIdx.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_create_bitmap");
    return hspmm_cpp::run_plan(plan, dense_b, dense_c);
}

inline PERF_RESULT hspmm_cpp_spmm(GBTCF_MTX &a, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    hspmm_cpp::check_shapes(a.rows, a.cols, dense_b, dense_c);
    hspmm_plan *plan = nullptr;
#ifdef SPARSE_A_TRANSPOSE
    std::fprintf(stderr, "hspmm: groups of transposed bitmap tiles (-DSPARSE_A_TRANSPOSE) are not accepted; use BTCF_MTX\n");
    std::exit(1);
#endif
    if (hspmm_create_grouped(&plan, HSPMM_BUILD_DTYPE, a.rows, a.cols, a.total_groups, a.groupOffset.data(),
                             a.nnzOffset.data(), a.tcA2B.data(), a.tcBit.data(), a.data.data(), a.rowIdx.data(),
                             a.atomic.data()) != HSPMM_OK)
        hspmm_cpp::die("hspmm_create_grouped");
    return hspmm_cpp::run_plan(plan, dense_b, dense_c);
}

// Writes one byte into every page of a buffer on worker threads, so that the pages of a freshly
// allocated result matrix exist before the copy from the device lands in them (a copy into
// untouched pages takes its page faults one by one: 78 ms instead of 15 ms for 268 MB).
class hspmm_cpp::PageToucher {
public:
    PageToucher(void *buffer, size_t bytes)
    {
        const size_t page = 4096;
        unsigned n = std::thread::hardware_concurrency();
        n = n < 1 ? 1 : n > 16 ? 16 : n;
        if (bytes < (size_t(8) << 20)) return;                 // small results: not worth a thread
        const size_t per = ((bytes + n - 1) / n + page - 1) / page * page;
        char *p = static_cast<char *>(buffer);
        for (unsigned t = 0; t < n; ++t)
            workers_.emplace_back([=] {
                for (size_t i = size_t(t) * per; i < bytes && i < size_t(t + 1) * per; i += page)
                    static_cast<volatile char *>(p)[i] = 0;
            });
    }
    void wait()
    {
        for (std::thread &w : workers_) w.join();
        workers_.clear();
    }
    ~PageToucher() { wait(); }
private:
    std::vector<std::thread> workers_;
};

inline PERF_RESULT hspmm_cpp::run_plan(hspmm_plan *plan, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    PERF_RESULT perf{0.0f, RUNS};
    const size_t b_bytes = size_t(dense_b.rows) * dense_b.cols * sizeof(MAT_VAL_TYPE);
    const size_t c_bytes = size_t(dense_c.rows) * dense_c.cols * sizeof(MAT_VAL_TYPE);
    hspmm_cpp::PageToucher touch_c(dense_c.values, c_bytes);   // while B goes up and the GPU works
    void *d_b = nullptr, *d_c = nullptr;
    hspmm_cpp::check_hip(hipMalloc(&d_b, b_bytes ? b_bytes : 4), "hipMalloc B");
    hspmm_cpp::check_hip(hipMalloc(&d_c, c_bytes ? c_bytes : 4), "hipMalloc C");
    hspmm_cpp::check_hip(hipMemcpy(d_b, dense_b.values, b_bytes, hipMemcpyHostToDevice), "copy B");
    if (dense_c.cols && hspmm_bench(plan, d_b, d_c, dense_c.cols, WARMUP_RUNS, RUNS, nullptr, &perf.time) != HSPMM_OK)
        hspmm_cpp::die("hspmm_bench");
    touch_c.wait();
    hspmm_cpp::check_hip(hipMemcpy(dense_c.values, d_c, c_bytes, hipMemcpyDeviceToHost), "copy C");
    hspmm_cpp::check_hip(hipFree(d_b), "hipFree");
    hspmm_cpp::check_hip(hipFree(d_c), "hipFree");
    hspmm_destroy(plan);
    return perf;
}

// With BTCF_MTX_NO_BITMAP this is the reference's signature; BTCF_MTX and
// GBTCF_MTX are accepted as well.
#if defined(USE_FP16)
template <class SPARSE_MTX>
inline PERF_RESULT fp16_spmm(SPARSE_MTX &btcf_a, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    return hspmm_cpp_spmm(btcf_a, dense_b, dense_c);
}
#elif defined(USE_BF16)
template <class SPARSE_MTX>
inline PERF_RESULT bf16_spmm(SPARSE_MTX &btcf_a, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    return hspmm_cpp_spmm(btcf_a, dense_b, dense_c);
}
#else
template <class SPARSE_MTX>
inline PERF_RESULT tf32_spmm(SPARSE_MTX &btcf_a, DENSE_MTX &dense_b, DENSE_MTX &dense_c)
{
    return hspmm_cpp_spmm(btcf_a, dense_b, dense_c);
}
#endif

// Element-wise comparison of two dense matrices.  The reference's helper counts
// |a - b| > 1 (src/utils/verify.h:28); here the bound is the relative / absolute
// form of its tile checks (src/tf32.cu:46-70): relative `tol` when |b| > 1e-6,
// absolute 1e-5 otherwise - plus, where the caller knows it, abs_tol x sum |a||b| of
// the element (what a sum that cancels may be off by: rounding errors scale with
// the terms, not with the result).
inline bool verify_dense_matrix(const DENSE_MTX *A, const DENSE_MTX *B, double tol = 1e-2,
                                const double *sum_abs = nullptr, double abs_tol = 0.0)
{
    const size_t total = size_t(A->rows) * A->cols;
    size_t failed = 0;
    int printed = 0;
    for (size_t i = 0; i < total; ++i) {
        const double a = double(A->values[i]), b = double(B->values[i]);
        const double err = std::fabs(a - b), ref = std::fabs(b);
        const double slack = sum_abs ? abs_tol * sum_abs[i] : 0.0;
        const bool bad = ref > 1e-6 ? !(err <= tol * ref + slack) : !(err <= 1e-5 + slack);
        if (bad) {
            ++failed;
            if (printed++ < 20)
                std::printf("mismatch at [%zu][%zu]: %g vs %g\n", i / A->cols, i % A->cols, a, b);
        }
    }
    if (failed) std::printf("verification: %zu of %zu elements differ (%.2f%%)\n", failed, total, 100.0 * failed / total);
    return failed == 0;
}
