// Command-line driver with the reference's arguments (reference src/fp16.cu:283-319):
//   fp16_test <matrix_file> <feature_dim> [--seed S] [--verify] [--format tiles|bitmap|grouped|balanced]
// built with -DUSE_FP16; the same source with -DUSE_TF32 / -DUSE_BF16 gives
// tf32_test / bf16_test.
// B is filled with rand() / RAND_MAX as in the reference (src/fp16.cu:303-309);
// --seed calls srand first (the reference never seeds, i.e. seed 1).  --verify
// fills in the reference's empty "verify" step (src/fp16.cu:317) with the check its
// test programs make (src/test_fp16.cu:284-315, src/tf32.cu:11-82): the product again
// on the host, C[i][j] += float(a) * float(b) in fp32 over the stored entries of row i
// in column order, compared element by element (1e-2 relative, 1e-3 for tf32_test,
// plus a term in sum |a||b| for sums that cancel).  The check only reads what the GPU
// wrote; nothing of it is ever returned as a result.
// --format hands the matrix to the operator as uncompressed tiles (the reference's
// only path, the default), as bitmap tiles (CSR2BTCF), as groups of the reference's
// fixed length (BTCF2GBTCF) or as the groups of the library's balanced partition.
#include <algorithm>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "hopper_spmm.hpp"

int main(int argc, char *argv[])
{
    if (argc < 3) {
        std::printf("Usage: %s <matrix_file> <feature_dim> [--seed S] [--verify] [--format tiles|bitmap|grouped|balanced]\n",
                    argv[0]);
        return 1;
    }
    const char *matrix_file = argv[1];
    const int fd = std::atoi(argv[2]);
    bool verify = false;
    std::string format = "tiles";
    for (int i = 3; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--verify")) verify = true;
        else if (!std::strcmp(argv[i], "--format") && i + 1 < argc) format = argv[++i];
        else if (!std::strcmp(argv[i], "--seed") && i + 1 < argc) std::srand(unsigned(std::atol(argv[++i])));
        else { std::printf("unknown argument %s\n", argv[i]); return 1; }
    }
    if (fd <= 0) { std::printf("feature_dim must be positive\n"); return 1; }
    if (format != "tiles" && format != "bitmap" && format != "grouped" && format != "balanced") {
        std::printf("unknown format %s\n", format.c_str());
        return 1;
    }
    const vint feature_dim = vint(fd);

    CSR_MTX csr = load_matrix(matrix_file, 0);
    if (!csr.row_ptr) return 1;                       // the reference carries on with an empty matrix
    BTCF_MTX_NO_BITMAP btcf;
    CSR2BTCFNOBITMAP(csr, btcf);
    std::printf("=== condensed tile matrix ===\n");
    std::printf("rows: %u\ncols: %u\nstored entries: %u\n", btcf.rows, btcf.cols, btcf.nnzs);
    std::printf("row windows: %u\nnon-empty row windows: %u\n", btcf.total_row_windows, btcf.eff_row_windows);
    std::printf("tiles (%d x %d): %zu\n", ROW_WINDOW, COL_WINDOW, btcf.tcA2B.size() / COL_WINDOW);

    DENSE_MTX dense_b{btcf.cols, feature_dim, new MAT_VAL_TYPE[size_t(btcf.cols) * feature_dim]};
    for (size_t i = 0; i < size_t(dense_b.rows) * dense_b.cols; ++i)
        dense_b.values[i] = MAT_VAL_TYPE(static_cast<float>(std::rand()) / static_cast<float>(RAND_MAX));
    DENSE_MTX dense_c{btcf.rows, feature_dim, new MAT_VAL_TYPE[size_t(btcf.rows) * feature_dim]};

#if defined(USE_FP16)
#define SPMM fp16_spmm
#elif defined(USE_BF16)
#define SPMM bf16_spmm
#else
#define SPMM tf32_spmm
#endif
    PERF_RESULT perf{0.0f, RUNS};
    if (format == "tiles") perf = SPMM(btcf, dense_b, dense_c);
    else {
        BTCF_MTX bitmap;
        CSR2BTCF(csr, bitmap);
        if (format == "bitmap") perf = SPMM(bitmap, dense_b, dense_c);
        else {
            GBTCF_MTX grouped;
            if (format == "balanced") BTCF2GBTCF_balanced(bitmap, grouped);
            else {
                BTCF2GBTCF(bitmap, grouped);
                if (!validateBTCF2GBTCFConversion(bitmap, grouped)) { std::printf("grouping failed its checks\n"); return 2; }
            }
            perf = SPMM(grouped, dense_b, dense_c);
        }
    }
    perf.print();
    const double t = perf.time / perf.runs * 1e-3;
    if (t > 0) std::printf("effective rate: %.3f TFLOP/s (2 * nnz * N / t)\n", 2.0 * btcf.nnzs * feature_dim / t / 1e12);

    int rc = 0;
    if (verify) {
        // the reference's check arithmetic on the host, rows dealt out over worker threads; with it
        // sum |a||b| per element: the scale of what the two results may differ by where a sum cancels
        // (fp32 accumulation in another order; for tf32_test also the products of bf16 parts)
        DENSE_MTX expected{btcf.rows, feature_dim, new MAT_VAL_TYPE[size_t(btcf.rows) * feature_dim]};
        std::vector<double> sum_abs(size_t(btcf.rows) * feature_dim, 0.0);
        unsigned workers = std::thread::hardware_concurrency();
        workers = workers < 1 ? 1 : workers > 16 ? 16 : workers;
        std::vector<std::thread> pool;
        for (unsigned w = 0; w < workers; ++w)
            pool.emplace_back([&, w] {
                std::vector<float> acc(feature_dim);
                for (vint r = w; r < csr.rows; r += workers) {
                    std::fill(acc.begin(), acc.end(), 0.0f);
                    double *srow = sum_abs.data() + size_t(r) * feature_dim;
                    for (MAT_PTR_TYPE i = csr.row_ptr[r]; i < csr.row_ptr[r + 1]; ++i) {
                        const float a = float(csr.values[i]);
                        const MAT_VAL_TYPE *brow = dense_b.values + size_t(csr.col_idx[i]) * feature_dim;
                        for (vint j = 0; j < feature_dim; ++j) {
                            const float b = float(brow[j]);
                            acc[j] += a * b;                                     // src/test_fp16.cu:292-297
                            srow[j] += std::fabs(double(a)) * std::fabs(double(b));
                        }
                    }
                    MAT_VAL_TYPE *erow = expected.values + size_t(r) * feature_dim;
                    for (vint j = 0; j < feature_dim; ++j) erow[j] = MAT_VAL_TYPE(acc[j]);
                }
            });
        for (std::thread &t : pool) t.join();
#if defined(USE_TF32)
        // the tf32 bound: 1e-3 relative; products of bf16 parts: 2^-16 of sum |a||b| more where a sum cancels
        const double rel_tol = 1e-3, abs_tol = 1e-5 + 1.0 / 65536.0;
#else
        const double rel_tol = 1e-2, abs_tol = 1e-5;
#endif
        const bool ok = verify_dense_matrix(&dense_c, &expected, rel_tol, sum_abs.data(), abs_tol);
        std::printf(ok ? "verification passed\n" : "verification FAILED\n");
        rc = ok ? 0 : 2;
        delete[] expected.values;
    }
    delete[] dense_b.values;
    delete[] dense_c.values;
    free_csr_matrix(&csr);
    return rc;
}
