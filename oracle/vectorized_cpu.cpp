// TEST / BASELINE INFRASTRUCTURE - NOT PART OF THE PRODUCT.
//
// Restatement of the reference's multithreaded vectorized CPU engine for dense row-split
// pipelines, used (a) as the checker for the fused device pipeline and (b) as the timed CPU
// baseline of the benchmark. It drives the kernels of daphne_cpu_oracle.cpp the way
// MTWrapper<DenseMatrix<VT>>::executeCpuQueues does
// (reference: src/runtime/local/vectorized/MTWrapper_dense.cpp:82-201):
//   * one task per worker under the default STATIC partitioning, ceil(rows / workers) rows each
//     (vectorized/LoadPartitioning.h:78-81, api/cli/DaphneUserConfig.h:93);
//   * every task walks its rows in batches of max(1, 96 KiB / bytes-per-row) rows
//     (MTWrapper_dense.cpp:113, DaphneUserConfig.h:103) and calls the pipeline body - one kernel
//     call per operator, every intermediate materialised - on each batch
//     (vectorized/Tasks.cpp:22-49);
//   * ROWS outputs are copied into the result slice, ADD outputs are accumulated per task and
//     combined into the shared result under one mutex (Tasks.cpp:51-160).
// Operators that are not vectorizable in the reference (colMeans / colVars: only column SUM / MIN /
// MAX implement the interface, ir/daphneir/DaphneVectorizableOpInterface.cpp:345-350) run as one
// single-threaded kernel call over the whole matrix, as they would in the reference.
#include <algorithm>
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

extern "C" {
int oracle_ew_binary_f32(int op, float *res, size_t ld_res, const float *lhs, size_t lr, size_t lc, size_t ld_lhs,
                         const float *rhs, size_t rr, size_t rc, size_t ld_rhs);
int oracle_ew_binary_sca_f32(int op, float *res, size_t ld_res, const float *lhs, size_t rows, size_t cols,
                             size_t ld_lhs, float rhs);
int oracle_ew_unary_f32(int op, float *res, size_t ld_res, const float *arg, size_t rows, size_t cols, size_t ld_arg);
int oracle_agg_all_f32(int op, const float *arg, size_t rows, size_t cols, size_t ld, float *out);
int oracle_agg_row_f32(int op, float *res, size_t ld_res, const float *arg, size_t rows, size_t cols, size_t ld);
int oracle_agg_col_f32(int op, float *res, const float *arg, size_t rows, size_t cols, size_t ld);
}

namespace {
enum { B_ADD = 0, B_SUB = 1, B_MUL = 2, B_DIV = 3, B_GT = 11 };
enum { A_SUM = 0, A_MEAN = 6, A_VAR = 8 };
enum { U_SQRT = 3 };
using clk = std::chrono::steady_clock;
double secs(clk::time_point a, clk::time_point b) { return std::chrono::duration<double>(b - a).count(); }
} // namespace

// Z-score-then-reduce pipeline on X (rows x cols, contiguous):
//   mu = colMeans(X); sd = sqrt(colVars(X)); Z = (X - mu) / sd; r = rowSums(Z * Z); s = sum(r > thr)
// mu, sd: cols values; r: rows values; s: one value. Returns 0. seconds[0] = column statistics
// (single-threaded), seconds[1] = the vectorized pipeline on `threads` workers.
extern "C" int oracle_zscore_pipeline_f32(const float *X, size_t rows, size_t cols, int threads, float thr, float *mu,
                                          float *sd, float *r, float *s, double *seconds) {
    const auto t0 = clk::now();
    oracle_agg_col_f32(A_MEAN, mu, X, rows, cols, cols);
    std::vector<float> var(cols);
    oracle_agg_col_f32(A_VAR, var.data(), X, rows, cols, cols);
    oracle_ew_unary_f32(U_SQRT, sd, cols, var.data(), 1, cols, cols);
    const auto t1 = clk::now();

    if (threads < 1)
        threads = 1;
    const size_t row_mem = cols * sizeof(float);
    const size_t batch = std::max<size_t>(1, (96 * 1024) / row_mem);
    const size_t chunk = (rows + threads - 1) / threads; // STATIC: one task per worker
    std::mutex res_lock;
    float total = 0.0f;
    bool total_set = false;
    auto worker = [&](size_t lo, size_t hi) {
        float local = 0.0f;
        bool local_set = false;
        for (size_t b0 = lo; b0 < hi; b0 += batch) {
            const size_t nb = std::min(batch, hi - b0);
            const float *xb = X + b0 * cols;
            // one kernel call per operator, each producing a fresh intermediate
            std::vector<float> t1v(nb * cols), t2v(nb * cols), t3v(nb * cols), rr(nb), gt(nb);
            oracle_ew_binary_f32(B_SUB, t1v.data(), cols, xb, nb, cols, cols, mu, 1, cols, cols);
            oracle_ew_binary_f32(B_DIV, t2v.data(), cols, t1v.data(), nb, cols, cols, sd, 1, cols, cols);
            oracle_ew_binary_f32(B_MUL, t3v.data(), cols, t2v.data(), nb, cols, cols, t2v.data(), nb, cols, cols);
            oracle_agg_row_f32(A_SUM, rr.data(), 1, t3v.data(), nb, cols, cols);
            oracle_ew_binary_sca_f32(B_GT, gt.data(), 1, rr.data(), nb, 1, 1, thr);
            float part = 0.0f;
            oracle_agg_all_f32(A_SUM, gt.data(), nb, 1, 1, &part);
            std::memcpy(r + b0, rr.data(), nb * sizeof(float)); // combine ROWS
            if (local_set)
                local = local + part; // combine ADD, task-local
            else {
                local = part;
                local_set = true;
            }
        }
        if (local_set) {
            std::lock_guard<std::mutex> g(res_lock);
            if (total_set)
                total = total + local;
            else {
                total = local;
                total_set = true;
            }
        }
    };
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; t++) {
        const size_t lo = std::min(rows, static_cast<size_t>(t) * chunk), hi = std::min(rows, lo + chunk);
        if (lo < hi)
            pool.emplace_back(worker, lo, hi);
    }
    for (auto &th : pool)
        th.join();
    const auto t2 = clk::now();
    *s = total;
    if (seconds) {
        seconds[0] = secs(t0, t1);
        seconds[1] = secs(t1, t2);
    }
    return 0;
}
