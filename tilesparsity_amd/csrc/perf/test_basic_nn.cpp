// Perf driver of the TW GEMM engine with the command line of the reference's
// StreamMaskedGEMM/perf/basic_nn.cu:
//
//     test_basic_nn <M> <N> <K> <N_pruned> <K_pruned> [--bf16] [--iters I] [--seed S]
//
// (<N_pruned>/<K_pruned> are the KEPT sizes, as in the reference.)  It draws the same
// inputs the reference draws (glibc rand(), never seeded unless --seed; init_matrix A, B,
// then per tile mask_gen(K) and mask_gen(N_ori), basic_nn.cu:822-825, 891-903), builds the
// masked-dense and the compacted stream weight, then
//   * times the dense baseline: the same kernel on an all-kept plan over B (.) mask
//     (role of Cutlass_Gemm_NN, :315-375), printed as "Dense   GEMM : %f us."
//   * times the TW GEMM through tw_gemm (role of Stream_Gemm_NN, :378-445), printed as
//     "Stream  GEMM : %f us."  -- both also in the reference's protocol (a device-wide
//     synchronise after every launch, :408-430) as "... (sync each) : %f us."
//   * runs the gather -> dense GEMM -> scatter form (Stream_Gemm_NN_reference, :450-503)
//     with the engine's deleteRow / insertRow kernels,
// and checks them against each other and against a host fp32 product: the first pair must be
// identical under the reference's checkout rule (:771-798, err 1e-10 as at :1074,:1081); the
// others pass on max relative error <= 1e-2 (fp16) / 2e-2 (bf16).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "twgemm.h"

#define CHECK_TW(call)                                                                   \
    do {                                                                                 \
        int st_ = (call);                                                                \
        if (st_ != TW_OK) {                                                              \
            fprintf(stderr, "%s failed: %s (%s)\n", #call, tw_status_string(st_),        \
                    tw_last_error());                                                    \
            return 1;                                                                    \
        }                                                                                \
    } while (0)
#define CHECK_HIP(call)                                                                  \
    do {                                                                                 \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess) {                                                          \
            fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));            \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

static const int N_dim = 128; // kept columns per tile, basic_nn.cu:73

// value stream of the reference: U(-0.5, 0.5) from rand(), basic_nn.cu:612-621
static void init_matrix(std::vector<float> &mat)
{
    for (float &v : mat)
        v = (float)((double)rand() / (double)RAND_MAX - 0.5);
}

// kept-index list of the reference: shuffle 0..n-1 with rand(), keep the first n_kept,
// sort, store kept[i] - i  (basic_nn.cu:697-718)
static std::vector<int32_t> mask_gen(int n, int n_kept)
{
    std::vector<int32_t> perm(n);
    for (int i = 0; i < n; ++i)
        perm[i] = i;
    for (int i = 1; i < n; ++i) // the loop std::random_shuffle runs without a generator
        std::swap(perm[i], perm[rand() % (i + 1)]);
    std::sort(perm.begin(), perm.begin() + n_kept);
    std::vector<int32_t> rel(n_kept);
    for (int i = 0; i < n_kept; ++i)
        rel[i] = perm[i] - i;
    return rel;
}

static uint16_t to_bits(float f, int dtype)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    if (dtype == TW_BF16) {
        x += 0x7FFFu + ((x >> 16) & 1u);
        return (uint16_t)(x >> 16);
    }
    _Float16 h = (_Float16)f;
    uint16_t b;
    memcpy(&b, &h, 2);
    return b;
}

static float from_bits(uint16_t b, int dtype)
{
    if (dtype == TW_BF16) {
        uint32_t x = (uint32_t)b << 16;
        float f;
        memcpy(&f, &x, 4);
        return f;
    }
    _Float16 h;
    memcpy(&h, &b, 2);
    return (float)h;
}

// Number of elements the reference's acceptance rule rejects (basic_nn.cu:771-798):
// v1/v2 > 1+err || v2/v1 > 1+err || |v2-v1| > err; 0/0 is NaN and passes, as there.
static long rule_errors(const std::vector<float> &a, const std::vector<float> &b, double err)
{
    long errors = 0;
    for (size_t i = 0; i < a.size(); ++i) {
        float v1 = b[i], v2 = a[i];
        if (v1 / v2 > (1 + err) || v2 / v1 > (1 + err) || std::fabs(v2 - v1) > err)
            ++errors;
    }
    return errors;
}

// exact == true: the reference's rule with err 1e-10 must reject nothing (bit-identical
// results).  Otherwise the pass criterion is max |a-b| / max(|b|, 1e-2 rms(b)) <= tol; the
// count under the reference's ratio rule is printed for information (it also rejects
// near-zero outputs whose fp32 summation order differs).
static long checkout(const std::vector<float> &a, const std::vector<float> &b, double tol, bool exact)
{
    if (exact) {
        long errors = rule_errors(a, b, 1e-10);
        if (errors)
            fprintf(stderr, "results differ. Errors : %ld / %zu\n\n", errors, a.size());
        else
            fprintf(stderr, "PASSED !!!\n\n");
        return errors;
    }
    double ss = 0;
    for (float v : b)
        ss += (double)v * v;
    const double floor_ = 1e-2 * std::sqrt(ss / std::max<size_t>(b.size(), 1)) + 1e-30;
    double worst = 0;
    for (size_t i = 0; i < a.size(); ++i)
        worst = std::max(worst, std::fabs((double)a[i] - b[i]) / std::max((double)std::fabs(b[i]), floor_));
    fprintf(stderr, "max relative error %.3g (tolerance %.0e); reference rule rejects %ld / %zu\n",
            worst, tol, rule_errors(a, b, tol), a.size());
    if (worst <= tol) {
        fprintf(stderr, "PASSED !!!\n\n");
        return 0;
    }
    fprintf(stderr, "results incorrect.\n\n");
    return 1;
}

template <typename F> static int time_us(F launch, int iters, bool sync_each, float *us)
{
    hipEvent_t t0, t1;
    CHECK_HIP(hipEventCreate(&t0));
    CHECK_HIP(hipEventCreate(&t1));
    for (int i = 0; i < 5; ++i)
        if (launch())
            return 1;
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipEventRecord(t0, nullptr));
    for (int i = 0; i < iters; ++i) {
        if (launch())
            return 1;
        if (sync_each)
            CHECK_HIP(hipDeviceSynchronize());
    }
    CHECK_HIP(hipEventRecord(t1, nullptr));
    CHECK_HIP(hipEventSynchronize(t1));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, t0, t1));
    *us = ms * 1000.0f / iters;
    hipEventDestroy(t0);
    hipEventDestroy(t1);
    return 0;
}

int main(int argc, const char *argv[])
{
    int problem[5] = {768, 768, 768, 768, 768};
    int dtype = TW_F16, iters = 100, npos = 0;
    long seed = -1;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--bf16")
            dtype = TW_BF16;
        else if (a == "--iters" && i + 1 < argc)
            iters = atoi(argv[++i]);
        else if (a == "--seed" && i + 1 < argc)
            seed = atol(argv[++i]);
        else if (npos < 5)
            problem[npos++] = (atoi(argv[i]) + 7) / 8 * 8; // multiples of 8, basic_nn.cu:1156-1157
    }
    const int M = problem[0], N = problem[1], K = problem[2];
    const int N_pruned = problem[3], K_pruned = problem[4];
    if (seed >= 0)
        srand((unsigned)seed);

    std::vector<float> hA((size_t)M * K), hB((size_t)K * N);
    init_matrix(hA);
    init_matrix(hB);

    int block_num = 0;
    const int max_tiles = (N_pruned + N_dim - 1) / N_dim + 1;
    std::vector<int32_t> N_ori(max_tiles), N_cal(max_tiles), K_cal(max_tiles);
    std::vector<int64_t> off_B(max_tiles), off_C(max_tiles);
    CHECK_TW(tw_tile_partition(M, N, K, N_pruned, K_pruned, N_dim, max_tiles, &block_num,
                               N_ori.data(), N_cal.data(), K_cal.data(), off_B.data(),
                               off_C.data()));

    // per tile: relative offsets, kept lists, and the masked-dense weight B (.) mask
    std::vector<int32_t> col0(block_num), kp(block_num + 1, 0), np(block_num + 1, 0), ki, ni;
    std::vector<std::vector<int32_t>> rel_k(block_num), rel_n(block_num);
    std::vector<float> hB_pruned((size_t)K * N, 0.0f);
    for (int t = 0; t < block_num; ++t) {
        col0[t] = (int32_t)(off_C[t] / std::max(M, 1));
        rel_k[t] = mask_gen(K, K_cal[t]);
        rel_n[t] = mask_gen(N_ori[t], N_cal[t]);
        for (int i = 0; i < K_cal[t]; ++i)
            ki.push_back(rel_k[t][i] + i);
        for (int j = 0; j < N_cal[t]; ++j)
            ni.push_back(rel_n[t][j] + j);
        kp[t + 1] = (int32_t)ki.size();
        np[t + 1] = (int32_t)ni.size();
        for (int i = 0; i < K_cal[t]; ++i) // gen_cutlass_weight, basic_nn.cu:743-755
            for (int j = 0; j < N_cal[t]; ++j) {
                size_t idx = (size_t)(rel_k[t][i] + i) * N + rel_n[t][j] + j + col0[t];
                hB_pruned[idx] = hB[idx];
            }
    }

    tw_plan *stream_plan = nullptr, *dense_plan = nullptr;
    CHECK_TW(tw_plan_create(K, N, dtype, block_num, col0.data(), N_ori.data(), kp.data(), ki.data(),
                            np.data(), ni.data(), hB.data(), &stream_plan));
    CHECK_TW(tw_plan_create_dense(K, N, N_dim, dtype, hB_pruned.data(), &dense_plan));

    // device operands in the reference's layouts: A column-major M x K, C column-major M x N
    std::vector<uint16_t> hAt((size_t)K * M);
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k)
            hAt[(size_t)k * M + m] = to_bits(hA[(size_t)m * K + k], dtype);
    uint16_t *dA = nullptr, *dC_dense = nullptr, *dC_stream = nullptr, *dC_ref = nullptr;
    const size_t a_bytes = (size_t)K * M * 2, c_bytes = (size_t)N * M * 2;
    CHECK_HIP(hipMalloc((void **)&dA, a_bytes));
    CHECK_HIP(hipMalloc((void **)&dC_dense, c_bytes));
    CHECK_HIP(hipMalloc((void **)&dC_stream, c_bytes));
    CHECK_HIP(hipMalloc((void **)&dC_ref, c_bytes));
    CHECK_HIP(hipMemcpy(dA, hAt.data(), a_bytes, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemset(dC_dense, 0, c_bytes));
    CHECK_HIP(hipMemset(dC_stream, 0, c_bytes));
    CHECK_HIP(hipMemset(dC_ref, 0, c_bytes));

    auto run_dense = [&]() {
        return tw_gemm(dense_plan, dA, TW_LAYOUT_KMAJOR, M, dC_dense, TW_LAYOUT_KMAJOR, M, M, 1.0f,
                       0.0f, TW_PRUNED_UNTOUCHED, nullptr);
    };
    auto run_stream = [&]() {
        return tw_gemm(stream_plan, dA, TW_LAYOUT_KMAJOR, M, dC_stream, TW_LAYOUT_KMAJOR, M, M,
                       1.0f, 0.0f, TW_PRUNED_UNTOUCHED, nullptr);
    };
    float us = 0;
    if (time_us(run_dense, iters, false, &us))
        return 1;
    printf("Dense   GEMM : %f us.\n", us);
    const float us_dense = us;
    if (time_us(run_dense, iters, true, &us))
        return 1;
    printf("Dense   GEMM (sync each) : %f us.\n", us);
    if (time_us(run_stream, iters, false, &us))
        return 1;
    printf("Stream  GEMM : %f us.\n", us);
    const float us_stream = us;
    if (time_us(run_stream, iters, true, &us))
        return 1;
    printf("Stream  GEMM (sync each) : %f us.\n", us);
    const double flops_dense = 2.0 * M * N * K, flops_kept = 2.0 * M * (double)N_pruned * K_pruned;
    printf("speedup %.2fx | dense %.1f TFLOP/s | stream effective %.1f TFLOP/s, actual %.1f TFLOP/s\n",
           us_dense / us_stream, flops_dense / us_dense * 1e-6, flops_dense / us_stream * 1e-6,
           flops_kept / us_stream * 1e-6);

    // gather -> dense GEMM -> scatter with the engine's own kernels (Stream_Gemm_NN_reference)
    {
        uint16_t *dA2 = nullptr, *dC2 = nullptr;
        CHECK_HIP(hipMalloc((void **)&dA2, a_bytes));
        CHECK_HIP(hipMalloc((void **)&dC2, c_bytes));
        for (int t = 0; t < block_num; ++t) {
            int32_t *d_rk = nullptr, *d_rn = nullptr;
            CHECK_HIP(hipMalloc((void **)&d_rk, sizeof(int32_t) * std::max(K_cal[t], 1)));
            CHECK_HIP(hipMalloc((void **)&d_rn, sizeof(int32_t) * std::max(N_cal[t], 1)));
            CHECK_HIP(hipMemcpy(d_rk, rel_k[t].data(), sizeof(int32_t) * K_cal[t], hipMemcpyHostToDevice));
            CHECK_HIP(hipMemcpy(d_rn, rel_n[t].data(), sizeof(int32_t) * N_cal[t], hipMemcpyHostToDevice));
            std::vector<float> comp((size_t)K_cal[t] * N_cal[t]);
            for (int i = 0; i < K_cal[t]; ++i)
                for (int j = 0; j < N_cal[t]; ++j)
                    comp[(size_t)i * N_cal[t] + j] =
                        hB[(size_t)(rel_k[t][i] + i) * N + rel_n[t][j] + j + col0[t]];
            tw_plan *tile_plan = nullptr;
            CHECK_TW(tw_plan_create_dense(K_cal[t], N_cal[t], N_cal[t], dtype, comp.data(), &tile_plan));
            CHECK_TW(tw_delete_row(dA, dA2, K_cal[t], M, d_rk, nullptr));
            CHECK_TW(tw_gemm(tile_plan, dA2, TW_LAYOUT_KMAJOR, M, dC2, TW_LAYOUT_KMAJOR, M, M, 1.0f,
                             0.0f, TW_PRUNED_UNTOUCHED, nullptr));
            CHECK_TW(tw_insert_row(dC_ref + off_C[t], dC2, N_cal[t], M, d_rn, nullptr));
            CHECK_HIP(hipDeviceSynchronize());
            tw_plan_destroy(tile_plan);
            hipFree(d_rk);
            hipFree(d_rn);
        }
        hipFree(dA2);
        hipFree(dC2);
    }

    auto fetch = [&](uint16_t *d, std::vector<float> &out) {
        std::vector<uint16_t> bits((size_t)N * M);
        if (hipMemcpy(bits.data(), d, c_bytes, hipMemcpyDeviceToHost) != hipSuccess)
            return 1;
        out.resize(bits.size());
        for (size_t i = 0; i < bits.size(); ++i)
            out[i] = from_bits(bits[i], dtype);
        return 0;
    };
    std::vector<float> c_dense, c_stream, c_ref;
    if (fetch(dC_dense, c_dense) || fetch(dC_stream, c_stream) || fetch(dC_ref, c_ref))
        return 1;

    // host fp32 product on the 16-bit inputs, column-major like the device results
    std::vector<float> c_host((size_t)N * M, 0.0f);
    {
        std::vector<float> Aq((size_t)M * K);
        for (size_t i = 0; i < Aq.size(); ++i)
            Aq[i] = from_bits(to_bits(hA[i], dtype), dtype);
        const int rows = std::min(M, 64); // a bounded sample of rows keeps the host check short
        for (int t = 0; t < block_num; ++t)
            for (int j = 0; j < N_cal[t]; ++j) {
                const int c = rel_n[t][j] + j + col0[t];
                for (int m = 0; m < rows; ++m) {
                    double acc = 0;
                    for (int i = 0; i < K_cal[t]; ++i) {
                        const int k = rel_k[t][i] + i;
                        acc += (double)Aq[(size_t)m * K + k] *
                               from_bits(to_bits(hB[(size_t)k * N + c], dtype), dtype);
                    }
                    c_host[(size_t)c * M + m] = (float)acc;
                }
            }
        for (int c = 0; c < N; ++c) // outside the sample, compare the engine with itself
            for (int m = rows; m < M; ++m)
                c_host[(size_t)c * M + m] = c_stream[(size_t)c * M + m];
    }

    long bad = 0;
    fprintf(stderr, "gather/dense/scatter vs fused stream GEMM (must be identical):\n");
    bad += checkout(c_ref, c_stream, 0, true);
    fprintf(stderr, "fused stream GEMM vs host fp32 product (sampled rows):\n");
    bad += checkout(c_stream, c_host, dtype == TW_BF16 ? 2e-2 : 1e-2, false);
    fprintf(stderr, "dense baseline on B (.) mask vs fused stream GEMM:\n");
    bad += checkout(c_dense, c_stream, dtype == TW_BF16 ? 2e-2 : 1e-2, false);

    tw_plan_destroy(stream_plan);
    tw_plan_destroy(dense_plan);
    hipFree(dA);
    hipFree(dC_dense);
    hipFree(dC_stream);
    hipFree(dC_ref);
    return bad == 0 ? 0 : 2;
}
