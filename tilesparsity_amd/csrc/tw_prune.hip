// TW mask producers on the GPU: network-global thresholds on per-tile row norms (and column
// norms) of the importance scores, as the reference's pruning scripts compute them with NumPy
// (Pruning/VGG/prune_algo.py:55-148; Pruning/BERT/utils/MyHook.py:226-313).
//
// The masks are integer results of floating-point comparisons, so every float operation here
// repeats NumPy's, in NumPy's order:
//   * a tile row norm is sqrt(add.reduce(x*x)) / width in float32, the sum being NumPy's
//     pairwise sum along the contiguous axis (8 running sums over blocks of up to 128 elements,
//     halves combined above that);
//   * a column norm accumulates the rows one after the other;
//   * np.percentile with linear interpolation: the two neighbouring order statistics are found
//     here with a radix select, the interpolation runs on the host in the arithmetic type
//     NumPy would use for the given kind of `q`;
//   * comparisons are strict.
// This file is compiled with floating-point contraction off (pragma below): a product and the sum
// that takes it stay two rounded operations, as in NumPy.  The __fmul_rn / __fadd_rn intrinsics
// would not do: their bodies live in a header outside the pragma and are fused after inlining.
// sqrtf and the division are the compiler's correctly rounded ones (the __fsqrt_rn / __fdiv_rn
// intrinsics map to the approximate hardware instructions).
#include "tw_internal.h"

#include <cmath>
#include <cstring>

#pragma clang fp contract(off)

namespace tw {

__device__ __forceinline__ float sq_term(const float *x, const uint8_t *keep, int i)
{
    const float v = (!keep || keep[i]) ? x[i] : 0.0f;
    return v * v;
}

// NumPy's pairwise sum for n <= 128 terms
__device__ float pairwise_block(const float *x, const uint8_t *keep, int n)
{
    if (n < 8) {
        float r = 0.0f;
        for (int i = 0; i < n; ++i)
            r = r + sq_term(x, keep, i);
        return r;
    }
    float r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
        r[j] = sq_term(x, keep, j);
    int i = 8;
    for (; i < n - (n % 8); i += 8) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            r[j] = r[j] + sq_term(x, keep, i + j);
    }
    float res = ((r[0] + r[1]) + (r[2] + r[3])) + ((r[4] + r[5]) + (r[6] + r[7]));
    for (; i < n; ++i)
        res = res + sq_term(x, keep, i);
    return res;
}

// ... and for any n: halves (the first a multiple of 8) are summed separately and added
__device__ float pairwise_sq_sum(const float *x, const uint8_t *keep, int n)
{
    if (n <= 128)
        return pairwise_block(x, keep, n);
    struct Frame {
        int off, n, stage;
        float left;
    };
    Frame st[32];
    int sp = 0;
    float ret = 0.0f;
    st[sp++] = Frame{0, n, 0, 0.0f};
    while (sp > 0) {
        Frame &f = st[sp - 1];
        if (f.n <= 128) {
            ret = pairwise_block(x + f.off, keep ? keep + f.off : nullptr, f.n);
            --sp;
            continue;
        }
        int n2 = f.n / 2;
        n2 -= n2 % 8;
        if (f.stage == 0) {
            f.stage = 1;
            st[sp++] = Frame{f.off, n2, 0, 0.0f};
        } else if (f.stage == 1) {
            f.left = ret;
            f.stage = 2;
            st[sp++] = Frame{f.off + n2, f.n - n2, 0, 0.0f};
        } else {
            ret = f.left + ret;
            --sp;
        }
    }
    return ret;
}

// norms[t*K + k] = ||score[k][tcol0[t] .. tcol0[t+1])|| / width, pruned columns counting as 0
__global__ void tile_row_norms_kernel(const float *score, int K, int N, const int32_t *tcol0,
                                      int n_tiles, const uint8_t *colkeep, float *norms)
{
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)K * n_tiles)
        return;
    const int t = (int)(idx % n_tiles);
    const int k = (int)(idx / n_tiles);
    const int c0 = tcol0[t], w = tcol0[t + 1] - c0;
    const float s = pairwise_sq_sum(score + (int64_t)k * N + c0, colkeep ? colkeep + c0 : nullptr, w);
    norms[(int64_t)t * K + k] = sqrtf(s) / (float)w; // both correctly rounded (compiler default)
}

// cnorm[c] = ||score[:, c]|| / K, the rows accumulated in order.  The chain of additions is
// sequential by definition; the loads are not, so they are issued 32 rows at a time.
__global__ void col_norms_kernel(const float *score, int K, int N, float *cnorm)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= N)
        return;
    constexpr int U = 32;
    const float *p = score + c;
    float acc = 0.0f;
    int k = 0;
    for (; k + U <= K; k += U) {
        float v[U];
#pragma unroll
        for (int j = 0; j < U; ++j)
            v[j] = p[(int64_t)(k + j) * N];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const float sq = v[j] * v[j];
            acc = acc + sq;
        }
    }
    for (; k < K; ++k) {
        const float v = p[(int64_t)k * N];
        const float sq = v * v;
        acc = acc + sq;
    }
    cnorm[c] = sqrtf(acc) / (float)K;
}

// order-preserving map float -> uint32
__device__ __forceinline__ uint32_t sort_key(float v)
{
    const uint32_t b = __float_as_uint(v);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
static float key_value(uint32_t key)
{
    const uint32_t b = (key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key;
    float v;
    std::memcpy(&v, &b, 4);
    return v;
}

// hist[d] = number of values whose key matches `prefix` in the bits of `mask` and has digit d
// at `shift`
__global__ void __launch_bounds__(256)
    select_hist_kernel(const float *v, int64_t n, uint32_t mask, uint32_t prefix, int shift,
                       unsigned long long *hist)
{
    __shared__ unsigned int s_h[256];
    s_h[threadIdx.x] = 0;
    __syncthreads();
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x) {
        const uint32_t key = sort_key(v[i]);
        if ((key & mask) == prefix)
            atomicAdd(&s_h[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (s_h[threadIdx.x])
        atomicAdd(&hist[threadIdx.x], (unsigned long long)s_h[threadIdx.x]);
}

// out[0] = number of values <= a, out[1] = smallest key above a's (0xFFFFFFFF if none)
__global__ void __launch_bounds__(256)
    rank_stats_kernel(const float *v, int64_t n, uint32_t key_a, unsigned long long *count_le,
                      unsigned int *min_gt)
{
    unsigned long long cnt = 0;
    unsigned int mn = 0xFFFFFFFFu;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x) {
        const uint32_t key = sort_key(v[i]);
        if (key <= key_a)
            ++cnt;
        else
            mn = min(mn, key);
    }
    // one pair of atomics per workgroup
    __shared__ unsigned long long s_cnt;
    __shared__ unsigned int s_min;
    if (threadIdx.x == 0) {
        s_cnt = 0;
        s_min = 0xFFFFFFFFu;
    }
    __syncthreads();
    for (int off = 32; off > 0; off >>= 1) {
        cnt += __shfl_down(cnt, off);
        mn = min(mn, (unsigned int)__shfl_down(mn, off));
    }
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&s_cnt, cnt);
        atomicMin(&s_min, mn);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (s_cnt)
            atomicAdd(count_le, s_cnt);
        if (s_min != 0xFFFFFFFFu)
            atomicMin(min_gt, s_min);
    }
}

// keep[c] = cnorm[c] > threshold
__global__ void col_keep_kernel(const float *cnorm, int N, float thr32, double thr64, int f64,
                                uint8_t *keep)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c < N)
        keep[c] = (f64 ? (double)cnorm[c] > thr64 : cnorm[c] > thr32) ? 1 : 0;
}

// mask[k][c] = (norm of row k in c's tile > threshold) and column c kept
__global__ void fill_mask_kernel(const float *norms, int K, int N, const int32_t *tcol0,
                                 int n_tiles, const uint8_t *colkeep, float thr32, double thr64,
                                 int f64, uint8_t *mask)
{
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)K * N)
        return;
    const int c = (int)(idx % N);
    const int k = (int)(idx / N);
    int lo = 0, hi = n_tiles;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tcol0[mid] <= c)
            lo = mid;
        else
            hi = mid;
    }
    const float nv = norms[(int64_t)lo * K + k];
    bool keep = f64 ? (double)nv > thr64 : nv > thr32;
    if (colkeep)
        keep = keep && colkeep[c];
    mask[idx] = keep ? 1 : 0;
}

// ---------------------------------------------------------------------------------
// host side

namespace {

struct DevBuf {
    void *p = nullptr;
    ~DevBuf() { hipFree(p); }
    template <class T> T *as() { return static_cast<T *>(p); }
};

// The k-th (0-based) smallest of v[0..n) and its upper neighbour in sorted order.
int order_statistics(const float *d_v, int64_t n, int64_t k, hipStream_t s, float *a, float *b)
{
    DevBuf scratch;
    if (hipMalloc(&scratch.p, 256 * sizeof(unsigned long long) + 16) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of the selection scratch failed");
    unsigned long long *d_hist = scratch.as<unsigned long long>();
    const int grid = (int)std::min<int64_t>(1024, (n + 255) / 256);
    uint32_t mask = 0, prefix = 0;
    int64_t rank = k;
    unsigned long long hist[256];
    for (int shift = 24; shift >= 0; shift -= 8) {
        TW_HIP(hipMemsetAsync(d_hist, 0, 256 * sizeof(unsigned long long), s));
        hipLaunchKernelGGL(select_hist_kernel, dim3(grid), dim3(256), 0, s, d_v, n, mask, prefix,
                           shift, d_hist);
        TW_HIP(hipGetLastError());
        TW_HIP(hipMemcpyAsync(hist, d_hist, sizeof(hist), hipMemcpyDeviceToHost, s));
        TW_HIP(hipStreamSynchronize(s));
        int d = 0;
        for (; d < 256; ++d) {
            if (rank < (int64_t)hist[d])
                break;
            rank -= (int64_t)hist[d];
        }
        if (d == 256)
            return fail(TW_ERR_DEVICE, "radix select lost rank %lld", (long long)k);
        prefix |= (uint32_t)d << shift;
        mask |= 255u << shift;
    }
    *a = key_value(prefix);
    // upper neighbour: a again if more than k+1 values are <= a, else the smallest value above
    unsigned long long *d_cnt = d_hist;
    unsigned int *d_min = reinterpret_cast<unsigned int *>(d_hist + 1);
    unsigned long long cnt = 0;
    unsigned int mn = 0xFFFFFFFFu;
    TW_HIP(hipMemsetAsync(d_cnt, 0, sizeof(unsigned long long), s));
    TW_HIP(hipMemcpyAsync(d_min, &mn, sizeof(mn), hipMemcpyHostToDevice, s));
    hipLaunchKernelGGL(rank_stats_kernel, dim3(grid), dim3(256), 0, s, d_v, n, prefix, d_cnt, d_min);
    TW_HIP(hipGetLastError());
    TW_HIP(hipMemcpyAsync(&cnt, d_cnt, sizeof(cnt), hipMemcpyDeviceToHost, s));
    TW_HIP(hipMemcpyAsync(&mn, d_min, sizeof(mn), hipMemcpyDeviceToHost, s));
    TW_HIP(hipStreamSynchronize(s));
    *b = ((int64_t)cnt > k + 1 || mn == 0xFFFFFFFFu) ? *a : key_value(mn);
    return TW_OK;
}

struct Threshold {
    float f32;
    double f64;
    int is_f64;
};

// np.percentile(v, q) with linear interpolation for a float32 vector on the device.  With
// q_is_f64 == 0 (q was a Python number) the quantile q/100, the virtual index (n-1)*quantile
// and the interpolation are float32; with 1 (q was a NumPy float64) they are float64, only
// the difference of the two neighbours stays float32.
int percentile_linear(const float *d_v, int64_t n, double q, int q_is_f64, hipStream_t s,
                      Threshold *out)
{
    if (n <= 0)
        return fail(TW_ERR_SHAPE, "percentile of an empty set");
    if (!(q >= 0.0 && q <= 100.0))
        return fail(TW_ERR_SHAPE, "percentile %g is outside [0, 100]", q);
    int64_t lo;
    double gamma64 = 0.0;
    float gamma32 = 0.0f;
    bool top;
    if (q_is_f64) {
        const double quant = q / 100.0;
        const double virt = (double)(n - 1) * quant;
        top = virt >= (double)(n - 1);
        lo = top ? n - 1 : (int64_t)std::floor(virt);
        gamma64 = virt - std::floor(virt);
    } else {
        const float quant = (float)q / 100.0f;
        const float virt = (float)(n - 1) * quant;
        top = virt >= (float)(n - 1);
        lo = top ? n - 1 : (int64_t)std::floor(virt);
        gamma32 = virt - std::floor(virt);
    }
    float a, b;
    int st = order_statistics(d_v, n, std::min(lo, n - 1), s, &a, &b);
    if (st)
        return st;
    if (top)
        b = a;
    const float diff = b - a;
    out->is_f64 = q_is_f64;
    if (q_is_f64) {
        const double r = gamma64 >= 0.5 ? (double)b - (double)diff * (1.0 - gamma64)
                                        : (double)a + (double)diff * gamma64;
        out->f64 = r;
        out->f32 = (float)r;
    } else {
        volatile float prod; // keep the product a rounded float32 (no fma on the host either)
        float r;
        if (gamma32 >= 0.5f) {
            prod = diff * (1.0f - gamma32);
            r = b - prod;
        } else {
            prod = diff * gamma32;
            r = a + prod;
        }
        out->f32 = r;
        out->f64 = (double)r;
    }
    return TW_OK;
}

int check_layers(int n_layers, const int32_t *K, const int32_t *N, const float *const *scores,
                 uint8_t *const *masks, int granularity)
{
    if (n_layers <= 0 || granularity <= 0)
        return fail(TW_ERR_SHAPE, "n_layers=%d granularity=%d must be positive", n_layers,
                    granularity);
    if (!K || !N || !scores || !masks)
        return fail(TW_ERR_NULL, "K, N, scores or masks is NULL");
    for (int l = 0; l < n_layers; ++l) {
        if (K[l] <= 0 || N[l] <= 0)
            return fail(TW_ERR_SHAPE, "layer %d: K=%d N=%d must be positive", l, K[l], N[l]);
        if (!scores[l] || !masks[l])
            return fail(TW_ERR_NULL, "layer %d: scores or mask pointer is NULL", l);
    }
    return TW_OK;
}

// per layer: the tile table on the device, offsets of the layer's norms in the pooled vector
struct LayerTiles {
    std::vector<int32_t> tcol0; // n_tiles + 1 entries
    int64_t norm_off = 0;
};

// norms of all layers into one pooled vector, one threshold, masks
int rows_stage(int n_layers, const int32_t *K, const int32_t *N, const float *const *scores,
               std::vector<LayerTiles> &lt, const std::vector<uint8_t *> &d_colkeep, double q,
               int q_is_f64, uint8_t *const *masks, Threshold *thr, hipStream_t s)
{
    int64_t total = 0, tab = 0;
    for (int l = 0; l < n_layers; ++l) {
        lt[l].norm_off = total;
        total += (int64_t)K[l] * ((int64_t)lt[l].tcol0.size() - 1);
        tab += (int64_t)lt[l].tcol0.size();
    }
    DevBuf norms, tables;
    if (hipMalloc(&norms.p, sizeof(float) * total) != hipSuccess ||
        hipMalloc(&tables.p, sizeof(int32_t) * tab) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of %lld norms failed", (long long)total);
    std::vector<int32_t> flat;
    std::vector<int64_t> tab_off(n_layers);
    for (int l = 0; l < n_layers; ++l) {
        tab_off[l] = (int64_t)flat.size();
        flat.insert(flat.end(), lt[l].tcol0.begin(), lt[l].tcol0.end());
    }
    TW_HIP(hipMemcpyAsync(tables.p, flat.data(), sizeof(int32_t) * flat.size(),
                          hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s)); // `flat` is pageable host memory
    for (int l = 0; l < n_layers; ++l) {
        const int nt = (int)lt[l].tcol0.size() - 1;
        const int64_t n_rt = (int64_t)K[l] * nt;
        hipLaunchKernelGGL(tile_row_norms_kernel, dim3((unsigned)((n_rt + 255) / 256)), dim3(256),
                           0, s, scores[l], K[l], N[l], tables.as<int32_t>() + tab_off[l], nt,
                           d_colkeep.empty() ? nullptr : d_colkeep[l],
                           norms.as<float>() + lt[l].norm_off);
    }
    TW_HIP(hipGetLastError());
    int st = percentile_linear(norms.as<float>(), total, q, q_is_f64, s, thr);
    if (st)
        return st;
    for (int l = 0; l < n_layers; ++l) {
        const int nt = (int)lt[l].tcol0.size() - 1;
        const int64_t n_el = (int64_t)K[l] * N[l];
        hipLaunchKernelGGL(fill_mask_kernel, dim3((unsigned)((n_el + 255) / 256)), dim3(256), 0, s,
                           norms.as<float>() + lt[l].norm_off, K[l], N[l],
                           tables.as<int32_t>() + tab_off[l], nt,
                           d_colkeep.empty() ? nullptr : d_colkeep[l], thr->f32, thr->f64,
                           thr->is_f64, masks[l]);
    }
    TW_HIP(hipGetLastError());
    TW_HIP(hipStreamSynchronize(s)); // the temporaries are freed on return
    return TW_OK;
}

} // namespace
} // namespace tw

using namespace tw;

extern "C" {

int tw_tiles_every_g_columns(int N, int G, int32_t *tile_col0, int32_t *tile_width, int32_t *n_tiles)
{
    if (N <= 0 || G <= 0)
        return fail(TW_ERR_SHAPE, "N=%d G=%d must be positive", N, G);
    if (!tile_col0 || !tile_width || !n_tiles)
        return fail(TW_ERR_NULL, "an output pointer is NULL");
    int t = 0;
    for (int c = 0; c < N; c += G, ++t) {
        tile_col0[t] = c;
        tile_width[t] = std::min(G, N - c);
    }
    *n_tiles = t;
    return TW_OK;
}

int tw_tiles_every_g_kept_columns(int N, int G, const uint8_t *col_mask, int32_t *tile_col0,
                                  int32_t *tile_width, int32_t *n_tiles)
{
    if (N <= 0 || G <= 0)
        return fail(TW_ERR_SHAPE, "N=%d G=%d must be positive", N, G);
    if (!col_mask || !tile_col0 || !tile_width || !n_tiles)
        return fail(TW_ERR_NULL, "a pointer is NULL");
    int t = 0, start = 0, kept = 0;
    for (int c = 0; c < N; ++c) {
        kept += col_mask[c] != 0;
        if (kept == G && c + 1 < N) {
            tile_col0[t] = start;
            tile_width[t] = c + 1 - start;
            ++t;
            start = c + 1;
            kept = 0;
        }
    }
    tile_col0[t] = start;
    tile_width[t] = N - start;
    *n_tiles = t + 1;
    return TW_OK;
}

int tw_prune_tile_row_norms(int K, int N, const float *scores, int n_tiles,
                            const int32_t *tile_col0, const int32_t *tile_width,
                            const uint8_t *col_keep, float *norms, void *stream)
{
    if (K <= 0 || N <= 0 || n_tiles <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d n_tiles=%d must be positive", K, N, n_tiles);
    if (!scores || !tile_col0 || !tile_width || !norms)
        return fail(TW_ERR_NULL, "a pointer is NULL");
    std::vector<int32_t> tcol0(n_tiles + 1);
    int c = 0;
    for (int t = 0; t < n_tiles; ++t) {
        if (tile_col0[t] != c || tile_width[t] <= 0)
            return fail(TW_ERR_TILE_TABLE, "tile %d: col0=%d width=%d", t, tile_col0[t], tile_width[t]);
        tcol0[t] = c;
        c += tile_width[t];
    }
    if (c != N)
        return fail(TW_ERR_TILE_TABLE, "tiles cover %d columns, N=%d", c, N);
    tcol0[n_tiles] = N;
    hipStream_t s = (hipStream_t)stream;
    DevBuf tab;
    if (hipMalloc(&tab.p, sizeof(int32_t) * (n_tiles + 1)) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of the tile table failed");
    TW_HIP(hipMemcpyAsync(tab.p, tcol0.data(), sizeof(int32_t) * (n_tiles + 1), hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s));
    const int64_t n_rt = (int64_t)K * n_tiles;
    hipLaunchKernelGGL(tile_row_norms_kernel, dim3((unsigned)((n_rt + 255) / 256)), dim3(256), 0, s,
                       scores, K, N, tab.as<int32_t>(), n_tiles, col_keep, norms);
    TW_HIP(hipGetLastError());
    TW_HIP(hipStreamSynchronize(s));
    return TW_OK;
}

int tw_prune_col_norms(int K, int N, const float *scores, float *norms, void *stream)
{
    if (K <= 0 || N <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d must be positive", K, N);
    if (!scores || !norms)
        return fail(TW_ERR_NULL, "a pointer is NULL");
    hipLaunchKernelGGL(col_norms_kernel, dim3((N + 63) / 64), dim3(64), 0, (hipStream_t)stream, scores,
                       K, N, norms);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int tw_percentile_linear(const float *values, int64_t n, double q, int q_type, double *result,
                         void *stream)
{
    if (!values || !result)
        return fail(TW_ERR_NULL, "a pointer is NULL");
    if (q_type != TW_Q_F32 && q_type != TW_Q_F64)
        return fail(TW_ERR_LAYOUT, "q_type=%d: unknown", q_type);
    Threshold t;
    int st = percentile_linear(values, n, q, q_type, (hipStream_t)stream, &t);
    if (!st)
        *result = t.f64;
    return st;
}

int tw_prune_tiled_wise_1d(int n_layers, const int32_t *K, const int32_t *N,
                           const float *const *scores, double sparsity, int q_type,
                           int granularity, uint8_t *const *masks, double *threshold, void *stream)
{
    int st = check_layers(n_layers, K, N, scores, masks, granularity);
    if (st)
        return st;
    if (q_type != TW_Q_F32 && q_type != TW_Q_F64)
        return fail(TW_ERR_LAYOUT, "q_type=%d: unknown", q_type);
    std::vector<LayerTiles> lt(n_layers);
    for (int l = 0; l < n_layers; ++l) {
        for (int c = 0; c < N[l]; c += granularity)
            lt[l].tcol0.push_back(c);
        lt[l].tcol0.push_back(N[l]);
    }
    Threshold thr;
    st = rows_stage(n_layers, K, N, scores, lt, {}, sparsity, q_type, masks, &thr,
                    (hipStream_t)stream);
    if (!st && threshold)
        *threshold = thr.f64;
    return st;
}

int tw_prune_tiled_wise_2d(int n_layers, const int32_t *K, const int32_t *N,
                           const float *const *scores, double sparsity, int q_type, int transform,
                           int granularity, uint8_t *const *masks, uint8_t *const *col_masks,
                           double *thresholds, void *stream)
{
    int st = check_layers(n_layers, K, N, scores, masks, granularity);
    if (st)
        return st;
    if (q_type != TW_Q_F32 && q_type != TW_Q_F64)
        return fail(TW_ERR_LAYOUT, "q_type=%d: unknown", q_type);
    hipStream_t s = (hipStream_t)stream;
    double q = sparsity;
    if (transform) {
        // the two prunings compose to `sparsity`; NumPy's result here is a float64
        if (!(sparsity >= 0.0 && sparsity <= 100.0))
            return fail(TW_ERR_SHAPE, "sparsity %g is outside [0, 100]", sparsity);
        q = 100.0 - std::sqrt(10000.0 - sparsity * 100.0);
        q_type = TW_Q_F64;
    }
    // columns: one pooled vector of column norms, one threshold
    int64_t total_n = 0;
    std::vector<int64_t> coff(n_layers);
    for (int l = 0; l < n_layers; ++l) {
        coff[l] = total_n;
        total_n += N[l];
    }
    DevBuf cnorm, ckeep;
    if (hipMalloc(&cnorm.p, sizeof(float) * total_n) != hipSuccess ||
        hipMalloc(&ckeep.p, (size_t)total_n) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of %lld column norms failed", (long long)total_n);
    for (int l = 0; l < n_layers; ++l)
        hipLaunchKernelGGL(col_norms_kernel, dim3((N[l] + 63) / 64), dim3(64), 0, s, scores[l], K[l],
                           N[l], cnorm.as<float>() + coff[l]);
    TW_HIP(hipGetLastError());
    Threshold thr_c;
    st = percentile_linear(cnorm.as<float>(), total_n, q, q_type, s, &thr_c);
    if (st)
        return st;
    hipLaunchKernelGGL(col_keep_kernel, dim3((unsigned)((total_n + 255) / 256)), dim3(256), 0, s,
                       cnorm.as<float>(), (int)total_n, thr_c.f32, thr_c.f64, thr_c.is_f64,
                       ckeep.as<uint8_t>());
    TW_HIP(hipGetLastError());
    std::vector<uint8_t> h_keep(total_n);
    TW_HIP(hipMemcpyAsync(h_keep.data(), ckeep.p, (size_t)total_n, hipMemcpyDeviceToHost, s));
    TW_HIP(hipStreamSynchronize(s));
    // tiles end after every `granularity` kept columns
    std::vector<LayerTiles> lt(n_layers);
    std::vector<uint8_t *> d_colkeep(n_layers);
    std::vector<int32_t> col0, width;
    for (int l = 0; l < n_layers; ++l) {
        col0.resize(N[l]);
        width.resize(N[l]);
        int32_t nt = 0;
        st = tw_tiles_every_g_kept_columns(N[l], granularity, h_keep.data() + coff[l], col0.data(),
                                           width.data(), &nt);
        if (st)
            return st;
        lt[l].tcol0.assign(col0.begin(), col0.begin() + nt);
        lt[l].tcol0.push_back(N[l]);
        d_colkeep[l] = ckeep.as<uint8_t>() + coff[l];
        if (col_masks && col_masks[l])
            TW_HIP(hipMemcpyAsync(col_masks[l], d_colkeep[l], (size_t)N[l], hipMemcpyDeviceToDevice, s));
    }
    Threshold thr_r;
    st = rows_stage(n_layers, K, N, scores, lt, d_colkeep, q, q_type, masks, &thr_r, s);
    if (!st && thresholds) {
        thresholds[0] = thr_c.f64;
        thresholds[1] = thr_r.f64;
    }
    return st;
}

} // extern "C"
