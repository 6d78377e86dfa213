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
#include <mutex>

#pragma clang fp contract(off)

namespace tw {

__device__ __forceinline__ float sq_term(const float *x, const uint8_t *keep, int i)
{
    const float v = (!keep || keep[i]) ? x[i] : 0.0f;
    return v * v;
}

// NumPy's pairwise sum for n <= 128 terms, by a group of 8 adjacent lanes: lane j keeps NumPy's
// running sum r[j] (terms j, j+8, j+16, ...), the three shuffle steps are NumPy's
// ((r0+r1)+(r2+r3)) + ((r4+r5)+(r6+r7)), lane 0 then adds the n % 8 trailing terms.  The result
// is valid in lane 0 of the group.
__device__ float pairwise_block(const float *x, const uint8_t *keep, int n, int l8)
{
    if (n < 8) {
        float r = 0.0f;
        for (int i = 0; i < n; ++i)
            r = r + sq_term(x, keep, i);
        return r;
    }
    float r = sq_term(x, keep, l8);
    int i = 8;
    for (; i < n - (n % 8); i += 8)
        r = r + sq_term(x, keep, i + l8);
    r = r + __shfl_down(r, 1, 8);
    r = r + __shfl_down(r, 2, 8);
    r = r + __shfl_down(r, 4, 8);
    for (; i < n; ++i)
        r = r + sq_term(x, keep, i);
    return r;
}

// ... and for any n: halves (the first a multiple of 8) are summed separately and added
__device__ float pairwise_sq_sum(const float *x, const uint8_t *keep, int n, int l8)
{
    if (n <= 128)
        return pairwise_block(x, keep, n, l8);
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
            ret = pairwise_block(x + f.off, keep ? keep + f.off : nullptr, f.n, l8);
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

constexpr int kNormNotDivided = 1;   // norms are not divided by the tile width
constexpr int kPerTileThreshold = 2; // tile t compares with selection state t, not with state 0

// One entry per layer of a producer call; all layers run in one launch per stage.
struct PruneLayer {
    const float *score;
    uint8_t *mask;
    const uint8_t *colkeep; // nullptr: every column counts
    const int32_t *tcol0;   // n_tiles + 1 entries
    float *norms;           // [n_tiles][K]
    int32_t K, N, n_tiles;
    int32_t flags;          // kNormNotDivided, kPerTileThreshold
    int64_t rt_begin;       // first (row, tile) pair of this layer in the launch-wide numbering
    int64_t el_begin;       // first item of the mask fill likewise (ceil(K/4) x ceil(N/16) items)
};

__device__ __forceinline__ int find_layer(const PruneLayer *layers, int n_layers, int64_t idx,
                                          bool by_elements)
{
    int lo = 0, hi = n_layers;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if ((by_elements ? layers[mid].el_begin : layers[mid].rt_begin) <= idx)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// norms[t*K + k] = ||score[k][tcol0[t] .. tcol0[t+1])|| / width, pruned columns counting as 0;
// 8 lanes per (row, tile), neighbouring groups take neighbouring tiles of a row
__global__ void __launch_bounds__(256)
    tile_row_norms_kernel(const PruneLayer *layers, int n_layers, int64_t n_pairs)
{
    const int64_t gid = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 3;
    const int l8 = threadIdx.x & 7;
    if (gid >= n_pairs)
        return; // whole groups leave together
    const PruneLayer L = layers[find_layer(layers, n_layers, gid, false)];
    const int64_t idx = gid - L.rt_begin;
    const int t = (int)(idx % L.n_tiles);
    const int k = (int)(idx / L.n_tiles);
    const int c0 = L.tcol0[t], w = L.tcol0[t + 1] - c0;
    const float s = pairwise_sq_sum(L.score + (int64_t)k * L.N + c0,
                                    L.colkeep ? L.colkeep + c0 : nullptr, w, l8);
    if (l8 == 0)
        L.norms[(int64_t)t * L.K + k] =
            (L.flags & kNormNotDivided) ? sqrtf(s) : sqrtf(s) / (float)w; // both correctly rounded
}

// One entry per layer for the column stage.
struct ColLayer {
    const float *score;
    int32_t K, N;
    int64_t col_begin; // first column of this layer in the pooled numbering
};

// cnorm[pooled c] = ||score[:, c]|| / K, the rows accumulated in order.  The chain of additions
// is sequential by definition; the loads are not, so they are issued 32 rows at a time, and all
// layers share one launch.
__global__ void col_norms_kernel(const ColLayer *layers, int n_layers, int64_t n_cols, float *cnorm)
{
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_cols)
        return;
    int lo = 0, hi = n_layers;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (layers[mid].col_begin <= g)
            lo = mid;
        else
            hi = mid;
    }
    const ColLayer L = layers[lo];
    const int K = L.K, N = L.N;
    constexpr int U = 32;
    const float *p = L.score + (g - L.col_begin);
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
    cnorm[g] = sqrtf(acc) / (float)K;
}

// order-preserving map float -> uint32
__device__ __forceinline__ uint32_t sort_key(float v)
{
    const uint32_t b = __float_as_uint(v);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
// Selection state in device memory, so that the passes follow each other on the stream without
// a host round trip.  Pass p (p = 0..3) counts, among the values whose key agrees with the digits
// fixed by the passes before it, the digit at bit 24 - 8 p; which digit holds the rank is worked
// out from the histograms by whoever needs it next (resolve_prefix).
struct SelectState {
    unsigned long long hist[4][256];
    unsigned long long rank0;     // rank (0-based) of the wanted value
    unsigned long long count_le;  // values <= the k-th smallest
    uint32_t prefix;              // key of the k-th smallest (written with the threshold)
    uint32_t min_gt;              // smallest key above the k-th smallest's (0xFFFFFFFF: none)
    int32_t lost;                 // set if a pass found no digit (cannot happen for rank < n)
    float thr32;                  // the threshold, for the kernels that follow
    double thr64;
};

// The selection kernels work on segments of equal length laid end to end (one segment for the
// network-wide thresholds, one per tile for per-tile thresholds): segment g = blockIdx.y (or
// blockIdx.x for the one-workgroup kernels) uses state st[g] and values v[g*n .. g*n+n).
__global__ void __launch_bounds__(256) select_init_kernel(SelectState *st, unsigned long long rank)
{
    st += blockIdx.x;
#pragma unroll
    for (int p = 0; p < 4; ++p)
        st->hist[p][threadIdx.x] = 0;
    if (threadIdx.x == 0) {
        st->rank0 = rank;
        st->count_le = 0;
        st->prefix = 0;
        st->min_gt = 0xFFFFFFFFu;
        st->lost = 0;
    }
}

// The key digits that passes 0 .. npass-1 have fixed, the rank that is left among the values
// matching them, and whether a pass found no digit.  Called by all 256 threads of a workgroup
// (an inclusive scan of each histogram finds the digit whose count range holds the rank); every
// thread returns the same values.
__device__ void resolve_prefix(const SelectState *st, int npass, uint32_t &prefix, uint32_t &mask,
                               unsigned long long &rank, bool &lost)
{
    __shared__ unsigned long long s_wave[4];
    __shared__ unsigned long long s_before;
    __shared__ int s_digit;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    prefix = 0;
    mask = 0;
    rank = st->rank0;
    lost = false;
    for (int p = 0; p < npass; ++p) {
        const int shift = 24 - 8 * p;
        const unsigned long long c = st->hist[p][tid];
        unsigned long long incl = c;
        for (int off = 1; off < 64; off <<= 1) {
            const unsigned long long up = __shfl_up(incl, off);
            if (lane >= off)
                incl += up;
        }
        if (lane == 63)
            s_wave[wave] = incl;
        if (tid == 0)
            s_digit = -1;
        __syncthreads();
        for (int w = 0; w < wave; ++w)
            incl += s_wave[w];
        const unsigned long long excl = incl - c;
        if (c > 0 && excl <= rank && rank < incl) { // exactly one digit, if any
            s_digit = tid;
            s_before = excl;
        }
        __syncthreads();
        int d = s_digit;
        if (d < 0) {
            lost = true;
            d = 255;
        } else {
            rank -= s_before;
        }
        prefix |= (uint32_t)d << shift;
        mask |= 255u << shift;
        __syncthreads(); // the shared words are rewritten by the next pass
    }
}

// Calls f(value) for every element of v[0..n) once, the workgroups of blockIdx.x sharing the
// work: 16-byte loads over the aligned middle (four of them in flight per thread), single
// elements at the ragged ends.
template <class F> __device__ __forceinline__ void for_each_value(const float *v, int64_t n, F f)
{
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nthr = (int64_t)gridDim.x * blockDim.x;
    const int64_t head = min(n, (int64_t)((16 - ((uintptr_t)v & 15)) & 15) >> 2);
    const int64_t nvec = (n - head) >> 2;
    const float4 *v4 = reinterpret_cast<const float4 *>(v + head);
    int64_t i = tid;
    for (; i + 3 * nthr < nvec; i += 4 * nthr) {
        const float4 a = v4[i], b = v4[i + nthr], c = v4[i + 2 * nthr], d = v4[i + 3 * nthr];
        f(a.x); f(a.y); f(a.z); f(a.w);
        f(b.x); f(b.y); f(b.z); f(b.w);
        f(c.x); f(c.y); f(c.z); f(c.w);
        f(d.x); f(d.y); f(d.z); f(d.w);
    }
    for (; i < nvec; i += nthr) {
        const float4 a = v4[i];
        f(a.x); f(a.y); f(a.z); f(a.w);
    }
    // the elements before the first and after the last whole vector
    const int64_t tail0 = head + 4 * nvec;
    for (int64_t j = tid; j < head + (n - tail0); j += nthr)
        f(v[j < head ? j : tail0 + (j - head)]);
}

// hist[pass][d] += number of values whose key matches the digits fixed so far and has digit d
// at bit 24 - 8 pass
__global__ void __launch_bounds__(256)
    select_hist_kernel(const float *v, int64_t n, int pass, SelectState *st)
{
    st += blockIdx.y;
    v += (int64_t)blockIdx.y * n;
    __shared__ unsigned int s_h[256];
    s_h[threadIdx.x] = 0;
    uint32_t prefix, mask;
    unsigned long long rank;
    bool lost;
    resolve_prefix(st, pass, prefix, mask, rank, lost);
    __syncthreads(); // s_h is zeroed
    const int shift = 24 - 8 * pass;
    for_each_value(v, n, [&](float x) {
        const uint32_t key = sort_key(x);
        if ((key & mask) == prefix)
            atomicAdd(&s_h[(key >> shift) & 255u], 1u);
    });
    __syncthreads();
    if (s_h[threadIdx.x])
        atomicAdd(&st->hist[pass][threadIdx.x], (unsigned long long)s_h[threadIdx.x]);
}

// count_le = number of values <= the selected one, min_gt = smallest key above it
__global__ void __launch_bounds__(256) rank_stats_kernel(const float *v, int64_t n, SelectState *st)
{
    st += blockIdx.y;
    v += (int64_t)blockIdx.y * n;
    uint32_t key_a, mask;
    unsigned long long rank;
    bool lost;
    resolve_prefix(st, 4, key_a, mask, rank, lost);
    unsigned long long cnt = 0;
    unsigned int mn = 0xFFFFFFFFu;
    for_each_value(v, n, [&](float x) {
        const uint32_t key = sort_key(x);
        if (key <= key_a)
            ++cnt;
        else
            mn = min(mn, key);
    });
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
            atomicAdd(&st->count_le, s_cnt);
        if (s_min != 0xFFFFFFFFu)
            atomicMin(&st->min_gt, s_min);
    }
}

__device__ __forceinline__ float key_to_float(uint32_t key)
{
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

// NumPy's two-sided linear interpolation between the k-th smallest value a and its upper
// neighbour b (a again if it is repeated, or if the index is the last one): float32 throughout
// for a float32 gamma, float64 with a float32 difference b - a otherwise.
__global__ void __launch_bounds__(256)
    select_lerp_kernel(SelectState *st, unsigned long long k, int top, int f64, float gamma32,
                       double gamma64)
{
    st += blockIdx.x;
    uint32_t key_a, mask;
    unsigned long long rank;
    bool lost;
    resolve_prefix(st, 4, key_a, mask, rank, lost);
    if (threadIdx.x != 0)
        return;
    st->prefix = key_a;
    st->lost = lost ? 1 : 0;
    const float a = key_to_float(key_a);
    float b = a;
    if (!top && st->count_le <= k + 1 && st->min_gt != 0xFFFFFFFFu)
        b = key_to_float(st->min_gt);
    const float diff = b - a;
    if (f64) {
        const double prod = gamma64 >= 0.5 ? (double)diff * (1.0 - gamma64) : (double)diff * gamma64;
        const double r = gamma64 >= 0.5 ? (double)b - prod : (double)a + prod;
        st->thr64 = r;
        st->thr32 = (float)r;
    } else {
        const float prod = gamma32 >= 0.5f ? diff * (1.0f - gamma32) : diff * gamma32;
        const float r = gamma32 >= 0.5f ? b - prod : a + prod;
        st->thr32 = r;
        st->thr64 = (double)r;
    }
}

// keep[c] = cnorm[c] > threshold
__global__ void col_keep_kernel(const float *cnorm, int N, const SelectState *st, int f64,
                                uint8_t *keep)
{
    const float thr32 = st->thr32;
    const double thr64 = st->thr64;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c < N)
        keep[c] = (f64 ? (double)cnorm[c] > thr64 : cnorm[c] > thr32) ? 1 : 0;
}

// mask[k][c] = (norm of row k in c's tile > threshold) and column c kept.  One thread per 16
// consecutive columns of kFillRows consecutive rows: one 16-byte store per row where the chunk
// is whole and aligned; the layer and tile look-ups are shared by the rows.
constexpr int kFillRows = 4;
__global__ void __launch_bounds__(256)
    fill_mask_kernel(const PruneLayer *layers, int n_layers, int64_t n_chunks,
                     const SelectState *st, int f64)
{
    // the first chunk of every layer, so that a thread finds its layer without a chain of
    // global loads (the first kFillCached layers; a search beyond them reads the table itself)
    constexpr int kFillCached = 128;
    __shared__ int64_t s_begin[kFillCached];
    const int n_cached = min(n_layers, kFillCached);
    for (int i = (int)threadIdx.x; i < n_cached; i += (int)blockDim.x)
        s_begin[i] = layers[i].el_begin;
    __syncthreads();
    const int64_t gidx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gidx >= n_chunks)
        return;
    int li;
    if (n_layers > kFillCached && layers[kFillCached].el_begin <= gidx) {
        li = kFillCached + find_layer(layers + kFillCached, n_layers - kFillCached, gidx, true);
    } else {
        int lo = 0, hi = n_cached;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (s_begin[mid] <= gidx)
                lo = mid;
            else
                hi = mid;
        }
        li = lo;
    }
    const PruneLayer L = layers[li];
    const bool per_tile = (L.flags & kPerTileThreshold) != 0;
    float thr32 = st->thr32;
    double thr64 = st->thr64;
    const int64_t idx = gidx - L.el_begin;
    const int cpr = (L.N + 15) >> 4; // chunks per row
    // (a 32-bit division where the layer's item count allows it: the 64-bit one is long)
    const int kg = (idx >> 31) == 0 ? (int)((uint32_t)idx / (uint32_t)cpr) : (int)(idx / cpr);
    const int c0 = (int)(idx - (int64_t)kg * cpr) << 4;
    const int k0 = kg * kFillRows;
    const int nrows = min(kFillRows, L.K - k0);
    // the tile of column c0: start near where tiles of equal width would put it, then walk
    int t = min(L.n_tiles - 1, (int)((float)c0 * (float)L.n_tiles / (float)L.N));
    while (L.tcol0[t] > c0)
        --t;
    while (L.tcol0[t + 1] <= c0)
        ++t;
    int t_end = L.tcol0[t + 1];
    bool row_keep[kFillRows];
    auto enter_tile = [&]() { // the rows' norms in tile t against its threshold
        if (per_tile) {
            thr32 = st[t].thr32;
            thr64 = st[t].thr64;
        }
#pragma unroll
        for (int r = 0; r < kFillRows; ++r) {
            const float nv = r < nrows ? L.norms[(int64_t)t * L.K + k0 + r] : 0.0f;
            row_keep[r] = r < nrows && (f64 ? (double)nv > thr64 : nv > thr32);
        }
    };
    enter_tile();
    uint32_t w[kFillRows][4];
#pragma unroll
    for (int r = 0; r < kFillRows; ++r)
        w[r][0] = w[r][1] = w[r][2] = w[r][3] = 0u;
    const int n = min(16, L.N - c0);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        if (e < n) {
            const int c = c0 + e;
            if (c >= t_end) {
                ++t;
                t_end = L.tcol0[t + 1];
                enter_tile();
            }
            const bool col = !L.colkeep || L.colkeep[c];
#pragma unroll
            for (int r = 0; r < kFillRows; ++r)
                w[r][e >> 2] |= (col && row_keep[r] ? 1u : 0u) << ((e & 3) * 8);
        }
    }
#pragma unroll
    for (int r = 0; r < kFillRows; ++r) {
        if (r >= nrows)
            break;
        uint8_t *dst = L.mask + (int64_t)(k0 + r) * L.N + c0;
        if (n == 16 && (((uintptr_t)dst) & 15) == 0) {
            uint4 v;
            v.x = w[r][0];
            v.y = w[r][1];
            v.z = w[r][2];
            v.w = w[r][3];
            *reinterpret_cast<uint4 *>(dst) = v;
        } else {
            for (int e = 0; e < n; ++e)
                dst[e] = (uint8_t)(w[r][e >> 2] >> ((e & 3) * 8));
        }
    }
}

// ---------------------------------------------------------------------------------
// mixed masks: a TW mask plus the largest remaining single elements

struct MixLayer {
    const float *score;
    const uint8_t *mask0; // the TW mask of the layer
    uint8_t *out;         // may be mask0 itself
    int64_t begin;        // first element of the layer in the pooled vector
};

__device__ inline int find_mix_layer(const MixLayer *layers, int n_layers, int64_t idx)
{
    int lo = 0, hi = n_layers;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (layers[mid].begin <= idx)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// Both mixed-mask kernels walk the pooled element numbering in groups of four: a group that lies
// in one layer and is 16-byte aligned there moves as vectors, any other group element by element.
struct MixGroup {
    MixLayer L;
    int64_t e;   // first element inside the layer
    bool vec;
};

__device__ __forceinline__ MixGroup mix_group(const MixLayer *layers, int n_layers, int64_t total,
                                              int64_t i)
{
    MixGroup g;
    const int l = find_mix_layer(layers, n_layers, i);
    g.L = layers[l];
    g.e = i - g.L.begin;
    const int64_t end = l + 1 < n_layers ? layers[l + 1].begin : total;
    g.vec = i + 4 <= end && (((uintptr_t)(g.L.score + g.e)) & 15) == 0 &&
            (((uintptr_t)(g.L.mask0 + g.e)) & 3) == 0 && (((uintptr_t)(g.L.out + g.e)) & 3) == 0;
    return g;
}

__device__ __forceinline__ float mix_value(float x, uint8_t m0)
{
    const float sq = x * x;
    const float nrm = sqrtf(sq) / 1.0f;
    return nrm - (m0 ? 1.0f : 0.0f);
}

// pool[i] = ||x|| of the single element (sqrt(x*x) / 1, the reference's norm over a tile of one
// column) minus 1 where the TW mask already keeps it (prune_algo.py:159-161)
__global__ void __launch_bounds__(256)
    mix_values_kernel(const MixLayer *layers, int n_layers, int64_t total, float *pool)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x * 4;
    for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < total; i += stride) {
        const MixGroup g = mix_group(layers, n_layers, total, i);
        if (g.vec) {
            const float4 x = *reinterpret_cast<const float4 *>(g.L.score + g.e);
            const uint32_t m = *reinterpret_cast<const uint32_t *>(g.L.mask0 + g.e);
            float4 r;
            r.x = mix_value(x.x, (uint8_t)(m & 255u));
            r.y = mix_value(x.y, (uint8_t)((m >> 8) & 255u));
            r.z = mix_value(x.z, (uint8_t)((m >> 16) & 255u));
            r.w = mix_value(x.w, (uint8_t)(m >> 24));
            *reinterpret_cast<float4 *>(pool + i) = r; // the pool is 256-byte aligned, i = 0 mod 4
        } else {
            for (int64_t j = i; j < min(i + 4, total); ++j) {
                const MixLayer L = layers[find_mix_layer(layers, n_layers, j)];
                const int64_t e = j - L.begin;
                pool[j] = mix_value(L.score[e], L.mask0[e]);
            }
        }
    }
}

// out = mask0 | (pool > threshold)   (prune_algo.py:171-176)
__global__ void __launch_bounds__(256)
    mix_mask_kernel(const MixLayer *layers, int n_layers, int64_t total, const float *pool,
                    const SelectState *st, int f64)
{
    const float thr32 = st->thr32;
    const double thr64 = st->thr64;
    auto above = [&](float v) { return f64 ? (double)v > thr64 : v > thr32; };
    const int64_t stride = (int64_t)gridDim.x * blockDim.x * 4;
    for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < total; i += stride) {
        const MixGroup g = mix_group(layers, n_layers, total, i);
        if (g.vec) {
            const float4 v = *reinterpret_cast<const float4 *>(pool + i);
            const uint32_t m = *reinterpret_cast<const uint32_t *>(g.L.mask0 + g.e);
            uint32_t o = 0;
            o |= ((m & 0x000000FFu) || above(v.x)) ? 0x00000001u : 0u;
            o |= ((m & 0x0000FF00u) || above(v.y)) ? 0x00000100u : 0u;
            o |= ((m & 0x00FF0000u) || above(v.z)) ? 0x00010000u : 0u;
            o |= ((m & 0xFF000000u) || above(v.w)) ? 0x01000000u : 0u;
            *reinterpret_cast<uint32_t *>(g.L.out + g.e) = o;
        } else {
            for (int64_t j = i; j < min(i + 4, total); ++j) {
                const MixLayer L = layers[find_mix_layer(layers, n_layers, j)];
                const int64_t e = j - L.begin;
                L.out[e] = (L.mask0[e] || above(pool[j])) ? 1 : 0;
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// host side

namespace {

// Temporaries of one producer call come from a process-wide device buffer that only grows, so
// that a steady stream of calls does not pay for hipMalloc / hipFree.  The arena holds the
// buffer's lock for the duration of the call (producer calls are serialised).
std::mutex g_ws_mutex;
void *g_ws = nullptr;
size_t g_ws_size = 0;
int g_ws_device = -1; // the device the buffer lives on; calls on another device do not use it

class Arena {
public:
    // `s`: the stream the call queues its kernels on; the buffer is not handed to the next call
    // before that stream has run dry, whichever way the call ends (an error return after kernels
    // were queued included).
    explicit Arena(hipStream_t s) : lock_(g_ws_mutex), stream_(s)
    {
        if (hipGetDevice(&device_) != hipSuccess)
            device_ = -2;
        if (g_ws_device < 0)
            g_ws_device = device_;
        usable_ = device_ == g_ws_device;
    }
    ~Arena()
    {
        (void)hipStreamSynchronize(stream_);
        for (void *p : extras_)
            hipFree(p);
        if (usable_ && need_ > g_ws_size) { // grow for the next call
            hipFree(g_ws);
            g_ws = nullptr;
            g_ws_size = 0;
            const size_t want = need_ + need_ / 2;
            if (hipMalloc(&g_ws, want) == hipSuccess)
                g_ws_size = want;
        }
    }
    void *alloc(size_t bytes)
    {
        bytes = (bytes + 255) / 256 * 256;
        need_ += bytes;
        if (usable_ && off_ + bytes <= g_ws_size) {
            void *p = static_cast<char *>(g_ws) + off_;
            off_ += bytes;
            return p;
        }
        void *p = nullptr;
        if (hipMalloc(&p, bytes) != hipSuccess)
            return nullptr;
        extras_.push_back(p);
        return p;
    }
    template <class T> T *alloc_n(size_t n) { return static_cast<T *>(alloc(sizeof(T) * std::max<size_t>(n, 1))); }

private:
    std::lock_guard<std::mutex> lock_;
    hipStream_t stream_;
    int device_ = -1;
    bool usable_ = false;
    size_t off_ = 0, need_ = 0;
    std::vector<void *> extras_;
};

// The k-th (0-based) smallest of v[0..n) and its upper neighbour in sorted order.
struct Threshold {
    SelectState *state; // device; thr32 / thr64 are valid once the stream has run
    int is_f64;
};

// np.percentile(v, q) with linear interpolation for a float32 vector on the device, queued on the
// stream: four histogram passes of a radix select for the k-th smallest value, its upper
// neighbour, then the interpolation.  With q_is_f64 == 0 (q was a Python number) the quantile
// q/100, the virtual index (n-1)*quantile and the interpolation are float32; with 1 (q was a
// NumPy float64) they are float64, only the difference of the two neighbours stays float32.
int percentile_linear(Arena &ar, const float *d_v, int64_t n, double q, int q_is_f64, hipStream_t s,
                      Threshold *out, int n_segments = 1)
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
    const unsigned long long k = (unsigned long long)std::min(lo, n - 1);
    SelectState *st = ar.alloc_n<SelectState>(n_segments);
    if (!st)
        return fail(TW_ERR_ALLOC, "hipMalloc of the selection state failed");
    const int grid = (int)std::min<int64_t>(n_segments > 1 ? 64 : 1024, (n + 255) / 256);
    const dim3 g2(grid, n_segments), g1(n_segments);
    hipLaunchKernelGGL(select_init_kernel, g1, dim3(256), 0, s, st, k);
    for (int pass = 0; pass < 4; ++pass)
        hipLaunchKernelGGL(select_hist_kernel, g2, dim3(256), 0, s, d_v, n, pass, st);
    hipLaunchKernelGGL(rank_stats_kernel, g2, dim3(256), 0, s, d_v, n, st);
    hipLaunchKernelGGL(select_lerp_kernel, g1, dim3(256), 0, s, st, k, top ? 1 : 0, q_is_f64,
                       gamma32, gamma64);
    TW_HIP(hipGetLastError());
    out->state = st;
    out->is_f64 = q_is_f64;
    return TW_OK;
}

// waits for the stream and returns the threshold as a double
int read_threshold(const Threshold &t, hipStream_t s, double *value)
{
    // the words behind the histograms are all the host needs
    struct Tail {
        int32_t lost;
        float thr32;
        double thr64;
    } h;
    static_assert(offsetof(SelectState, thr64) - offsetof(SelectState, lost) == offsetof(Tail, thr64) &&
                      sizeof(SelectState) - offsetof(SelectState, lost) == sizeof(Tail),
                  "Tail mirrors the end of SelectState");
    TW_HIP(hipMemcpyAsync(&h, reinterpret_cast<const char *>(t.state) + offsetof(SelectState, lost),
                          sizeof(h), hipMemcpyDeviceToHost, s));
    TW_HIP(hipStreamSynchronize(s));
    if (h.lost)
        return fail(TW_ERR_DEVICE, "radix select lost its rank");
    *value = h.thr64;
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
int rows_stage(Arena &ar, int n_layers, const int32_t *K, const int32_t *N,
               const float *const *scores, std::vector<LayerTiles> &lt,
               const std::vector<uint8_t *> &d_colkeep, double q, int q_is_f64,
               uint8_t *const *masks, Threshold *thr, hipStream_t s, int flags = 0)
{
    int64_t total = 0, tab = 0;
    for (int l = 0; l < n_layers; ++l) {
        lt[l].norm_off = total;
        total += (int64_t)K[l] * ((int64_t)lt[l].tcol0.size() - 1);
        tab += (int64_t)lt[l].tcol0.size();
    }
    float *d_norms = ar.alloc_n<float>(total);
    // the layer table and the tile tables behind it share one buffer: one upload
    const size_t table_bytes = (sizeof(PruneLayer) * n_layers + 15) / 16 * 16;
    char *d_both = static_cast<char *>(ar.alloc(table_bytes + sizeof(int32_t) * tab));
    if (!d_norms || !d_both)
        return fail(TW_ERR_ALLOC, "hipMalloc of %lld norms failed", (long long)total);
    PruneLayer *d_table = reinterpret_cast<PruneLayer *>(d_both);
    int32_t *d_tables = reinterpret_cast<int32_t *>(d_both + table_bytes);
    std::vector<char> both(table_bytes + sizeof(int32_t) * tab, 0);
    PruneLayer *pl = reinterpret_cast<PruneLayer *>(both.data());
    int32_t *flat = reinterpret_cast<int32_t *>(both.data() + table_bytes);
    size_t n_flat = 0;
    int64_t n_pairs = 0, n_elems = 0;
    for (int l = 0; l < n_layers; ++l) {
        PruneLayer e;
        e.score = scores[l];
        e.mask = masks ? masks[l] : nullptr;
        e.colkeep = d_colkeep.empty() ? nullptr : d_colkeep[l];
        e.tcol0 = d_tables + n_flat;
        e.norms = d_norms + lt[l].norm_off;
        e.K = K[l];
        e.N = N[l];
        e.n_tiles = (int32_t)lt[l].tcol0.size() - 1;
        e.flags = flags;
        e.rt_begin = n_pairs;
        e.el_begin = n_elems;
        n_pairs += (int64_t)e.K * e.n_tiles;
        n_elems += (int64_t)((e.K + kFillRows - 1) / kFillRows) * ((e.N + 15) / 16);
        std::memcpy(&pl[l], &e, sizeof(e));
        std::memcpy(flat + n_flat, lt[l].tcol0.data(), sizeof(int32_t) * lt[l].tcol0.size());
        n_flat += lt[l].tcol0.size();
    }
    TW_HIP(hipMemcpyAsync(d_both, both.data(), both.size(), hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s)); // `both` is pageable host memory
    hipLaunchKernelGGL(tile_row_norms_kernel, dim3((unsigned)((n_pairs * 8 + 255) / 256)), dim3(256),
                       0, s, d_table, n_layers, n_pairs);
    TW_HIP(hipGetLastError());
    // per-tile thresholds (one layer): every tile's K norms are one segment
    const int n_seg = (flags & kPerTileThreshold) ? (int)lt[0].tcol0.size() - 1 : 1;
    int st = percentile_linear(ar, d_norms, total / n_seg, q, q_is_f64, s, thr, n_seg);
    if (st)
        return st;
    hipLaunchKernelGGL(fill_mask_kernel, dim3((unsigned)((n_elems + 255) / 256)), dim3(256), 0, s,
                       d_table, n_layers, n_elems, thr->state, thr->is_f64);
    TW_HIP(hipGetLastError());
    return TW_OK; // the caller reads the threshold back, which waits for the stream
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
try {
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
TW_CATCH_TO_STATUS

int tw_prune_tile_row_norms(int K, int N, const float *scores, int n_tiles,
                            const int32_t *tile_col0, const int32_t *tile_width,
                            const uint8_t *col_keep, float *norms, void *stream)
try {
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
    Arena ar(s);
    int32_t *d_tab = ar.alloc_n<int32_t>(n_tiles + 1);
    PruneLayer *d_table = ar.alloc_n<PruneLayer>(1);
    if (!d_tab || !d_table)
        return fail(TW_ERR_ALLOC, "hipMalloc of the tile table failed");
    PruneLayer e;
    e.score = scores;
    e.mask = nullptr;
    e.colkeep = col_keep;
    e.tcol0 = d_tab;
    e.norms = norms;
    e.K = K;
    e.N = N;
    e.n_tiles = n_tiles;
    e.flags = 0;
    e.rt_begin = 0;
    e.el_begin = 0;
    TW_HIP(hipMemcpyAsync(d_tab, tcol0.data(), sizeof(int32_t) * (n_tiles + 1), hipMemcpyHostToDevice, s));
    TW_HIP(hipMemcpyAsync(d_table, &e, sizeof(e), hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s));
    const int64_t n_pairs = (int64_t)K * n_tiles;
    hipLaunchKernelGGL(tile_row_norms_kernel, dim3((unsigned)((n_pairs * 8 + 255) / 256)), dim3(256), 0, s,
                       d_table, 1, n_pairs);
    TW_HIP(hipGetLastError());
    TW_HIP(hipStreamSynchronize(s));
    return TW_OK;
}
TW_CATCH_TO_STATUS

int tw_prune_col_norms(int K, int N, const float *scores, float *norms, void *stream)
try {
    if (K <= 0 || N <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d must be positive", K, N);
    if (!scores || !norms)
        return fail(TW_ERR_NULL, "a pointer is NULL");
    hipStream_t s = (hipStream_t)stream;
    Arena ar(s);
    ColLayer *d_cl = ar.alloc_n<ColLayer>(1);
    if (!d_cl)
        return fail(TW_ERR_ALLOC, "hipMalloc of the layer table failed");
    const ColLayer cl{scores, K, N, 0};
    TW_HIP(hipMemcpyAsync(d_cl, &cl, sizeof(cl), hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s));
    hipLaunchKernelGGL(col_norms_kernel, dim3((N + 63) / 64), dim3(64), 0, s, d_cl, 1, (int64_t)N, norms);
    TW_HIP(hipGetLastError());
    TW_HIP(hipStreamSynchronize(s));
    return TW_OK;
}
TW_CATCH_TO_STATUS

int tw_percentile_linear(const float *values, int64_t n, double q, int q_type, double *result,
                         void *stream)
try {
    if (!values || !result)
        return fail(TW_ERR_NULL, "a pointer is NULL");
    if (q_type != TW_Q_F32 && q_type != TW_Q_F64)
        return fail(TW_ERR_LAYOUT, "q_type=%d: unknown", q_type);
    Threshold t;
    Arena ar((hipStream_t)stream);
    int st = percentile_linear(ar, values, n, q, q_type, (hipStream_t)stream, &t);
    if (!st)
        st = read_threshold(t, (hipStream_t)stream, result);
    return st;
}
TW_CATCH_TO_STATUS

int tw_prune_tiled_wise_1d(int n_layers, const int32_t *K, const int32_t *N,
                           const float *const *scores, double sparsity, int q_type,
                           int granularity, uint8_t *const *masks, double *threshold, void *stream)
try {
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
    Arena ar((hipStream_t)stream);
    st = rows_stage(ar, n_layers, K, N, scores, lt, {}, sparsity, q_type, masks, &thr,
                    (hipStream_t)stream);
    double value = 0.0;
    if (!st)
        st = read_threshold(thr, (hipStream_t)stream, &value); // also: the masks are complete
    if (!st && threshold)
        *threshold = value;
    return st;
}
TW_CATCH_TO_STATUS

int tw_prune_granularity(int K, int N, const float *scores, double sparsity, int q_type,
                         int granularity, uint8_t *mask, void *stream)
try {
    const float *const sc[1] = {scores};
    uint8_t *const mk[1] = {mask};
    int st = check_layers(1, &K, &N, sc, mk, granularity);
    if (st)
        return st;
    if (q_type != TW_Q_F32 && q_type != TW_Q_F64)
        return fail(TW_ERR_LAYOUT, "q_type=%d: unknown", q_type);
    if (N % granularity != 0)
        return fail(TW_ERR_SHAPE, "N=%d is not a multiple of the granularity %d", N, granularity);
    std::vector<LayerTiles> lt(1);
    for (int c = 0; c <= N; c += granularity)
        lt[0].tcol0.push_back(c);
    Threshold thr;
    Arena ar((hipStream_t)stream);
    st = rows_stage(ar, 1, &K, &N, sc, lt, {}, sparsity, q_type, mk, &thr, (hipStream_t)stream,
                    kNormNotDivided | kPerTileThreshold);
    double value = 0.0;
    if (!st)
        st = read_threshold(thr, (hipStream_t)stream, &value); // waits for the mask
    return st;
}
TW_CATCH_TO_STATUS

int tw_prune_tiled_wise_2d(int n_layers, const int32_t *K, const int32_t *N,
                           const float *const *scores, double sparsity, int q_type, int transform,
                           int granularity, uint8_t *const *masks, uint8_t *const *col_masks,
                           double *thresholds, void *stream)
try {
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
    Arena ar((hipStream_t)stream);
    float *d_cnorm = ar.alloc_n<float>(total_n);
    uint8_t *d_ckeep = ar.alloc_n<uint8_t>(total_n);
    ColLayer *d_cl = ar.alloc_n<ColLayer>(n_layers);
    if (!d_cnorm || !d_ckeep || !d_cl)
        return fail(TW_ERR_ALLOC, "hipMalloc of %lld column norms failed", (long long)total_n);
    std::vector<ColLayer> cl(n_layers);
    for (int l = 0; l < n_layers; ++l)
        cl[l] = ColLayer{scores[l], K[l], N[l], coff[l]};
    TW_HIP(hipMemcpyAsync(d_cl, cl.data(), sizeof(ColLayer) * n_layers, hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s)); // `cl` is pageable host memory
    hipLaunchKernelGGL(col_norms_kernel, dim3((unsigned)((total_n + 63) / 64)), dim3(64), 0, s, d_cl,
                       n_layers, total_n, d_cnorm);
    TW_HIP(hipGetLastError());
    Threshold thr_c;
    st = percentile_linear(ar, d_cnorm, total_n, q, q_type, s, &thr_c);
    if (st)
        return st;
    hipLaunchKernelGGL(col_keep_kernel, dim3((unsigned)((total_n + 255) / 256)), dim3(256), 0, s,
                       d_cnorm, (int)total_n, thr_c.state, thr_c.is_f64, d_ckeep);
    TW_HIP(hipGetLastError());
    std::vector<uint8_t> h_keep(total_n);
    TW_HIP(hipMemcpyAsync(h_keep.data(), d_ckeep, (size_t)total_n, hipMemcpyDeviceToHost, s));
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
        d_colkeep[l] = d_ckeep + coff[l];
        if (col_masks && col_masks[l])
            TW_HIP(hipMemcpyAsync(col_masks[l], d_colkeep[l], (size_t)N[l], hipMemcpyDeviceToDevice, s));
    }
    Threshold thr_r;
    st = rows_stage(ar, n_layers, K, N, scores, lt, d_colkeep, q, q_type, masks, &thr_r, s);
    double vc = 0.0, vr = 0.0;
    if (!st)
        st = read_threshold(thr_c, s, &vc);
    if (!st)
        st = read_threshold(thr_r, s, &vr);
    if (!st && thresholds) {
        thresholds[0] = vc;
        thresholds[1] = vr;
    }
    return st;
}
TW_CATCH_TO_STATUS

int tw_prune_mix(int n_layers, const int32_t *K, const int32_t *N, const float *const *scores,
                 const uint8_t *const *layer_masks, double g1percent, int q_type,
                 uint8_t *const *masks, double *threshold, void *stream)
try {
    int st = check_layers(n_layers, K, N, scores, masks, 1);
    if (st)
        return st;
    if (!layer_masks)
        return fail(TW_ERR_NULL, "layer_masks is NULL");
    if (q_type != TW_Q_F32 && q_type != TW_Q_F64)
        return fail(TW_ERR_LAYOUT, "q_type=%d: unknown", q_type);
    hipStream_t s = (hipStream_t)stream;
    std::vector<MixLayer> ml(n_layers);
    int64_t total = 0;
    for (int l = 0; l < n_layers; ++l) {
        if (!layer_masks[l])
            return fail(TW_ERR_NULL, "layer %d: layer mask pointer is NULL", l);
        ml[l].score = scores[l];
        ml[l].mask0 = layer_masks[l];
        ml[l].out = masks[l];
        ml[l].begin = total;
        total += (int64_t)K[l] * N[l];
    }
    Arena ar(s);
    float *d_pool = ar.alloc_n<float>(total);
    MixLayer *d_layers = ar.alloc_n<MixLayer>(n_layers);
    if (!d_pool || !d_layers)
        return fail(TW_ERR_ALLOC, "hipMalloc of %lld element scores failed", (long long)total);
    TW_HIP(hipMemcpyAsync(d_layers, ml.data(), sizeof(MixLayer) * n_layers, hipMemcpyHostToDevice, s));
    TW_HIP(hipStreamSynchronize(s)); // `ml` is pageable host memory
    const unsigned grid = (unsigned)std::min<int64_t>((total + 1023) / 1024, 256 * 32);
    hipLaunchKernelGGL(mix_values_kernel, dim3(grid), dim3(256), 0, s, d_layers, n_layers, total,
                       d_pool);
    TW_HIP(hipGetLastError());
    Threshold thr;
    st = percentile_linear(ar, d_pool, total, 100.0 - g1percent, q_type, s, &thr);
    if (st)
        return st;
    hipLaunchKernelGGL(mix_mask_kernel, dim3(grid), dim3(256), 0, s, d_layers, n_layers, total,
                       d_pool, thr.state, thr.is_f64);
    TW_HIP(hipGetLastError());
    double value = 0.0;
    st = read_threshold(thr, s, &value); // waits for the masks
    if (!st && threshold)
        *threshold = value;
    return st;
}
TW_CATCH_TO_STATUS

} // extern "C"
