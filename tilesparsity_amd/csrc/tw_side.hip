// The element-wise remainder of a mixed mask next to its tile-wise part.  The reference's mixed
// producers (tiled_wise_1d_mix / tiled_wise_2d_mix, Pruning/VGG/prune_algo.py:151-193) keep a
// tile-wise mask plus the g1percent largest of the elements it drops; the tile-wise part runs as
// a plan on the matrix cores, and this file adds  C += alpha * A * R  for the remainder R, a K x N
// matrix with about one element in a hundred set and no structure.
//
// K-major A and C make a column of the product a sum of scaled rows:
//   C[n][m] += alpha * sum_i v_i * A[k_i][m]   over the elements (k_i, n) of column n of R,
// contiguous in m on both sides, so the lanes run along m and nothing is transposed or gathered
// at element granularity.  A workgroup of four waves takes one column for a chunk of 256 rows m;
// a lane owns 4 rows m.  The elements of a column lie in memory as (k, v) pairs in batches of
// four (padded with v = 0); wave w takes the batches w, w + 4, ...: it reads a batch with one
// scalar load, so k and v are scalars - the row address is a scalar base plus the lane's fixed
// offset, the weight a scalar operand of the multiply-add - and a lane reads 8 bytes of row k_i
// and multiplies them into 4 fp32 sums.  The four waves' sums meet in LDS, wave 0 adds them in
// wave order and adds the result into C (read, add, one rounding, write).  v is the weight
// rounded to the 16-bit type, held in fp32.
//
// Every row of A is wanted by about N / 100 columns.  An accelerator die takes whole chunks
// (all K rows, 256 rows m: 2.4 MB for K = 4608), chunk after chunk, its workgroups side by side
// on the chunk's columns, so that a chunk comes from memory once and from that die's L2 for the
// other columns.  Measured (M 12544, K 4608, N 512, 1 % of the elements, fp16): 60 us, 4.7 TB/s
// from memory - twice A: with the 8 MB of loads in flight that the L2 latency asks for, the L2s
// take part of the lines without keeping them (a quarter of the workgroups fetch A once, and
// take 88 us).  The pass reads all of A whatever the remainder holds (28 us for 0.1 %), so on that
// shape the covering plan (tw_plan_from_mask_cover) is faster at every density measured (0.1 to
// 5 %); the pair can only come out ahead for a small remainder on a layer so wide that the pass
// over A is a small part of it.
#include "tw_internal.h"

#include <algorithm>
#include <memory>
#include <numeric>

struct tw_side {
    int K = 0, N = 0, dtype = 0, device = 0;
    int64_t nnz = 0;
    int n_cols = 0;                 // columns with at least one element
    int cu_count = 0;
    int32_t *d_cols = nullptr;      // [n_cols][4]: column number, its first batch in d_entries, its batches
                                    // of four elements, 0; columns with most elements first
    int32_t *d_entries = nullptr;   // batches of four (k, v as fp32 bits) pairs
    void *d_slab = nullptr;         // the one allocation behind the two
};

namespace tw {
namespace {

constexpr int kSideChunk = 256;   // rows m of a work item
constexpr int kSideBatch = 4;     // elements of a batch
constexpr int kSideWaves = 4;     // waves of a workgroup
constexpr int kSideWgsPerCu = 8;  // workgroups per compute unit

struct SideArgs {
    const int32_t *cols, *entries;
    const uint16_t *A;
    uint16_t *C;
    int64_t lda, ldc;
    int32_t M, n_cols, n_chunks;
    float alpha;
};

__device__ __forceinline__ float side_from16(uint32_t b, int dtype)
{
    if (dtype == TW_F16)
        return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
    return __builtin_bit_cast(float, b << 16);
}

__device__ __forceinline__ uint32_t side_to16(float f, int dtype)
{
    if (dtype == TW_F16)
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}

// the weight values of the entries: rounded to the 16-bit type like the packed weight of a plan
__global__ void side_round_kernel(int32_t *entries, int64_t n_pairs, int dtype)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_pairs) {
        const float v = __builtin_bit_cast(float, entries[2 * i + 1]);
        entries[2 * i + 1] = __builtin_bit_cast(int32_t, side_from16(side_to16(v, dtype), dtype));
    }
}

typedef unsigned int su32x2 __attribute__((ext_vector_type(2)));

template <int DT> __global__ void __launch_bounds__(64 * kSideWaves, kSideWgsPerCu) tw_side_kernel(const SideArgs p)
{
    __shared__ float part[2][kSideWaves][64 * 4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // The work of this die: whole row chunks die, die + 8, ... with all their columns, so that
    // its workgroups are on one chunk of A at a time; of the chunks left over at the end (fewer
    // than 8) every die takes an eighth of the columns.  The workgroups of a die take the
    // columns of a chunk in turn.
    const int die = blockIdx.x % kXcd, slot = blockIdx.x / kXcd;
    const int n_slots = gridDim.x / kXcd;
    const int n_whole = p.n_chunks / kXcd * kXcd;
    const uint32_t lane_off = (uint32_t)lane * 8u; // bytes of this lane's rows m inside a chunk
    const unsigned char *const A = reinterpret_cast<const unsigned char *>(p.A);
    const uint64_t lda_b = (uint64_t)p.lda * 2u;
    int flip = 0;
    int mc = die < n_whole ? die : n_whole; // current chunk
    int c_end = mc < n_whole ? p.n_cols : (int)((int64_t)p.n_cols * (die + 1) / kXcd);
    int c_begin = mc < n_whole ? 0 : (int)((int64_t)p.n_cols * die / kXcd);
    int ci = slot; // position among the columns [c_begin, c_end) of the chunk
    for (;;) {
        while (ci >= (c_end - c_begin + n_slots - 1) / n_slots * n_slots && mc < p.n_chunks) { // on to this die's next chunk
            mc = mc < n_whole ? (mc + kXcd < n_whole ? mc + kXcd : n_whole) : mc + 1;
            c_end = mc < n_whole ? p.n_cols : (int)((int64_t)p.n_cols * (die + 1) / kXcd);
            c_begin = mc < n_whole ? 0 : (int)((int64_t)p.n_cols * die / kXcd);
            ci = slot;
        }
        if (mc >= p.n_chunks)
            break;
        // The columns are sorted by their number of elements and dealt out in a serpentine (pass 0:
        // workgroup s takes column s, pass 1: column 2 S - 1 - s, ...), so that the workgroups of a
        // die finish a chunk at about the same time: if those with short columns ran chunks ahead,
        // the die would work on several chunks of A at once and they would not fit its L2 together.
        const int pass = ci / n_slots;
        const int cr = c_begin + pass * n_slots + ((pass & 1) ? n_slots - 1 - slot : slot);
        if (cr >= c_end) {
            ci += n_slots;
            continue;
        }
        const auto *col = (const __attribute__((address_space(4))) int32_t *)(uintptr_t)p.cols + (int64_t)cr * 4;
        const int n = col[0], ptr = col[1], nb = col[2];
        const int m = mc * kSideChunk + lane * 4;
        // rows past M: a lane reads the chunk's first rows instead and stores nothing
        const unsigned char *const a_chunk = A + (uint64_t)mc * (kSideChunk * 2);
        const bool m_in = m < p.M && lane * 4 < kSideChunk;
        const uint32_t a_off = m_in ? lane_off : 0u;
        uint16_t *const c_lane = p.C + (int64_t)n * p.ldc + m;
        su32x2 old = {0u, 0u};
        if (wave == 0 && m_in)
            old = *reinterpret_cast<const su32x2 *>(c_lane);
        const auto *ent = (const __attribute__((address_space(4))) int32_t *)(uintptr_t)p.entries +
                          (int64_t)ptr * (2 * kSideBatch);
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        struct Batch {
            su32x2 a[kSideBatch];
            float v[kSideBatch];
        };
        auto fetch = [&](int b) {
            Batch r;
#pragma unroll
            for (int i = 0; i < kSideBatch; ++i) {
                const int k = ent[b * (2 * kSideBatch) + 2 * i];
                r.v[i] = __builtin_bit_cast(float, ent[b * (2 * kSideBatch) + 2 * i + 1]);
                // the row's address in scalar registers, the lane's offset on top
                const uint64_t row = (uint64_t)(uintptr_t)a_chunk + (uint64_t)(uint32_t)k * lda_b;
                const uint64_t row_s = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(row >> 32)) << 32) |
                                       (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)row);
                r.a[i] = *(const __attribute__((address_space(1))) su32x2 *)(
                    (const __attribute__((address_space(1))) unsigned char *)row_s + a_off);
            }
            return r;
        };
        auto multiply = [&](const Batch &r) {
#pragma unroll
            for (int i = 0; i < kSideBatch; ++i) {
                acc[0] = fmaf(side_from16(r.a[i].x & 0xFFFFu, DT), r.v[i], acc[0]);
                acc[1] = fmaf(side_from16(r.a[i].x >> 16, DT), r.v[i], acc[1]);
                acc[2] = fmaf(side_from16(r.a[i].y & 0xFFFFu, DT), r.v[i], acc[2]);
                acc[3] = fmaf(side_from16(r.a[i].y >> 16, DT), r.v[i], acc[3]);
            }
        };
        // two register sets: one batch is multiplied while the loads of the next are in flight
        if (wave < nb) {
            Batch b0 = fetch(wave), b1 = {};
            for (int b = wave;;) {
                if (b + kSideWaves < nb)
                    b1 = fetch(b + kSideWaves);
                multiply(b0);
                if ((b += kSideWaves) >= nb)
                    break;
                if (b + kSideWaves < nb)
                    b0 = fetch(b + kSideWaves);
                multiply(b1);
                if ((b += kSideWaves) >= nb)
                    break;
            }
        }
        *reinterpret_cast<float4 *>(&part[flip][wave][lane * 4]) = float4{acc[0], acc[1], acc[2], acc[3]};
        __syncthreads();
        if (wave == 0 && m_in) {
            float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int w = 0; w < kSideWaves; ++w) {
                const float4 q = *reinterpret_cast<const float4 *>(&part[flip][w][lane * 4]);
                sum[0] += q.x;
                sum[1] += q.y;
                sum[2] += q.z;
                sum[3] += q.w;
            }
            const uint32_t q[2] = {old.x, old.y};
            uint32_t h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = side_from16((q[e >> 1] >> ((e & 1) * 16)) & 0xFFFFu, DT) + p.alpha * sum[e];
                asm volatile("" : "+v"(v)); // rounded to fp32, then to 16 bits
                h[e] = side_to16(v, DT);
            }
            if (m + 4 <= p.M) {
                *reinterpret_cast<su32x2 *>(c_lane) = su32x2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
            } else {
                for (int e = 0; e < p.M - m; ++e)
                    c_lane[e] = (uint16_t)h[e];
            }
        }
        ci += n_slots;
        flip ^= 1;
    }
}

} // namespace
} // namespace tw

using namespace tw;

extern "C" {

int tw_side_create(int K, int N, int dtype, const uint8_t *mask, const float *B, tw_side **out)
try {
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (dtype != TW_F16 && dtype != TW_BF16)
        return fail(TW_ERR_DTYPE, "dtype %d is neither TW_F16 nor TW_BF16", dtype);
    if (K <= 0 || N <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d must be positive", K, N);
    if (!mask || !B)
        return fail(TW_ERR_NULL, "mask or B is NULL");
    // the elements of every column, rows ascending
    std::vector<int32_t> count(N, 0);
    for (int64_t k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n)
            count[n] += mask[k * N + n] != 0;
    std::vector<int32_t> cols;
    for (int n = 0; n < N; ++n)
        if (count[n])
            cols.push_back(n);
    std::stable_sort(cols.begin(), cols.end(), [&](int a, int b) { return count[a] > count[b]; });
    std::unique_ptr<tw_side> s(new tw_side);
    s->K = K;
    s->N = N;
    s->dtype = dtype;
    s->n_cols = (int)cols.size();
    s->nnz = std::accumulate(count.begin(), count.end(), (int64_t)0);
    TW_HIP(hipGetDevice(&s->device));
    hipDeviceProp_t prop;
    TW_HIP(hipGetDeviceProperties(&prop, s->device));
    s->cu_count = prop.multiProcessorCount;
    std::vector<int32_t> col_info(cols.size() * 4, 0), slot_of(N, -1);
    int64_t batches = 0;
    for (size_t i = 0; i < cols.size(); ++i) {
        col_info[4 * i] = cols[i];
        col_info[4 * i + 1] = (int32_t)batches;
        col_info[4 * i + 2] = (count[cols[i]] + kSideBatch - 1) / kSideBatch;
        batches += col_info[4 * i + 2];
        slot_of[cols[i]] = (int)i;
        if (batches > 0x7fffffff / (2 * kSideBatch))
            return fail(TW_ERR_SHAPE, "%lld elements: more than the remainder's 32-bit offsets take",
                        (long long)s->nnz);
    }
    // padding: row 0 with a zero weight
    std::vector<int32_t> entries((size_t)batches * 2 * kSideBatch, 0);
    std::vector<int32_t> fill(cols.size(), 0);
    for (int64_t k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n)
            if (mask[k * N + n]) {
                const int i = slot_of[n];
                const size_t at = ((size_t)col_info[4 * i + 1] * kSideBatch + fill[i]++) * 2;
                entries[at] = (int32_t)k;
                const float v = B[k * N + n];
                __builtin_memcpy(&entries[at + 1], &v, 4);
            }
    if (!cols.empty()) {
        auto up = [](size_t b) { return (b + 255) / 256 * 256; };
        const size_t o_ent = up(col_info.size() * 4), total = o_ent + up(entries.size() * 4);
        if (hipMalloc(&s->d_slab, total) != hipSuccess) {
            (void)hipGetLastError();
            return fail(TW_ERR_ALLOC, "out of device memory (%zu bytes for the remainder)", total);
        }
        char *slab = static_cast<char *>(s->d_slab);
        s->d_cols = reinterpret_cast<int32_t *>(slab);
        s->d_entries = reinterpret_cast<int32_t *>(slab + o_ent);
        auto copy = [&](void *dst, const void *src, size_t n) { return hipMemcpy(dst, src, n, hipMemcpyHostToDevice); };
        hipError_t e = copy(s->d_cols, col_info.data(), col_info.size() * 4);
        if (e == hipSuccess)
            e = copy(s->d_entries, entries.data(), entries.size() * 4);
        if (e == hipSuccess) {
            const int64_t n_pairs = (int64_t)entries.size() / 2;
            hipLaunchKernelGGL(side_round_kernel, dim3((unsigned)((n_pairs + 255) / 256)), dim3(256), 0, nullptr,
                               s->d_entries, n_pairs, dtype);
            e = hipGetLastError();
            if (e == hipSuccess)
                e = hipStreamSynchronize(nullptr);
        }
        if (e != hipSuccess) {
            (void)hipFree(s->d_slab);
            return fail(TW_ERR_DEVICE, "building the remainder failed: %s", hipGetErrorString(e));
        }
    }
    *out = s.release();
    return TW_OK;
}
TW_CATCH_TO_STATUS

void tw_side_destroy(tw_side *side)
{
    if (!side)
        return;
    if (side->d_slab)
        (void)hipFree(side->d_slab);
    delete side;
}

int64_t tw_side_nnz(const tw_side *side) { return side ? side->nnz : 0; }

int tw_side_gemm(const tw_side *side, const void *A, int64_t lda, void *C, int64_t ldc, int M, float alpha,
                 void *stream)
{
    if (!side)
        return fail(TW_ERR_NULL, "side is NULL");
    if (M < 0)
        return fail(TW_ERR_SHAPE, "M=%d is negative", M);
    if (M == 0 || side->n_cols == 0)
        return TW_OK;
    if (!A || !C)
        return fail(TW_ERR_NULL, "A or C is NULL");
    if (lda < M || ldc < M)
        return fail(TW_ERR_SHAPE, "lda=%lld ldc=%lld must be >= M=%d", (long long)lda, (long long)ldc, M);
    if ((lda & 7) || (ldc & 7))
        return fail(TW_ERR_ALIGNMENT, "lda=%lld and ldc=%lld must be multiples of 8 elements", (long long)lda,
                    (long long)ldc);
    if (((uintptr_t)A & 15) || ((uintptr_t)C & 15))
        return fail(TW_ERR_ALIGNMENT, "A and C must be 16-byte aligned");
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    if (dev != side->device)
        return fail(TW_ERR_DEVICE, "the remainder was built on device %d, the current device is %d", side->device,
                    dev);
    SideArgs a;
    a.cols = side->d_cols;
    a.entries = side->d_entries;
    a.A = static_cast<const uint16_t *>(A);
    a.C = static_cast<uint16_t *>(C);
    a.lda = lda;
    a.ldc = ldc;
    a.M = M;
    a.n_cols = side->n_cols;
    a.n_chunks = (M + kSideChunk - 1) / kSideChunk;
    a.alpha = alpha;
    // as many workgroups as the chip holds at once, or as there are items
    const int64_t items = (int64_t)a.n_chunks * a.n_cols;
    if (items > 0x7fffffff)
        return fail(TW_ERR_SHAPE, "%lld work items (M=%d): a launch takes at most %d", (long long)items, M, 0x7fffffff);
    int64_t wgs = std::min<int64_t>((int64_t)side->cu_count * kSideWgsPerCu, items + kXcd);
    wgs = std::max<int64_t>(kXcd, wgs / kXcd * kXcd);
    if (side->dtype == TW_F16)
        hipLaunchKernelGGL((tw_side_kernel<TW_F16>), dim3((unsigned)wgs), dim3(64 * kSideWaves), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((tw_side_kernel<TW_BF16>), dim3((unsigned)wgs), dim3(64 * kSideWaves), 0, (hipStream_t)stream, a);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

} // extern "C"
