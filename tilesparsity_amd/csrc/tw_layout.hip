// Row-major operands at the speed of the K-major kernels (tw_gemm_staged): the reference's Python
// operator multiplies a row-major x[M,K] into a row-major [M,N] result (mask_dense,
// Pruning/BERT/utils/modeling.py:992-1007), its CUDA driver a column-major A into a column-major C
// (Stream_Gemm_NN, StreamMaskedGEMM/perf/basic_nn.cu:378-445).  The TW kernels gather whole kept
// rows of a K-major A; from a row-major A a kept k is one 2-byte element per row.  So a
// row-major operand is turned into its K-major copy in a workspace the caller brings (one pass
// over the operand at the memory rate), the K-major kernel runs, and a row-major C is turned
// back.  Nothing is allocated here.
#include "tw_internal.h"

namespace tw {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// dst[c * ld_dst + r] = src[r * ld_src + c] for r < rows, c < cols, 16-bit elements, in tiles of
// T x T through LDS: 16-byte loads along the rows of src, 16-byte stores along the rows of dst
// (128 contiguous bytes per row of a tile on either side; 128 x 128 tiles measured slower).
// ld_src is a multiple of 8, so a chunk of 8 elements that starts below cols ends inside the
// row's allocation.  A chunk of 8 destination elements that ends beyond `rows` is written whole
// when the destination's rows are padded (`dst_padded`: a workspace), else element by element.
constexpr int kTransposeTile = 64;

__global__ void __launch_bounds__(256)
    transpose16_kernel(const uint16_t *__restrict__ src, int64_t ld_src, int rows, int cols,
                       uint16_t *__restrict__ dst, int64_t ld_dst, int dst_padded)
{
    constexpr int T = kTransposeTile, CH = T / 8, PITCH = T + 8; // rows 16-byte aligned, 4 banks apart
    constexpr int PER_THREAD = T * CH / 256;
    __shared__ __align__(16) uint16_t tile[T * PITCH];
    const int r0 = blockIdx.y * T, c0 = blockIdx.x * T;
    const int tid = threadIdx.x;
#pragma unroll
    for (int q = 0; q < PER_THREAD; ++q) {
        const int idx = tid + q * 256;
        const int r = idx / CH, cc = (idx % CH) * 8;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (r0 + r < rows && c0 + cc < cols)
            v = *reinterpret_cast<const u32x4 *>(src + (int64_t)(r0 + r) * ld_src + c0 + cc);
        *reinterpret_cast<u32x4 *>(tile + r * PITCH + cc) = v;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < PER_THREAD; ++q) {
        const int idx = tid + q * 256;
        const int c = idx / CH, rc = (idx % CH) * 8;
        if (c0 + c >= cols || r0 + rc >= rows)
            continue;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            w[e] = (uint32_t)tile[(rc + 2 * e) * PITCH + c] |
                   ((uint32_t)tile[(rc + 2 * e + 1) * PITCH + c] << 16);
        uint16_t *out = dst + (int64_t)(c0 + c) * ld_dst + r0 + rc;
        if (dst_padded || r0 + rc + 8 <= rows) {
            const u32x4 v = {w[0], w[1], w[2], w[3]};
            *reinterpret_cast<u32x4 *>(out) = v;
        } else {
            for (int e = 0; r0 + rc + e < rows; ++e)
                out[e] = (uint16_t)(w[e >> 1] >> ((e & 1) * 16));
        }
    }
}

int transpose16(const void *src, int64_t ld_src, int rows, int cols, void *dst, int64_t ld_dst,
                bool dst_padded, hipStream_t s)
{
    if (rows <= 0 || cols <= 0)
        return TW_OK;
    constexpr int T = kTransposeTile;
    const dim3 grid((unsigned)((cols + T - 1) / T), (unsigned)((rows + T - 1) / T));
    if (grid.y > 65535u)
        return fail(TW_ERR_SHAPE, "%d rows: the layout kernels take at most %d", rows, 65535 * T);
    hipLaunchKernelGGL(transpose16_kernel, grid, dim3(256), 0, s, (const uint16_t *)src, ld_src, rows,
                       cols, (uint16_t *)dst, ld_dst, dst_padded ? 1 : 0);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int64_t staged_ld(int M) { return ((int64_t)M + 63) / 64 * 64; }

} // namespace
} // namespace tw

using namespace tw;

extern "C" int64_t tw_gemm_staged_workspace(const tw_plan *plan, int M, int a_layout, int c_layout)
{
    if (!plan || M <= 0)
        return 0;
    int64_t rows = 0;
    if (a_layout == TW_LAYOUT_ROWMAJOR)
        rows += plan->K;
    if (c_layout == TW_LAYOUT_ROWMAJOR)
        rows += plan->N;
    return rows * staged_ld(M) * 2;
}

extern "C" int tw_gemm_staged(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C,
                              int c_layout, int64_t ldc, int M, float alpha, float beta,
                              int pruned_cols, const tw_epilogue *ep, void *workspace,
                              int64_t workspace_bytes, void *stream)
try {
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    const bool a_rm = a_layout == TW_LAYOUT_ROWMAJOR, c_rm = c_layout == TW_LAYOUT_ROWMAJOR;
    if ((!a_rm && !c_rm) || M <= 0 || !A || !C || (a_rm && c_rm && takes_row_major_directly(plan, beta)))
        return tw_gemm_ex(plan, A, a_layout, lda, C, c_layout, ldc, M, alpha, beta, pruned_cols, ep,
                          stream); // nothing to stage (K-major operands, or row-major ones a GEMM
                                   // kernel takes as they are); also reports every argument error
    if ((a_rm && (lda < plan->K || (lda & 7))) || (c_rm && (ldc < plan->N || (ldc & 7))) ||
        ((uintptr_t)A & 15) || ((uintptr_t)C & 15))
        return tw_gemm_ex(plan, A, a_layout, lda, C, c_layout, ldc, M, alpha, beta, pruned_cols, ep,
                          stream); // reports the error
    // (row-major operands the GEMM kernels take directly need no staging: tw_gemm_ex tells)
    const int64_t need = tw_gemm_staged_workspace(plan, M, a_layout, c_layout);
    if (!workspace || workspace_bytes < need)
        return fail(TW_ERR_BUFFER, "workspace of %lld bytes, %lld needed (tw_gemm_staged_workspace)",
                    (long long)(workspace ? workspace_bytes : 0), (long long)need);
    if ((uintptr_t)workspace & 15)
        return fail(TW_ERR_ALIGNMENT, "the workspace must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int64_t ldw = staged_ld(M);
    uint16_t *ws = static_cast<uint16_t *>(workspace);
    const void *Ak = A;
    int64_t lda_k = lda;
    if (a_rm) {
        // A [M][lda] -> A^T [K][ldw]
        const int st = transpose16(A, lda, M, plan->K, ws, ldw, true, s);
        if (st != TW_OK)
            return st;
        Ak = ws;
        lda_k = ldw;
        ws += (int64_t)plan->K * ldw;
    }
    void *Ck = C;
    int64_t ldc_k = ldc;
    if (c_rm) {
        Ck = ws;
        ldc_k = ldw;
        // The K-major kernel leaves columns alone that no tile covers, and pruned columns unless
        // they are to be filled; beta reads C.  In those cases the old C goes in first.
        int64_t covered = 0;
        for (int w : plan->tile_width)
            covered += w;
        const bool writes_all = pruned_cols == TW_PRUNED_ZERO && beta == 0.0f && covered == plan->N;
        if (!writes_all) {
            const int st = transpose16(C, ldc, M, plan->N, Ck, ldw, true, s);
            if (st != TW_OK)
                return st;
        }
    }
    const int st = tw_gemm_ex(plan, Ak, TW_LAYOUT_KMAJOR, lda_k, Ck, TW_LAYOUT_KMAJOR, ldc_k, M, alpha,
                              beta, pruned_cols, ep, stream);
    if (st != TW_OK)
        return st;
    if (c_rm) // C^T [N][ldw] -> C [M][ldc]; nothing beyond column N of a row of C is written
        return transpose16(Ck, ldw, plan->N, M, C, ldc, false, s);
    return TW_OK;
}
TW_CATCH_TO_STATUS
