// The tile-wise-sparse GEMM of libtwgemm: one persistent grouped kernel for gfx950.
//
// Work decomposition.  A work item is (unit, m-block): a unit is up to 128
// compact columns of one weight tile, an m-block is BM consecutive rows of A.
// Units are sorted by kept-K descending at plan time, so ticket order hands out
// the heaviest items first (longest-processing-time order); workgroups take
// tickets from a global counter until the queue is empty.  With
// TW_PRUNED_ZERO the queue ends with zero-fill items for the pruned columns.
//
// Data path of one item (K-major layout: A[k*lda + m], C[n*ldc + m]):
//   * the kept K rows of A are gathered row by row: every gathered row is one
//     contiguous M-vector, fetched as 16-byte pieces (256 B per 16 lanes) and
//     staged in LDS as [k][m];
//   * the MFMA A operand (32 m x 16 k per instruction, 8 k per lane) is read
//     from that [k][m] stage with the transposing LDS read ds_read_b64_tr_b16;
//   * the MFMA B operand comes straight from the packed weight (already in
//     per-lane operand order, 16 bytes per lane, 1 KiB per wave), no LDS;
//   * v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulators;
//   * epilogue: alpha/beta in fp32, round to the 16-bit type, transpose through
//     LDS, then scatter whole C columns (col0 + kept_n[j]) with 16-byte stores.
#include "tw_internal.h"

#include <atomic>
#include <cstdlib>

namespace tw {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define TW_LDS(T) __attribute__((address_space(3))) T *

template <int DT> struct Elem;
template <> struct Elem<TW_F16> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t to_bits(float f)
    {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
    static __device__ __forceinline__ float from_bits(uint16_t h)
    {
        return (float)__builtin_bit_cast(_Float16, h);
    }
};
template <> struct Elem<TW_BF16> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t to_bits(float f)
    {
        uint32_t x = __float_as_uint(f);
        if ((x & 0x7F800000u) == 0x7F800000u && (x & 0x007FFFFFu))
            return (x >> 16) | 0x0040u;
        x += 0x7FFFu + ((x >> 16) & 1u);
        return x >> 16;
    }
    static __device__ __forceinline__ float from_bits(uint16_t h)
    {
        return __uint_as_float((uint32_t)h << 16);
    }
};

// 16-byte chunk of column c, rows m..m+7 of a K-major matrix, honouring the M edge
__device__ __forceinline__ void store_chunk(uint16_t *dst, u32x4 v, int m, int M)
{
    if (m + 8 <= M) {
        *reinterpret_cast<u32x4 *>(dst) = v;
    } else if (m < M) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        for (int e = 0; e < M - m; ++e)
            dst[e] = (uint16_t)(w[e >> 1] >> ((e & 1) * 16));
    }
}

template <int DT, int WM, int WN, bool TR>
__global__ void __launch_bounds__(64 * WM * WN, 2) tw_gemm_kmajor_kernel(const GemmArgs p)
{
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 64 * WM;
    constexpr int BN = 64 * WN;
    constexpr int BK = kBlockK;
    constexpr int CPR = BM / 8;       // 16-byte chunks per staged row / stored column
    constexpr int RPP = NT / CPR;     // rows (columns) covered by one pass of the block
    constexpr int PASSES = BK / RPP;
    constexpr int PITCH = BM + 16;    // halfs; +32 B keeps the 4 rows of a transposed read apart
    constexpr int STAGE = BK * PITCH;
    constexpr int CPITCH = BM + 8;
    constexpr int SMEM = (2 * STAGE > BN * CPITCH) ? 2 * STAGE : BN * CPITCH;
    constexpr int D = BM >= 256 ? 2 : 3; // prefetch distance in steps (24-32 KiB of A in flight)
    constexpr int R = D + 1;         // register ring slots; the main loop is unrolled R times
    constexpr int RPW = 64 / CPR;    // staged rows covered by one wave in one pass
    typedef int IdxVec __attribute__((ext_vector_type(RPW)));
    using E = Elem<DT>;

    __shared__ __align__(16) uint16_t smem[SMEM];
    __shared__ int s_item;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = __builtin_amdgcn_readfirstlane(wave % WM);
    const int wn = __builtin_amdgcn_readfirstlane(wave / WM);
    const int chunk = tid % CPR;
    const int rrow = tid / CPR;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int sub = lane / CPR;
    const uint16_t *const A = reinterpret_cast<const uint16_t *>(p.A);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    const uint16_t *const Bp = reinterpret_cast<const uint16_t *>(p.Bp);

    for (;;) {
        if (tid == 0)
            s_item = atomicAdd(&p.ticket[0], 1);
        __syncthreads();
        const int item = s_item;
        if (item >= p.n_items)
            break;

        if (item >= p.n_gemm_items) {
            // ---- zero-fill item: pruned columns of one tile receive beta*C ----
            const int z = item - p.n_gemm_items;
            const int zt = z / p.n_mblk;
            const int m = (z - zt * p.n_mblk) * BM + chunk * 8;
            const TileDev t = p.tiles[zt];
            for (int j = rrow; j < t.n_pruned; j += RPP) {
                const int c = t.col0 + p.pruned_n[t.pn_off + j];
                uint16_t *dst = C + (int64_t)c * p.ldc + m;
                u32x4 v = {0u, 0u, 0u, 0u};
                if (p.beta != 0.0f && m < p.M) {
                    uint32_t w[4] = {0u, 0u, 0u, 0u};
                    for (int e = 0; e < 8 && m + e < p.M; ++e)
                        w[e >> 1] |= E::to_bits(p.beta * E::from_bits(dst[e])) << ((e & 1) * 16);
                    v.x = w[0];
                    v.y = w[1];
                    v.z = w[2];
                    v.w = w[3];
                }
                store_chunk(dst, v, m, p.M);
            }
            __syncthreads();
            continue;
        }

        // ---- GEMM item ----------------------------------------------------------
        const int ui = item / p.n_mblk;
        const int m0 = (item - ui * p.n_mblk) * BM;
        const UnitDev u = p.units[ui];
        const int nsteps = u.k_pad / BK;
        const int32_t *const klist = p.kept_k + u.kk_off; // padded to k_pad entries
        const int m_ld = m0 + chunk * 8;
        const bool m_ok = m_ld < p.M;
        const int m_eff = m_ok ? m_ld : 0; // a valid chunk to read when this one is beyond M
        const int ksteps16 = u.k_pad / kMfmaK;
        // packed weight operand streams of this wave's two 32-column blocks; a block
        // beyond the unit reads block 0 (its products land in columns that are not stored)
        const uint16_t *b_base[2];
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int nb = wn * 2 + ni;
            b_base[ni] = Bp + u.b_off +
                         ((int64_t)(u.nb0 + (nb < u.nb_cnt ? nb : 0)) * ksteps16 * 64 + lane) * 8;
        }

        f32x16 acc[2][2];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[mi][ni][r] = 0.0f;

        // Register ring: the loads of step s+D are issued while step s is consumed, so D
        // steps of gathered A rows (and of packed weight operands) are in flight per
        // workgroup.  Loads return in order, so A and B share one prefetch distance.
        // The kept-K indices of a step are wave-uniform per 16-byte-chunk row group and come
        // through the scalar cache one step ahead of the loads that use them.
        auto load_idx = [&](int s, IdxVec(&ix)[PASSES]) {
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const int kkbase = s * BK + ps * RPP + wave_u * RPW;
                ix[ps] = *reinterpret_cast<const __attribute__((address_space(4))) IdxVec *>(
                    (uintptr_t)(klist + kkbase));
            }
        };
        // No lane-dependent branches here: rows beyond K_t and chunks beyond M are loaded
        // from a valid address and replaced by zeros when they are staged (not here, so that
        // nothing waits on a load that was just issued).
        auto issue = [&](int s, const IdxVec(&ix)[PASSES], u32x4(&ar)[PASSES], u32x4(&br)[2][2]) {
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                int my = ix[ps][0];
#pragma unroll
                for (int q = 1; q < RPW; ++q)
                    my = sub == q ? ix[ps][q] : my;
                ar[ps] = *reinterpret_cast<const u32x4 *>(A + (int64_t)my * p.lda + m_eff);
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    br[ks][ni] = *reinterpret_cast<const u32x4 *>(
                        b_base[ni] + (int64_t)(s * 2 + ks) * (64 * 8));
        };
        auto consume = [&](int s, int buf, const u32x4(&ar)[PASSES], const u32x4(&br)[2][2]) {
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const uint32_t keep =
                    (s * BK + ps * RPP + rrow < u.k_kept && m_ok) ? 0xFFFFFFFFu : 0u;
                u32x4 v = ar[ps];
                v.x &= keep;
                v.y &= keep;
                v.z &= keep;
                v.w &= keep;
                *reinterpret_cast<u32x4 *>(smem + buf * STAGE + (ps * RPP + rrow) * PITCH +
                                           chunk * 8) = v;
            }
            __syncthreads();
            const uint16_t *stage = smem + buf * STAGE;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                u32x4 af[2];
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) {
                    const int mcol = wm * 64 + mi * 32;
                    if (TR) {
                        // 16 lanes read a 4(k) x 16(m) block; lane L addresses row L/4,
                        // columns 4*(L%4)..+3 and receives column L of the 4 rows.
                        const int L = lane & 15;
                        const int row = ks * 16 + (lane >> 5) * 8 + (L >> 2);
                        const int col = mcol + ((lane >> 4) & 1) * 16 + (L & 3) * 4;
                        const uint16_t *q = stage + row * PITCH + col;
                        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))q);
                        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (TW_LDS(s16x4))(q + 4 * PITCH));
                        u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                        af[mi].x = l2.x;
                        af[mi].y = l2.y;
                        af[mi].z = h2.x;
                        af[mi].w = h2.y;
                    } else {
                        const uint16_t *q =
                            stage + (ks * 16 + (lane >> 5) * 8) * PITCH + mcol + (lane & 31);
                        uint32_t w[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            w[e] = (uint32_t)q[(2 * e) * PITCH] |
                                   ((uint32_t)q[(2 * e + 1) * PITCH] << 16);
                        af[mi].x = w[0];
                        af[mi].y = w[1];
                        af[mi].z = w[2];
                        af[mi].w = w[3];
                    }
                }
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int mi = 0; mi < 2; ++mi)
                        acc[mi][ni] = E::mfma(af[mi], br[ks][ni], acc[mi][ni]);
            }
        };

        u32x4 a_ring[R][PASSES];
        u32x4 b_ring[R][2][2];
        IdxVec idx[PASSES];
        if (nsteps > 0)
            load_idx(0, idx);
#pragma unroll
        for (int j = 0; j < D; ++j) {
            if (j < nsteps) {
                issue(j, idx, a_ring[j], b_ring[j]);
                load_idx(j + 1, idx); // the list is padded by one step, so this stays in bounds
            }
        }
        int s0 = 0;
        // steady state: every slot issues and consumes, no conditionals
        for (; s0 + R + D <= nsteps; s0 += R) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                issue(s0 + r + D, idx, a_ring[(r + D) % R], b_ring[(r + D) % R]);
                load_idx(s0 + r + D + 1, idx);
                consume(s0 + r, r & 1, a_ring[r], b_ring[r]);
            }
        }
        // drain: fewer than R + D steps remain
        for (; s0 < nsteps; s0 += R) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int s = s0 + r;
                if (s < nsteps) {
                    if (s + D < nsteps) {
                        issue(s + D, idx, a_ring[(r + D) % R], b_ring[(r + D) % R]);
                        load_idx(s + D + 1, idx);
                    }
                    consume(s, r & 1, a_ring[r], b_ring[r]);
                }
            }
        }
        __syncthreads();

        // ---- epilogue ------------------------------------------------------------
        const int32_t *const nlist = p.kept_n + u.kn_off;
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int j = wn * 64 + ni * 32 + (lane & 31); // compact column inside the unit
            int64_t coff = 0;
            if (p.beta != 0.0f && j < u.n_cnt)
                coff = (int64_t)(u.col0 + nlist[j]) * p.ldc;
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) {
                const int mloc = wm * 64 + mi * 32 + (lane >> 5) * 4;
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = p.alpha * acc[mi][ni][r4 * 4 + e];
                        if (p.beta != 0.0f) {
                            const int m = m0 + mloc + r4 * 8 + e;
                            if (j < u.n_cnt && m < p.M)
                                v[e] += p.beta * E::from_bits(C[coff + m]);
                        }
                    }
                    u32x2 pk;
                    pk.x = E::to_bits(v[0]) | (E::to_bits(v[1]) << 16);
                    pk.y = E::to_bits(v[2]) | (E::to_bits(v[3]) << 16);
                    *reinterpret_cast<u32x2 *>(smem + j * CPITCH + mloc + r4 * 8) = pk;
                }
            }
        }
        __syncthreads();
        for (int j = rrow; j < u.n_cnt; j += RPP) {
            const int c = u.col0 + nlist[j];
            const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + j * CPITCH + chunk * 8);
            store_chunk(C + (int64_t)c * p.ldc + m_ld, v, m_ld, p.M);
        }
        __syncthreads();
    }

    // the last workgroup to leave re-arms the ticket slot for the next launch
    if (tid == 0) {
        __threadfence();
        const int done = atomicAdd(&p.ticket[1], 1);
        if (done == (int)gridDim.x - 1) {
            p.ticket[0] = 0;
            p.ticket[1] = 0;
            __threadfence();
        }
    }
}

// ---------------------------------------------------------------------------------
// small elementwise kernels of the boundary

__global__ void cast_f32_kernel(const float *src, uint16_t *dst, int64_t n, int dtype)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) // strict bound; the reference's `idx > n` writes one element too many
        return;
    dst[i] = dtype == TW_BF16 ? (uint16_t)Elem<TW_BF16>::to_bits(src[i])
                              : (uint16_t)Elem<TW_F16>::to_bits(src[i]);
}

__global__ void delete_row_kernel(const uint16_t *matrix, uint16_t *matrix_2, int rows, int columns,
                                  const int32_t *mask)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    const int i = blockIdx.y;
    if (i < rows && j < columns)
        matrix_2[(int64_t)i * columns + j] = matrix[(int64_t)(i + mask[i]) * columns + j];
}

__global__ void insert_row_kernel(uint16_t *matrix, const uint16_t *matrix_2, int rows, int columns,
                                  const int32_t *mask)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    const int i = blockIdx.y;
    if (i < rows && j < columns)
        matrix[(int64_t)(i + mask[i]) * columns + j] = matrix_2[(int64_t)i * columns + j];
}

static int env_int(const char *name, int dflt)
{
    const char *v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}

template <int DT, int WM, int WN>
static void launch_kmajor(const GemmArgs &a, int grid, bool tr, hipStream_t s)
{
    if (tr)
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, WM, WN, true>), dim3(grid),
                           dim3(64 * WM * WN), 0, s, a);
    else
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, WM, WN, false>), dim3(grid),
                           dim3(64 * WM * WN), 0, s, a);
}

} // namespace tw

using namespace tw;

extern "C" {

int tw_gemm(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C, int c_layout,
            int64_t ldc, int M, float alpha, float beta, int pruned_cols, void *stream)
{
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    if (M < 0)
        return fail(TW_ERR_SHAPE, "M=%d is negative", M);
    if ((a_layout != TW_LAYOUT_KMAJOR && a_layout != TW_LAYOUT_ROWMAJOR) ||
        (c_layout != TW_LAYOUT_KMAJOR && c_layout != TW_LAYOUT_ROWMAJOR))
        return fail(TW_ERR_LAYOUT, "a_layout=%d c_layout=%d: unknown layout", a_layout, c_layout);
    if (pruned_cols != TW_PRUNED_UNTOUCHED && pruned_cols != TW_PRUNED_ZERO)
        return fail(TW_ERR_LAYOUT, "pruned_cols=%d: unknown mode", pruned_cols);
    if (M == 0)
        return TW_OK;
    if (!A || !C)
        return fail(TW_ERR_NULL, "A or C is NULL");
    const int64_t min_lda = a_layout == TW_LAYOUT_KMAJOR ? M : plan->K;
    const int64_t min_ldc = c_layout == TW_LAYOUT_KMAJOR ? M : plan->N;
    if (lda < min_lda || ldc < min_ldc)
        return fail(TW_ERR_SHAPE, "lda=%lld (need >= %lld) ldc=%lld (need >= %lld)", (long long)lda,
                    (long long)min_lda, (long long)ldc, (long long)min_ldc);
    if ((lda & 7) || (ldc & 7))
        return fail(TW_ERR_ALIGNMENT, "lda=%lld and ldc=%lld must be multiples of 8 elements",
                    (long long)lda, (long long)ldc);
    if (((uintptr_t)A & 15) || ((uintptr_t)C & 15))
        return fail(TW_ERR_ALIGNMENT, "A and C must be 16-byte aligned");
    if (a_layout != TW_LAYOUT_KMAJOR || c_layout != TW_LAYOUT_KMAJOR)
        return fail(TW_ERR_LAYOUT, "row-major operands are not implemented yet");

    const bool narrow = plan->max_unit_n <= 64;
    const int BM = narrow ? 256 : 128;
    GemmArgs a;
    a.units = plan->d_units;
    a.tiles = plan->d_tiles;
    a.kept_k = plan->d_kept_k_pad;
    a.kept_n = plan->d_kept_n;
    a.pruned_n = plan->d_pruned_n;
    a.Bp = plan->d_Bp;
    a.A = A;
    a.C = C;
    a.lda = lda;
    a.ldc = ldc;
    a.M = M;
    a.n_mblk = (M + BM - 1) / BM;
    a.n_gemm_items = plan->n_units * a.n_mblk;
    a.n_zero_tiles = pruned_cols == TW_PRUNED_ZERO ? plan->n_zero_tiles : 0;
    a.n_items = a.n_gemm_items + a.n_zero_tiles * a.n_mblk;
    a.alpha = alpha;
    a.beta = beta;
    if (a.n_items == 0)
        return TW_OK;
    const unsigned slot =
        __atomic_fetch_add(&plan->next_slot, 1u, __ATOMIC_RELAXED) % (unsigned)kTicketSlots;
    a.ticket = plan->d_tickets + 2 * slot;

    const int per_cu = env_int("TWGEMM_WGS_PER_CU", 2);
    const int grid = std::min<int64_t>(a.n_items, (int64_t)plan->cu_count * per_cu);
    const bool tr = env_int("TWGEMM_NO_TR_READ", 0) == 0;
    hipStream_t s = (hipStream_t)stream;
    if (plan->dtype == TW_F16) {
        if (narrow)
            launch_kmajor<TW_F16, 4, 1>(a, grid, tr, s);
        else
            launch_kmajor<TW_F16, 2, 2>(a, grid, tr, s);
    } else {
        if (narrow)
            launch_kmajor<TW_BF16, 4, 1>(a, grid, tr, s);
        else
            launch_kmajor<TW_BF16, 2, 2>(a, grid, tr, s);
    }
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int tw_stream_gemm_nn(int M, int N, int K, int dtype, float alpha, const void *A, const void *B,
                      float beta, void *C, int block_num, const int32_t *N_cal,
                      const int32_t *K_cal, const int32_t *const *mask_n,
                      const int32_t *const *mask_k, const int64_t *off_B, const int64_t *off_C,
                      void *stream)
{
    tw_plan *plan = nullptr;
    int st = tw_plan_from_stream_operands(M, N, K, dtype, B, block_num, N_cal, K_cal, mask_n,
                                          mask_k, off_B, off_C, &plan);
    if (st)
        return st;
    const int64_t ld = (M + 7) / 8 * 8;
    if (ld != M) {
        tw_plan_destroy(plan);
        return fail(TW_ERR_ALIGNMENT, "M=%d must be a multiple of 8 here (lda = ldc = M)", M);
    }
    st = tw_gemm(plan, A, TW_LAYOUT_KMAJOR, M, C, TW_LAYOUT_KMAJOR, M, M, alpha, beta,
                 TW_PRUNED_UNTOUCHED, stream);
    if (!st) {
        hipError_t e = hipStreamSynchronize((hipStream_t)stream);
        if (e != hipSuccess)
            st = fail(TW_ERR_DEVICE, "stream synchronise failed: %s", hipGetErrorString(e));
    }
    tw_plan_destroy(plan);
    return st;
}

int tw_cast_f32(const float *src, void *dst, int64_t n, int dtype, void *stream)
{
    if (dtype != TW_F16 && dtype != TW_BF16)
        return fail(TW_ERR_DTYPE, "dtype %d is neither TW_F16 nor TW_BF16", dtype);
    if (n < 0)
        return fail(TW_ERR_SHAPE, "n=%lld is negative", (long long)n);
    if (n == 0)
        return TW_OK;
    if (!src || !dst)
        return fail(TW_ERR_NULL, "src or dst is NULL");
    hipLaunchKernelGGL(cast_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, src, (uint16_t *)dst, n, dtype);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int tw_delete_row(const void *matrix, void *matrix_2, int rows, int columns, const int32_t *mask,
                  void *stream)
{
    if (rows < 0 || columns < 0)
        return fail(TW_ERR_SHAPE, "rows=%d columns=%d", rows, columns);
    if (rows == 0 || columns == 0)
        return TW_OK;
    if (!matrix || !matrix_2 || !mask)
        return fail(TW_ERR_NULL, "matrix, matrix_2 or mask is NULL");
    hipLaunchKernelGGL(delete_row_kernel, dim3((columns + 255) / 256, rows), dim3(256), 0,
                       (hipStream_t)stream, (const uint16_t *)matrix, (uint16_t *)matrix_2, rows,
                       columns, mask);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int tw_insert_row(void *matrix, const void *matrix_2, int rows, int columns, const int32_t *mask,
                  void *stream)
{
    if (rows < 0 || columns < 0)
        return fail(TW_ERR_SHAPE, "rows=%d columns=%d", rows, columns);
    if (rows == 0 || columns == 0)
        return TW_OK;
    if (!matrix || !matrix_2 || !mask)
        return fail(TW_ERR_NULL, "matrix, matrix_2 or mask is NULL");
    hipLaunchKernelGGL(insert_row_kernel, dim3((columns + 255) / 256, rows), dim3(256), 0,
                       (hipStream_t)stream, (uint16_t *)matrix, (const uint16_t *)matrix_2, rows,
                       columns, mask);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

} // extern "C"
