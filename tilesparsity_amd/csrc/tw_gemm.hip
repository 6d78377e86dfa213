// The tile-wise-sparse GEMM of libtwgemm: persistent grouped kernels for gfx950.  Two K-major
// kernels share the decomposition and the data path below: tw_gemm_ws_kernel (wave-specialised,
// the default for wide tiles) and tw_gemm_kmajor_kernel (every wave loads, stages and
// multiplies; used for narrow tiles and small launches); tw_gemm_generic_kernel takes the other
// layouts.
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
//   * the packed weight is stored per 32-row step in per-lane MFMA operand order; a
//     step's block is one contiguous run, copied once per workgroup into LDS and read
//     back 16 bytes per lane (every wave needs it, and the vector-memory path, not
//     HBM, is what limits a workgroup that fetches its own copy per wave);
//   * v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulators;
//   * epilogue: alpha/beta in fp32, round to the 16-bit type, transpose through
//     LDS, then scatter whole C columns (col0 + kept_n[j]) with 16-byte stores.
#include "tw_internal.h"

#include <atomic>
#include <type_traits>
#include <cstddef>
#include <cstdlib>

namespace tw {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define TW_LDS(T) __attribute__((address_space(3))) T *

#ifndef TW_A_PAD
#define TW_A_PAD 32 // halfs of padding per staged A row: 64 B, so that the 4 rows x 2 column
                    // halves one transposed read touches fall into 8 distinct 32-byte bank groups
#endif

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
        return __builtin_bit_cast(uint16_t, (__bf16)f); // v_cvt_pk_bf16_f32, nearest even
    }
    static __device__ __forceinline__ float from_bits(uint16_t h)
    {
        return __uint_as_float((uint32_t)h << 16);
    }
};

// 16-byte chunk of column c, rows m..m+7 of a K-major matrix, honouring the M edge.  With
// `through` the store writes through to memory (sc0 sc1) and does not linger in the caches (nt):
// C is written once and not read again by this launch, and lines left dirty in the L2s would
// otherwise all be written back after the last wave has ended, where nothing overlaps them.  A
// small output is better left in the L2s: that write-back is short then, and shorter than the
// last stores' way to memory.
__device__ __forceinline__ void store_chunk(uint16_t *dst, u32x4 v, int m, int M, bool through)
{
    if (m + 8 <= M) {
        if (through)
            asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
        else
            *reinterpret_cast<u32x4 *>(dst) = v;
    } else if (m < M) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        for (int e = 0; e < M - m; ++e)
            dst[e] = (uint16_t)(w[e >> 1] >> ((e & 1) * 16));
    }
}

// Activation of the fused epilogue (tw_gemm_ex): the activations the reference's dense layers
// can be given (get_activation, Pruning/BERT/utils/modeling.py:280-305); GELU in its tanh form
// (modeling.py:264-277).
__device__ __forceinline__ float tw_activate(float v, int act)
{
    if (act == TW_ACT_RELU)
        return v > 0.0f ? v : 0.0f;
    // tanh(u) = 1 - 2 / (exp(2u) + 1) with the hardware exponential and reciprocal (1 ulp each):
    // exact limits at +-inf, ~1e-6 relative error in between, far below the 16-bit rounding
    if (act == TW_ACT_GELU) {
        const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
        return v - v * __builtin_amdgcn_rcpf(__expf(2.0f * u) + 1.0f); // 0.5 v (1 + tanh u)
    }
    if (act == TW_ACT_TANH)
        return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * v) + 1.0f);
    return v;
}
// alpha*acc + beta*C is already in `v`: adds the bias of column c and applies the activation
__device__ __forceinline__ float tw_finish(float v, const float *bias, int c, int act)
{
    if (bias)
        v += bias[c];
    return tw_activate(v, act);
}

// WM x WN waves of 64 x 64 outputs each: workgroup tile BM = 64*WM rows by BN = 64*WN
// compact columns.  WGS is the number of workgroups meant to share a CU.
// BK k rows are staged per main-loop step (a multiple of 16 that divides kBlockK); the loads
// of the D steps after the one being multiplied are in flight.
template <int DT, int WM, int WN, int BK, int D, int WGS>
__global__ void __launch_bounds__(64 * WM * WN, (WM * WN * WGS) / 4)
    tw_gemm_kmajor_kernel(const GemmArgs p)
{
    constexpr int NT = 64 * WM * WN;
    constexpr int BM = 64 * WM;
    constexpr int BN = 64 * WN;
    constexpr int KS = BK / kMfmaK;      // MFMA k steps per main-loop step
    constexpr int PKS = kBlockK / kMfmaK; // MFMA k steps per packed weight step
    constexpr int CPR = BM / 8;          // 16-byte chunks per staged A row / stored C column
    constexpr int RPP = NT / CPR;        // A rows (C columns) covered by one pass of the block
    constexpr int PASSES = BK / RPP;     // A loads per thread and step
    constexpr int BCH = BN * BK / 8;     // 16-byte chunks of packed weight per step
    constexpr int BPASS = (BCH + NT - 1) / NT;
    constexpr int PITCH = BM + TW_A_PAD; // halfs; the pad spreads the rows of a transposed read
    constexpr int ASTAGE = BK * PITCH;
    constexpr int BSTAGE = BN * BK;
    constexpr int CPITCH = BM + 4;       // halfs; 8-byte accumulator writes of 32 lanes (one
                                         // column each) then fall into 32 distinct bank pairs
    constexpr int PIPE = 2 * ASTAGE + 2 * BSTAGE;
    constexpr int SMEM = PIPE > BN * CPITCH ? PIPE : BN * CPITCH;
    static_assert(NT % CPR == 0 && BK % RPP == 0 && kBlockK % BK == 0, "tile shape");
    static_assert(BCH % NT == 0 || BCH < NT, "weight chunks per thread");
    using E = Elem<DT>;

    __shared__ __align__(16) uint16_t smem[SMEM];
    __shared__ int s_tk[2];
    // Instrumented builds only (-DTW_EXP_TIMING): workgroup 0 records cycle stamps of its steps
    // and phases in LDS and copies them behind the ticket slots, where tw_exp_read_debug reads
    // them.  Not part of the shipped library.
#ifdef TW_EXP_TIMING
    __shared__ unsigned long long s_ts[64 * 4];
#define TW_STAMP(step, slot)                                                              \
    if (item == 0 && tid == 0 && (step) >= 8 && (step) < 72)                              \
        s_ts[((step)-8) * 4 + (slot)] = __builtin_readcyclecounter();
#define TW_PHASE(k)                                                                       \
    if (blockIdx.x == 0 && tid == 0 && n_done_items < 2)                                  \
        s_ts[240 + n_done_items * 8 + (k)] = __builtin_readcyclecounter();
#else
#define TW_STAMP(step, slot)
#define TW_PHASE(k)
#endif

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = __builtin_amdgcn_readfirstlane(wave % WM);
    const int wn = __builtin_amdgcn_readfirstlane(wave / WM);
    const int chunk = tid % CPR;
    const int rrow = tid / CPR;
    const uint16_t *const A = reinterpret_cast<const uint16_t *>(p.A);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    const uint16_t *const Bp = reinterpret_cast<const uint16_t *>(p.Bp);
    uint16_t *const sA = smem;
    uint16_t *const sB = smem + 2 * ASTAGE;

    // ---- work items ----------------------------------------------------------------
    // A ticket names an item: tickets below n_pipe_items are GEMM items with at least one
    // step, then come GEMM items of units that keep no K row (their kept columns receive
    // alpha*0 + beta*C), then the zero-fill items.  The workgroup always holds the ticket
    // of its current and its next item and has the atomic for the one after in flight, so
    // a ticket's round trip is hidden behind a whole item.
    struct Item {
        int ticket;
        int m0;
        UnitDev u; // valid for ticket < n_gemm_items
    };
    auto make_item = [&](int ticket) {
        Item it;
        it.ticket = ticket;
        it.m0 = 0;
        if (ticket < p.n_gemm_items) {
            const int ui = ticket / p.n_mblk;
            it.m0 = (ticket - ui * p.n_mblk) * BM;
            it.u = p.units[ui];
        }
        return it;
    };
    // per-thread addressing of an item
    struct Thr {
        const int32_t *klist;
        const uint16_t *b_src[BPASS];
        int64_t b_pack;
        int m_ld, m_eff;
        bool m_ok;
    };
    auto setup = [&](const Item &it) {
        Thr t;
        t.klist = p.kept_k + it.u.kk_off; // padded past k_pad
        t.m_ld = it.m0 + chunk * 8;
        t.m_ok = t.m_ld < p.M;
        t.m_eff = t.m_ok ? t.m_ld : 0; // a valid chunk to read when this one is beyond M
        // This thread's 16-byte chunks of a step's packed weight.  The weight is packed per
        // kBlockK rows as (step, nb, k16, lane); chunk c of a BK-row step of this kernel is
        // (nb = c / (KS*64), k16 = (c / 64) % KS, lane = c % 64).  A block beyond the unit
        // reads block 0 (its products land in columns that are never stored).
#pragma unroll
        for (int bp = 0; bp < BPASS; ++bp) {
            const int c = tid + bp * NT;
            const int nbl = c / (KS * 64);
            const int k16 = (c >> 6) % KS;
            t.b_src[bp] = Bp + it.u.b_off +
                          (((int64_t)(it.u.nb0 + (nbl < it.u.nb_cnt ? nbl : 0)) * PKS + k16) * 64 +
                           (c & 63)) * 8;
        }
        t.b_pack = (int64_t)it.u.nblk * (PKS * 64 * 8);
        return t;
    };

    // Kept-K indices: every wave fetches the BK indices of a step with one coalesced load
    // (lane l holds row l of the step) D iterations before the row loads that use them;
    // loads return in order, so the word has landed by then without an extra wait.  The row
    // loads pick their index out of that register with a cross-lane permute.
    auto load_idx = [&](const Thr &t, int s, int &ix) {
        ix = t.klist[s * BK + (lane & (BK - 1))];
    };
    // No lane-dependent branches here: rows beyond K_t and chunks beyond M are loaded from a
    // valid address and replaced by zeros when they are staged (not here, so that nothing
    // waits on a load that was just issued).
    auto issue = [&](const Thr &t, int s, int ix, u32x4(&ar)[PASSES], u32x4(&br)[BPASS]) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int row = __builtin_amdgcn_ds_bpermute((ps * RPP + rrow) * 4, ix);
            ar[ps] = *reinterpret_cast<const u32x4 *>(A + (int64_t)row * p.lda + t.m_eff);
        }
        // element offset of step s: inside a packed step the k16 index advances, across
        // packed steps the whole block does
        const int64_t boff =
            (int64_t)(s / (PKS / KS)) * t.b_pack + (int64_t)(s % (PKS / KS)) * (KS * 64 * 8);
#pragma unroll
        for (int bp = 0; bp < BPASS; ++bp)
            if (BCH >= NT || tid < BCH)
                br[bp] = *reinterpret_cast<const u32x4 *>(t.b_src[bp] + boff);
    };

    constexpr int R = D + 1; // register slots: the step being staged plus D steps in flight
    u32x4 a_ring[R][PASSES];
    u32x4 b_ring[R][BPASS];
    int i_ring[R];
    int n_idx[2 * D]; // index words of the next item's first 2 D steps

    // The first item of a workgroup is its block index; later ones are claimed from the
    // shared counter (which starts at 0 for every launch) one item ahead, with the atomic of
    // the claim after that already in flight.
    const int ticket_base = gridDim.x;
    int t_pending = 0;   // thread 0: claim in flight
    bool closed = false; // thread 0: the queue is exhausted, no claim is in flight
    int t_done = -1;     // thread 0: workgroups counted as done before this one
    if (tid == 0)
        t_pending = atomicAdd(&p.ticket[0], 1);
    Item cur = make_item(blockIdx.x);
    Item nxt = cur;
    bool have_next = false; // nxt is known for the current item
    // Publishes the claim in flight as the next item and starts the claim after it.  A ticket
    // past the end makes the current item the workgroup's last: all its claims have returned, so
    // it counts itself as done right away (the workgroup counted last re-arms the slot when it
    // leaves) and that count's round trip is over before the item ends.
    auto claim_next = [&]() {
        if (tid == 0) {
            const int t = closed ? p.n_items : ticket_base + t_pending;
            s_tk[0] = t;
            if (!closed) {
                if (t < p.n_items) {
                    t_pending = atomicAdd(&p.ticket[0], 1);
                } else {
                    closed = true;
                    t_done = atomicAdd(&p.ticket[1], 1);
                }
            }
        }
        __syncthreads();
        // tickets are workgroup-uniform: keep them, and everything derived from them, scalar
        nxt = make_item(__builtin_amdgcn_readfirstlane(s_tk[0]));
        have_next = true;
        __syncthreads();
    };
    bool preloaded = false; // cur's first D steps are already in flight, i_ring holds D..2D-1

    bool first = true;
    int n_done_items = 0;
    while (cur.ticket < p.n_items) {
        const int item = cur.ticket;
        TW_PHASE(0)
        // the very first claim of a workgroup is published after the first item's loads have
        // been issued, so that its round trip overlaps with them
        if (!first || item >= p.n_pipe_items)
            claim_next();
        first = false;
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
                if ((p.beta != 0.0f || p.bias || p.act) && m < p.M) {
                    uint32_t w[4] = {0u, 0u, 0u, 0u};
                    for (int e = 0; e < 8 && m + e < p.M; ++e) {
                        const float old = p.beta != 0.0f ? p.beta * E::from_bits(dst[e]) : 0.0f;
                        w[e >> 1] |= E::to_bits(tw_finish(old, p.bias, c, p.act)) << ((e & 1) * 16);
                    }
                    v.x = w[0];
                    v.y = w[1];
                    v.z = w[2];
                    v.w = w[3];
                }
                store_chunk(dst, v, m, p.M, p.store_through != 0);
            }
        } else {
            // ---- GEMM item ------------------------------------------------------
            const UnitDev &u = cur.u;
            const int m0 = cur.m0;
            const int nsteps = u.k_pad / BK;
            const Thr tc = setup(cur);

            f32x16 acc[2][2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[mi][ni][r] = 0.0f;

            // Pipeline over steps of BK rows.  Iteration s issues the global loads of step
            // s+D into a free register slot, writes the registers of step s (loaded D
            // iterations ago) to LDS buffer s&1, and after one barrier multiplies step s out
            // of LDS.  So D steps of gathered A rows and packed weight are in flight.
            auto stage = [&](int s, const u32x4(&ar)[PASSES], const u32x4(&br)[BPASS]) {
                uint16_t *const stA = sA + (s & 1) * ASTAGE;
                uint16_t *const stB = sB + (s & 1) * BSTAGE;
                if (s * BK + BK > u.k_kept || m0 + BM > p.M) {
                    // edge step: rows beyond K_t and chunks beyond M become zeros
#pragma unroll
                    for (int ps = 0; ps < PASSES; ++ps) {
                        const uint32_t keep =
                            (s * BK + ps * RPP + rrow < u.k_kept && tc.m_ok) ? 0xFFFFFFFFu : 0u;
                        u32x4 v = ar[ps];
                        v.x &= keep;
                        v.y &= keep;
                        v.z &= keep;
                        v.w &= keep;
                        *reinterpret_cast<u32x4 *>(stA + (ps * RPP + rrow) * PITCH + chunk * 8) = v;
                    }
                } else {
#pragma unroll
                    for (int ps = 0; ps < PASSES; ++ps)
                        *reinterpret_cast<u32x4 *>(stA + (ps * RPP + rrow) * PITCH + chunk * 8) =
                            ar[ps];
                }
#pragma unroll
                for (int bp = 0; bp < BPASS; ++bp)
                    if (BCH >= NT || tid < BCH)
                        *reinterpret_cast<u32x4 *>(stB + (tid + bp * NT) * 8) = br[bp];
            };
            auto frags = [&](int s, int ks, u32x4(&af)[2], u32x4(&bf)[2]) {
                const uint16_t *const stA = sA + (s & 1) * ASTAGE;
                const uint16_t *const stB = sB + (s & 1) * BSTAGE;
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) {
                    // ds_read_b64_tr_b16: 16 lanes read a 4(k) x 16(m) block; lane L addresses
                    // row L/4, columns 4*(L%4)..+3 and receives column L of the 4 rows.
                    const int L = lane & 15;
                    const int row = ks * 16 + (lane >> 5) * 8 + (L >> 2);
                    const int col = wm * 64 + mi * 32 + ((lane >> 4) & 1) * 16 + (L & 3) * 4;
                    const uint16_t *q = stA + row * PITCH + col;
                    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))q);
                    s16x4 hi =
                        __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(q + 4 * PITCH));
                    u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                    af[mi].x = l2.x;
                    af[mi].y = l2.y;
                    af[mi].z = h2.x;
                    af[mi].w = h2.y;
                }
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    bf[ni] = *reinterpret_cast<const u32x4 *>(
                        stB + ((((wn * 2 + ni) * KS + ks) * 64) + lane) * 8);
            };
            // one iteration; r == s % R is the register slot of step s
            auto iteration = [&](int s, int r, bool more_loads) {
                u32x4 af[2], bf[2];
                if (more_loads) {
                    load_idx(tc, s + 2 * D, i_ring[(r + 2 * D) % R]); // padded list: in bounds
                    issue(tc, s + D, i_ring[(r + D) % R], a_ring[(r + D) % R], b_ring[(r + D) % R]);
                }
                TW_STAMP(s, 0)
                stage(s, a_ring[r], b_ring[r]);
                TW_STAMP(s, 1)
                __syncthreads();
                TW_STAMP(s, 2)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    frags(s, ks, af, bf);
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                        for (int mi = 0; mi < 2; ++mi)
                            acc[mi][ni] = E::mfma(af[mi], bf[ni], acc[mi][ni]);
                }
                TW_STAMP(s, 3)
            };

            if (!preloaded) {
#pragma unroll
                for (int j = 0; j < D; ++j)
                    load_idx(tc, j, i_ring[j % R]);
#pragma unroll
                for (int j = 0; j < D; ++j) {
                    if (j < nsteps) {
                        issue(tc, j, i_ring[j % R], a_ring[j], b_ring[j]);
                        load_idx(tc, j + D, i_ring[(j + D) % R]);
                    }
                }
            }
            TW_PHASE(1)
            if (!have_next)
                claim_next();
            TW_PHASE(2)
            int s0 = 0;
            // steady state: every iteration issues, stages and multiplies, no conditionals
            for (; s0 + R + D <= nsteps; s0 += R) {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    iteration(s0 + r, r, true);
            }
            // The next item's index words are fetched before the drain, so that its first row
            // loads can be issued right after this item's last step and fly over the epilogue.
            const bool chain = nxt.ticket < p.n_pipe_items;
            Thr tn;
            if (chain) {
                tn = setup(nxt);
#pragma unroll
                for (int j = 0; j < 2 * D; ++j)
                    load_idx(tn, j, n_idx[j]);
            }
            // drain: fewer than R + D steps remain
            for (; s0 < nsteps; s0 += R) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int s = s0 + r;
                    if (s < nsteps)
                        iteration(s, r, s + D < nsteps);
                }
            }
            __syncthreads();
            TW_PHASE(3)
            if (chain) {
                const int nn = nxt.u.k_pad / BK;
#pragma unroll
                for (int j = 0; j < D; ++j) {
                    if (j < nn)
                        issue(tn, j, n_idx[j], a_ring[j], b_ring[j]);
                    i_ring[(j + D) % R] = n_idx[j + D];
                }
            }
            preloaded = chain;
            TW_PHASE(4)

            // ---- epilogue --------------------------------------------------------
            const int32_t *const nlist = p.kept_n + u.kn_off;
            float scale = p.alpha;
            if (p.beta != 0.0f || p.bias || p.act) {
                // rare path, kept out of the way of the common one: fold alpha, beta*C, the bias
                // and the activation into the accumulators first (C is read on kept columns only)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    const int j = wn * 64 + ni * 32 + (lane & 31);
                    const int col = j < u.n_cnt ? u.col0 + nlist[j] : 0;
                    const int64_t coff = (int64_t)col * p.ldc;
                    const float bj = p.bias ? p.bias[col] : 0.0f;
#pragma unroll
                    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int m = m0 + wm * 64 + mi * 32 + (lane >> 5) * 4 + (r >> 2) * 8 + (r & 3);
                            float old = 0.0f;
                            if (p.beta != 0.0f && j < u.n_cnt && m < p.M)
                                old = E::from_bits(C[coff + m]);
                            acc[mi][ni][r] =
                                tw_activate(p.alpha * acc[mi][ni][r] + p.beta * old + bj, p.act);
                        }
                }
                scale = 1.0f;
            }
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const int j = wn * 64 + ni * 32 + (lane & 31); // compact column inside the unit
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) {
                    const int mloc = wm * 64 + mi * 32 + (lane >> 5) * 4;
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        u32x2 pk;
                        pk.x = E::to_bits(scale * acc[mi][ni][r4 * 4 + 0]) |
                               (E::to_bits(scale * acc[mi][ni][r4 * 4 + 1]) << 16);
                        pk.y = E::to_bits(scale * acc[mi][ni][r4 * 4 + 2]) |
                               (E::to_bits(scale * acc[mi][ni][r4 * 4 + 3]) << 16);
                        *reinterpret_cast<u32x2 *>(smem + j * CPITCH + mloc + r4 * 8) = pk;
                    }
                }
            }
            __syncthreads();
            TW_PHASE(5)
            for (int j = rrow; j < u.n_cnt; j += RPP) {
                const int c = u.col0 + nlist[j];
                // rows of the staging tile are 8-byte aligned only: two 8-byte reads
                const u32x2 lo = *reinterpret_cast<const u32x2 *>(smem + j * CPITCH + chunk * 8);
                const u32x2 hi = *reinterpret_cast<const u32x2 *>(smem + j * CPITCH + chunk * 8 + 4);
                u32x4 v;
                v.x = lo.x;
                v.y = lo.y;
                v.z = hi.x;
                v.w = hi.y;
                store_chunk(C + (int64_t)c * p.ldc + tc.m_ld, v, tc.m_ld, p.M, p.store_through != 0);
            }
        }

        TW_PHASE(6)
        __syncthreads();
        TW_PHASE(7)
        cur = nxt;
        have_next = false;
        ++n_done_items;
    }

#ifdef TW_EXP_TIMING
    __syncthreads();
    if (blockIdx.x == 0 && tid < 256)
        reinterpret_cast<unsigned long long *>(p.dbg)[tid] = s_ts[tid];
#endif
    // the workgroup counted last re-arms the ticket slot for the next launch: every workgroup's
    // claims had returned before it was counted.  Plain stores, made visible by the end of the
    // kernel; a device-scope fence here would write back and invalidate this XCD's L2 under the
    // workgroups that still stream through it.
    if (tid == 0 && t_done == (int)gridDim.x - 1) {
        p.ticket[0] = 0;
        p.ticket[1] = 0;
    }
}

// Workgroup barrier for hand-overs through LDS only: waits for this wave's LDS operations, not
// for its global loads, stores or atomics in flight (which __syncthreads() would do for stores
// and atomics), so prefetched loads, the item's output stores and the ticket atomic keep flying.
#define TW_LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

// ---------------------------------------------------------------------------------
// Wave-specialised 256 x 128 kernel (8 waves, one workgroup per CU).  Waves 0-3 only multiply:
// wave w owns rows 64w..64w+63 of the row block and all 128 compact columns (2 x 4 MFMA
// blocks, 128 accumulator registers).  Waves 4-7 only move data: they gather the kept rows of
// A and the packed weight global -> registers -> LDS, R steps of 64 rows in flight.  Both
// halves meet at one barrier per step: while the multiplying waves read stage s & 1, the
// moving waves fill stage (s + 1) & 1, so LDS traffic, vector-memory traffic and MFMA work
// overlap instead of following each other.  One multiplying and one moving wave share a SIMD.
// Work items, tickets, the chained first loads of the next item and the epilogue are those of
// tw_gemm_kmajor_kernel.
template <int DT> __global__ void __launch_bounds__(512, 2) tw_gemm_ws_kernel(const GemmArgs p)
{
    constexpr int NT = 512, NP = 256, BM = 256, BN = 128, BK = 64;
    constexpr int KS = BK / kMfmaK, PKS = kBlockK / kMfmaK;
    constexpr int R = 2;                       // register slots = steps of loads in flight
    constexpr int MI = 2, NI = 4;
    constexpr int CPR = BM / 8;                // 16-byte chunks per staged A row / stored C column
    constexpr int RPP = NP / CPR;              // A rows covered by one pass of the moving waves
    constexpr int PASSES = BK / RPP;           // A loads per moving thread and step
    constexpr int BPASS = BN * BK / 8 / NP;    // weight loads per moving thread and step
    constexpr int PITCH = BM + TW_A_PAD;
    constexpr int ASTAGE = BK * PITCH, BSTAGE = BN * BK;
    constexpr int CPITCH = BM + 4;
    constexpr int PIPE = 2 * (ASTAGE + BSTAGE);
    constexpr int SMEM = PIPE > BN * CPITCH ? PIPE : BN * CPITCH;
    static_assert(BK == kBlockK && KS == PKS, "one packed weight step per main-loop step");
    using E = Elem<DT>;

    __shared__ __align__(16) uint16_t smem[SMEM];
    __shared__ int s_tk[2];
    __shared__ int s_cols[BN];   // output columns of the current item's unit
    __shared__ float s_bias[BN]; // ... and their bias values (fused epilogue)
    // Instrumented builds only (-DTW_EXP_TIMING=1: cycle stamps of workgroup 0's item number
    // TW_EXP_ITEM; =2: start and end time of every workgroup), read back with tw_exp_read_debug.
#ifdef TW_EXP_TIMING
    __shared__ unsigned long long s_ws[256];
#ifndef TW_EXP_ITEM
#define TW_EXP_ITEM 0
#endif
    int ws_item = 0;
#define ws_first (ws_item == TW_EXP_ITEM)
#define TW_WS_STAMP(step, k, t)                                                          \
    if (blockIdx.x == 0 && ws_first && threadIdx.x == (t) && (step) < 30)               \
        s_ws[(step)*8 + (k)] = __builtin_readcyclecounter();
#define TW_WS_PHASE(k, t)                                                                \
    if (blockIdx.x == 0 && ws_first && threadIdx.x == (t))                               \
        s_ws[240 + (k)] = __builtin_readcyclecounter();
#else
#define TW_WS_STAMP(step, k, t)
#define TW_WS_PHASE(k, t)
#endif

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint16_t *const A = reinterpret_cast<const uint16_t *>(p.A);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    const uint16_t *const Bp = reinterpret_cast<const uint16_t *>(p.Bp);
    uint16_t *const sA = smem;
    uint16_t *const sB = smem + 2 * ASTAGE;

    struct Item {
        int ticket;
        int m0, m_end; // rows [m0, m_end) of A and C, at most BM of them
        UnitDev u;     // valid for ticket < n_gemm_items
    };
    auto make_item = [&](int ticket) {
        Item it;
        it.ticket = ticket;
        it.m0 = 0;
        it.m_end = 0;
        if (ticket < p.n_gemm_items) {
            const auto *ka = (const __attribute__((address_space(4))) int32_t *)
                __builtin_amdgcn_kernarg_segment_ptr();
            const int ui = ticket / p.n_mblk;
            it.m0 = (ticket - ui * p.n_mblk) * BM;
            it.m_end = it.m0 + BM < p.M ? it.m0 + BM : p.M;
            static_assert(sizeof(UnitDev) == 48, "UnitDev is read as 12 words");
            int32_t w[12];
            if (p.n_arg_units) {
                // from the kernel-argument segment: scalar loads, no global round trip
#pragma unroll
                for (int i = 0; i < 12; ++i)
                    w[i] = ka[offsetof(GemmArgs, arg_units) / 4 + ui * 12 + i];
            } else {
                __builtin_memcpy(w, &p.units[ui], sizeof(UnitDev));
            }
            // the descriptor is workgroup-uniform: keep it, and all derived from it, scalar
#pragma unroll
            for (int i = 0; i < 12; ++i)
                w[i] = __builtin_amdgcn_readfirstlane(w[i]);
            __builtin_memcpy(&it.u, w, sizeof(UnitDev));
        }
        return it;
    };
    // Both halves of the workgroup walk the same item sequence and execute the same sequence
    // of barriers; thread 0 (a multiplying wave) owns the ticket counter.
#ifdef TW_EXP_TIMING
    if (blockIdx.x == 0 && tid == 0) {
        s_ws[248] = __builtin_readcyclecounter();
        s_ws[249] = __builtin_amdgcn_s_memrealtime();
    }
#if TW_EXP_TIMING == 2
    if (tid == 0 && blockIdx.x < 256)
        reinterpret_cast<unsigned *>(p.dbg)[blockIdx.x * 2] = (unsigned)__builtin_amdgcn_s_memrealtime();
#endif
#endif
    // The first two items of a workgroup are fixed (block index, block index + grid size), so
    // that no atomic's round trip sits between the start of the kernel and the first loads;
    // the shared counter hands out the items after those.
    const int ticket_base = 2 * gridDim.x;
    int t_pending = 0;                     // thread 0: result of the claim in flight
    int t_next = gridDim.x + blockIdx.x;   // thread 0: the next ticket once known, or -1
    bool closed = false;    // thread 0: no claim of this workgroup is in flight, none will follow
    bool announced = false; // thread 0: the workgroup has been counted as done with the counter
    int t_done = -1;        // thread 0: workgroups counted before this one (atomic's result)
    if (tid == 0)
        t_pending = atomicAdd(&p.ticket[0], 1);
    // Picks up the claim in flight and starts the one after it, unless the queue is exhausted.
    // Called before an item's output stores are issued: memory operations complete in order, so
    // waiting for an atomic issued after them (or overwriting its register) would wait for the
    // stores as well.
    auto pick_up = [&]() {
        if (tid == 0 && t_next < 0) {
            if (closed) {
                t_next = p.n_items;
            } else {
                t_next = ticket_base + t_pending;
                asm volatile("" : "+v"(t_next)); // here, not where it is published
                if (t_next < p.n_items)
                    t_pending = atomicAdd(&p.ticket[0], 1);
                else
                    closed = true;
            }
        }
    };
    // Thread 0, when it hands out the ticket after the current item: a ticket past the end means
    // that the current item is the workgroup's last.  All its claims have returned by then, so it
    // counts itself as done with the counter right away and the count's round trip is over long
    // before the item ends; the workgroup counted last re-arms the slot when it leaves.
    auto announce = [&]() {
        if (t_next >= p.n_items && !announced) {
            if (!closed) {
                // the second fixed item is already past the end: the first claim is in flight
                asm volatile("" ::"v"(t_pending));
                closed = true;
            }
            t_done = atomicAdd(&p.ticket[1], 1);
            announced = true;
        }
    };
    // An item with at least one step learns its successor without barriers of its own: thread 0
    // publishes the ticket before the item's first pipeline barrier, everybody reads it after.
    auto publish = [&]() {
        if (tid == 0) {
            pick_up();
            s_tk[0] = t_next;
            announce();
            t_next = -1;
        }
    };
    auto published = [&]() { return make_item(__builtin_amdgcn_readfirstlane(s_tk[0])); };
    auto claim = [&]() { // two barriers of its own: items without steps
        if (tid == 0) {
            pick_up();
            s_tk[0] = t_next;
            announce();
            t_next = -1;
        }
        TW_WS_STAMP(0, 6, 256)
        TW_LDS_BARRIER();
        TW_WS_STAMP(0, 7, 256)
        const Item it = make_item(__builtin_amdgcn_readfirstlane(s_tk[0]));
#ifdef TW_EXP_TIMING
        if (it.u.k_pad >= 0)
            TW_WS_STAMP(1, 6, 256)
#endif
        TW_LDS_BARRIER();
        TW_WS_STAMP(1, 7, 256)
        return it;
    };
    // zero-fill item: pruned columns of one tile receive beta*C (all threads, no barrier)
    auto zero_fill = [&](int item) {
        const int z = item - p.n_gemm_items;
        const int zt = z / p.n_mblk;
        const int m = (z - zt * p.n_mblk) * BM + (tid % CPR) * 8;
        const TileDev t = p.tiles[zt];
        for (int j = tid / CPR; j < t.n_pruned; j += NT / CPR) {
            const int c = t.col0 + p.pruned_n[t.pn_off + j];
            uint16_t *dst = C + (int64_t)c * p.ldc + m;
            u32x4 v = {0u, 0u, 0u, 0u};
            if ((p.beta != 0.0f || p.bias || p.act) && m < p.M) {
                uint32_t w[4] = {0u, 0u, 0u, 0u};
                for (int e = 0; e < 8 && m + e < p.M; ++e) {
                    const float old = p.beta != 0.0f ? p.beta * E::from_bits(dst[e]) : 0.0f;
                    w[e >> 1] |= E::to_bits(tw_finish(old, p.bias, c, p.act)) << ((e & 1) * 16);
                }
                v.x = w[0];
                v.y = w[1];
                v.z = w[2];
                v.w = w[3];
            }
            store_chunk(dst, v, m, p.M, p.store_through != 0);
        }
    };
    // scatters the staged C tile (all threads): whole columns col0 + kept_n[j], 16-byte stores
    // (the output columns col0 + kept_n[j] come from s_cols, filled by the moving waves)
    auto store_tile = [&](const UnitDev &u, int m0, int m_end) {
        const int m_st = m0 + (tid % CPR) * 8;
        for (int j = tid / CPR; j < u.n_cnt; j += NT / CPR) {
            const int c = s_cols[j];
            // rows of the staging tile are 8-byte aligned only: two 8-byte reads
            const u32x2 lo = *reinterpret_cast<const u32x2 *>(smem + j * CPITCH + (tid % CPR) * 8);
            const u32x2 hi = *reinterpret_cast<const u32x2 *>(smem + j * CPITCH + (tid % CPR) * 8 + 4);
            u32x4 v;
            v.x = lo.x;
            v.y = lo.y;
            v.z = hi.x;
            v.w = hi.y;
            store_chunk(C + (int64_t)c * p.ldc + m_st, v, m_st, m_end, p.store_through != 0);
        }
    };

    if (wave >= 4) {
        // ================= moving waves ===================================================
        // Thread pt moves chunk pt % 32 (8 consecutive m) of the rows 8 * (pt / 32) .. + 7 of a
        // step: a wave covers 16 consecutive kept rows, whose indices it fetches with one
        // scalar load.  Addresses are a uniform base plus a 32-bit byte offset per lane.
        const int pt = tid - NP;
        const int chunk = pt % CPR, rgrp = pt / CPR;
        const bool upper = (lane >> 5) != 0;           // second row group of this wave
        const int mw = wave - 4;
        const uint32_t lda_b = (uint32_t)p.lda * 2u;   // bytes; K * lda * 2 < 2^32 (host check)
        typedef int i32x16 __attribute__((ext_vector_type(16)));
        struct Idx {
            int k[16];
        };
        struct Thr {
            const int32_t *klist;   // + 16 * mw: this wave's rows of step 0
            const char *a_base;     // A + m0 (bytes), uniform
            const char *b_base[BPASS];
            int64_t b_pack_b;
            uint32_t v_chunk;       // byte offset of this lane's chunk inside a gathered row
            bool m_ok;
        };
        auto setup = [&](const Item &it) {
            Thr t;
            t.klist = p.kept_k + it.u.kk_off + 16 * mw; // padded past k_pad
            t.a_base = reinterpret_cast<const char *>(A + it.m0);
            t.m_ok = it.m0 + chunk * 8 < it.m_end;
            t.v_chunk = t.m_ok ? chunk * 16 : 0; // beyond the row block: re-read its first chunk
            // weight chunk c = pt + bp * NP of a step is (nb = bp, k16 = pt / 64, lane = pt % 64);
            // a block beyond the unit reads block 0 (its products are never stored)
#pragma unroll
            for (int bp = 0; bp < BPASS; ++bp)
                t.b_base[bp] = reinterpret_cast<const char *>(
                    Bp + it.u.b_off + (int64_t)(it.u.nb0 + (bp < it.u.nb_cnt ? bp : 0)) * (PKS * 64 * 8));
            t.b_pack_b = (int64_t)it.u.nblk * (PKS * 64 * 8 * 2);
            return t;
        };
        auto load_idx = [&](const Thr &t, int s, Idx &ix) {
            const i32x16 v = *reinterpret_cast<const __attribute__((address_space(4))) i32x16 *>(
                (uintptr_t)(t.klist + s * BK));
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                ix.k[i] = v[i];
                asm volatile("" : "+s"(ix.k[i])); // keep the words scalar and the load whole
            }
        };
        auto load_a = [&](const Thr &t, const Idx &ix, int ps) {
            uint32_t o0 = (uint32_t)ix.k[ps] * lda_b, o1 = (uint32_t)ix.k[8 + ps] * lda_b;
            asm volatile("" : "+s"(o0), "+s"(o1)); // multiply on the scalar unit, select afterwards
            return *reinterpret_cast<const u32x4 *>(t.a_base + ((upper ? o1 : o0) + t.v_chunk));
        };
        auto load_b = [&](const Thr &t, int s, int bp) {
            return *reinterpret_cast<const u32x4 *>(t.b_base[bp] + (int64_t)s * t.b_pack_b +
                                                    (uint32_t)(pt * 16));
        };
        auto issue = [&](const Thr &t, int s, const Idx &ix, u32x4(&ar)[PASSES], u32x4(&br)[BPASS]) {
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps)
                ar[ps] = load_a(t, ix, ps);
#pragma unroll
            for (int bp = 0; bp < BPASS; ++bp)
                br[bp] = load_b(t, s, bp);
        };
        u32x4 a_ring[R][PASSES];
        u32x4 b_ring[R][BPASS];
        Idx ix_next;            // row indices of the step issued next
        bool preloaded = false; // cur's first R steps are in flight, ix_next is that of step R

        TW_WS_PHASE(6, 256)
        Item cur = make_item(blockIdx.x);
        Item nxt = cur;
        bool have_next = false;
#ifdef TW_EXP_TIMING
        if (cur.u.k_pad >= 0)
            TW_WS_PHASE(7, 256)
#endif
        while (cur.ticket < p.n_items) {
            const int item = cur.ticket;
#if defined(TW_EXP_TIMING) && TW_EXP_ITEM > 0
            TW_WS_PHASE(6, 256)
#endif
            if (item >= p.n_pipe_items) { // no step, no pipeline barrier to ride on
                nxt = claim();
                have_next = true;
            }
#if defined(TW_EXP_TIMING) && TW_EXP_ITEM > 0
            TW_WS_PHASE(7, 256)
#endif
            if (item >= p.n_gemm_items) {
                zero_fill(item);
            } else {
                const UnitDev &u = cur.u;
                const int m0 = cur.m0;
                const int nsteps = u.k_pad / BK;
                const Thr tc = setup(cur);
                // output columns of the unit and their bias: fetched now, handed to the other waves
                // through LDS with the last step
                int out_col = 0;
                float out_bias = 0.0f;
                if (pt < BN)
                    out_col = u.col0 + p.kept_n[u.kn_off + (pt < u.n_cnt ? pt : 0)];
                if (!preloaded && nsteps > 0) {
                    Idx ix[R];
#pragma unroll
                    for (int j = 0; j < R; ++j)
                        load_idx(tc, j, ix[j]); // the padded list keeps every index load in bounds
                    load_idx(tc, R, ix_next);
                    // Every register slot is loaded whether or not the item has that many steps
                    // (the index list is padded, the weight step is clamped): the number of loads
                    // in flight is then the same on every path into the slots below, and the
                    // compiler can wait for exactly the loads a slot needs.
#pragma unroll
                    for (int j = 0; j < R; ++j)
                        issue(tc, j < nsteps ? j : nsteps - 1, ix[j], a_ring[j], b_ring[j]);
                }
                TW_WS_PHASE(0, 256)
                TW_WS_PHASE(1, 256)
                // time slot j: write step j (loaded R slots ago) into stage j & 1 and reuse its
                // registers for the loads of step j + R.  Every register is written to LDS and
                // refilled by its next load back to back, so that the LDS queue and the
                // vector-memory queue are fed at the same time.
                auto slot = [&](int j, int r, bool more) {
                    TW_WS_STAMP(j, 2, 256)
                    uint16_t *const stA = sA + (j & 1) * ASTAGE;
                    uint16_t *const stB = sB + (j & 1) * BSTAGE;
                    const bool edge = j * BK + BK > u.k_kept || m0 + BM > cur.m_end;
                    const Idx ix = ix_next;
                    if (more)
                        load_idx(tc, j + R + 1, ix_next);
#pragma unroll
                    for (int ps = 0; ps < PASSES; ++ps) {
                        u32x4 v = a_ring[r][ps];
                        if (edge) {
                            // rows beyond K_t and chunks beyond M become zeros
                            const uint32_t keep =
                                (j * BK + rgrp * 8 + ps < u.k_kept && tc.m_ok) ? 0xFFFFFFFFu : 0u;
                            v.x &= keep;
                            v.y &= keep;
                            v.z &= keep;
                            v.w &= keep;
                        }
                        *reinterpret_cast<u32x4 *>(stA + (rgrp * 8 + ps) * PITCH + chunk * 8) = v;
                        if (more)
                            a_ring[r][ps] = load_a(tc, ix, ps);
                    }
#pragma unroll
                    for (int bp = 0; bp < BPASS; ++bp) {
                        *reinterpret_cast<u32x4 *>(stB + (pt + bp * NP) * 8) = b_ring[r][bp];
                        if (more)
                            b_ring[r][bp] = load_b(tc, j + R, bp);
                    }
                    TW_WS_STAMP(j, 4, 256)
                    TW_LDS_BARRIER();
                    TW_WS_STAMP(j, 5, 256)
                    if (j == 0 && !have_next) {
                        nxt = published();
                        have_next = true;
                    }
                };
                int j0 = 0;
                for (; j0 + 2 * R <= nsteps; j0 += R) {
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        slot(j0 + r, r, true);
                }
                // (the column numbers have arrived by now: the bias load flies over the last slots)
                if (p.bias && pt < BN)
                    out_bias = p.bias[out_col];
                // The last one to three slots, written out so that each knows at compile time
                // whether it still fetches a step (a slot that decides this at run time makes the
                // compiler wait for every load in flight before the first LDS write).
                static_assert(R == 2, "the drain is written out for two register slots");
                if (nsteps - j0 == 3) {
                    slot(j0, 0, true);
                    slot(j0 + 1, 1, false);
                    slot(j0 + 2, 0, false);
                } else if (nsteps - j0 == 2) {
                    slot(j0, 0, false);
                    slot(j0 + 1, 1, false);
                } else if (nsteps - j0 == 1) {
                    slot(j0, 0, false); // an item of one step
                } // (a unit without kept rows has no step: its columns receive beta * C)
                // last time slot: the multiplying waves work on the last step; the first loads of
                // the next item start now and fly over the epilogue
                const bool chain = nxt.ticket < p.n_pipe_items;
                if (chain) {
                    const Thr tn = setup(nxt);
                    const int nn = nxt.u.k_pad / BK;
                    Idx ix[R];
#pragma unroll
                    for (int j = 0; j < R; ++j)
                        load_idx(tn, j, ix[j]);
                    load_idx(tn, R, ix_next);
#pragma unroll
                    for (int j = 0; j < R; ++j)
                        issue(tn, j < nn ? j : nn - 1, ix[j], a_ring[j], b_ring[j]);
                }
                preloaded = chain;
                if (pt < BN) {
                    s_cols[pt] = out_col;
                    s_bias[pt] = out_bias;
                }
                TW_WS_PHASE(2, 256)
                TW_LDS_BARRIER(); // end of the last time slot
                TW_WS_PHASE(3, 256)
                TW_LDS_BARRIER(); // the C tile is staged
                TW_WS_PHASE(4, 256)
                store_tile(u, m0, cur.m_end);
                TW_WS_PHASE(5, 256)
            }
            TW_LDS_BARRIER(); // LDS may be reused now
            cur = nxt;
            have_next = false;
#ifdef TW_EXP_TIMING
            ++ws_item;
#endif
        }
    } else {
        // ================= multiplying waves ==============================================
        Item cur = make_item(blockIdx.x);
        Item nxt = cur;
        bool have_next = false;
        while (cur.ticket < p.n_items) {
            const int item = cur.ticket;
            if (item >= p.n_pipe_items) {
                nxt = claim();
                have_next = true;
            }
            if (item >= p.n_gemm_items) {
                zero_fill(item);
            } else {
                const UnitDev &u = cur.u;
                const int m0 = cur.m0;
                const int nsteps = u.k_pad / BK;
                f32x16 acc[MI][NI];
#pragma unroll
                for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc[mi][ni][r] = 0.0f;
                const bool w_active = m0 + wave * 64 < cur.m_end;
                auto frags = [&](int s, int ks, u32x4(&af)[MI], u32x4(&bf)[NI]) {
                    const uint16_t *const stA = sA + (s & 1) * ASTAGE;
                    const uint16_t *const stB = sB + (s & 1) * BSTAGE;
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi) {
                        // ds_read_b64_tr_b16: 16 lanes read a 4(k) x 16(m) block; lane L addresses
                        // row L/4, columns 4*(L%4)..+3 and receives column L of the 4 rows.
                        const int L = lane & 15;
                        const int row = ks * 16 + (lane >> 5) * 8 + (L >> 2);
                        const int col = wave * 64 + mi * 32 + ((lane >> 4) & 1) * 16 + (L & 3) * 4;
                        const uint16_t *q = stA + row * PITCH + col;
                        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))q);
                        s16x4 hi =
                            __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(q + 4 * PITCH));
                        u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                        af[mi].x = l2.x;
                        af[mi].y = l2.y;
                        af[mi].z = h2.x;
                        af[mi].w = h2.y;
                    }
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni)
                        bf[ni] = *reinterpret_cast<const u32x4 *>(stB + ((ni * KS + ks) * 64 + lane) * 8);
                };
                if (!have_next)
                    publish();
                TW_LDS_BARRIER(); // time slot 0: step 0 is being staged
                if (!have_next) {
                    nxt = published();
                    have_next = true;
                }
                for (int s = 0; s < nsteps; ++s) {
                    TW_WS_STAMP(s, 0, 0)
                    if (w_active) {
                        u32x4 af[2][MI], bf[2][NI];
                        frags(s, 0, af[0], bf[0]);
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            if (ks + 1 < KS)
                                frags(s, ks + 1, af[(ks + 1) & 1], bf[(ks + 1) & 1]);
#pragma unroll
                            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                                for (int mi = 0; mi < MI; ++mi)
                                    acc[mi][ni] = E::mfma(af[ks & 1][mi], bf[ks & 1][ni], acc[mi][ni]);
                        }
                    }
                    TW_WS_STAMP(s, 1, 0)
                    TW_LDS_BARRIER();
                }

                // epilogue: alpha/beta in fp32, round, hand the tile over through LDS
                const int32_t *const nlist = p.kept_n + u.kn_off;
                float scale = p.alpha;
                const bool fused = (p.bias || p.act) && p.beta == 0.0f;
                if (p.beta != 0.0f) {
                    // rare path: fold alpha, beta*C, the bias and the activation into the
                    // accumulators first (C is read on kept columns only)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int j = ni * 32 + (lane & 31);
                        const int col = j < u.n_cnt ? u.col0 + nlist[j] : 0;
                        const int64_t coff = (int64_t)col * p.ldc;
#pragma unroll
                        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int m = m0 + wave * 64 + mi * 32 + (lane >> 5) * 4 + (r >> 2) * 8 + (r & 3);
                                float old = 0.0f;
                                if (p.beta != 0.0f && j < u.n_cnt && m < cur.m_end)
                                    old = E::from_bits(C[coff + m]);
                                acc[mi][ni][r] =
                                    tw_finish(p.alpha * acc[mi][ni][r] + p.beta * old, p.bias, col, p.act);
                            }
                    }
                    scale = 1.0f;
                }
                if (fused) {
                    // bias (handed over through LDS by the moving waves) and activation in fp32,
                    // one rounding; the activation is a compile-time constant of each copy
                    auto stage_fused = [&](auto act_tag) {
                        constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni) {
                            const int j = ni * 32 + (lane & 31);
                            const float bj = p.bias ? s_bias[j] : 0.0f;
#pragma unroll
                            for (int mi = 0; mi < MI; ++mi) {
                                const int mloc = wave * 64 + mi * 32 + (lane >> 5) * 4;
#pragma unroll
                                for (int r4 = 0; r4 < 4; ++r4) {
                                    float v[4];
#pragma unroll
                                    for (int e = 0; e < 4; ++e)
                                        v[e] = tw_activate(scale * acc[mi][ni][r4 * 4 + e] + bj, ACT);
                                    u32x2 pk;
                                    pk.x = E::to_bits(v[0]) | (E::to_bits(v[1]) << 16);
                                    pk.y = E::to_bits(v[2]) | (E::to_bits(v[3]) << 16);
                                    *reinterpret_cast<u32x2 *>(smem + j * CPITCH + mloc + r4 * 8) = pk;
                                }
                            }
                        }
                    };
                    switch (p.act) {
                    case TW_ACT_RELU:
                        stage_fused(std::integral_constant<int, TW_ACT_RELU>());
                        break;
                    case TW_ACT_GELU:
                        stage_fused(std::integral_constant<int, TW_ACT_GELU>());
                        break;
                    case TW_ACT_TANH:
                        stage_fused(std::integral_constant<int, TW_ACT_TANH>());
                        break;
                    default:
                        stage_fused(std::integral_constant<int, TW_ACT_NONE>());
                        break;
                    }
                } else {
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int j = ni * 32 + (lane & 31); // compact column inside the unit
#pragma unroll
                        for (int mi = 0; mi < MI; ++mi) {
                            const int mloc = wave * 64 + mi * 32 + (lane >> 5) * 4;
#pragma unroll
                            for (int r4 = 0; r4 < 4; ++r4) {
                                u32x2 pk;
                                pk.x = E::to_bits(scale * acc[mi][ni][r4 * 4 + 0]) |
                                       (E::to_bits(scale * acc[mi][ni][r4 * 4 + 1]) << 16);
                                pk.y = E::to_bits(scale * acc[mi][ni][r4 * 4 + 2]) |
                                       (E::to_bits(scale * acc[mi][ni][r4 * 4 + 3]) << 16);
                                *reinterpret_cast<u32x2 *>(smem + j * CPITCH + mloc + r4 * 8) = pk;
                            }
                        }
                    }
                }
                pick_up();
                if (tid == 0 && announced)
                    asm volatile("" : "+v"(t_done)); // the count has returned: read it before the stores
                TW_LDS_BARRIER(); // the C tile is staged
                store_tile(u, m0, cur.m_end);
            }
            TW_LDS_BARRIER(); // LDS may be reused now
            cur = nxt;
            have_next = false;
#ifdef TW_EXP_TIMING
            ++ws_item;
#endif
        }
#ifdef TW_EXP_TIMING
        if (blockIdx.x == 0 && tid == 0) {
            s_ws[250] = __builtin_readcyclecounter();
            s_ws[251] = __builtin_amdgcn_s_memrealtime();
        }
        __builtin_amdgcn_s_waitcnt(0);
#if TW_EXP_TIMING == 2
        if (tid == 0 && blockIdx.x < 256)
            reinterpret_cast<unsigned *>(p.dbg)[blockIdx.x * 2 + 1] = (unsigned)__builtin_amdgcn_s_memrealtime();
#else
        if (blockIdx.x == 0 && tid < 256)
            reinterpret_cast<unsigned long long *>(p.dbg)[tid] = s_ws[tid];
#endif
#endif
        // the workgroup counted last re-arms the ticket slot for the next launch: every
        // workgroup's claims had returned before it was counted.  Plain stores, made visible by
        // the end of the kernel; a device-scope fence here would write back and invalidate this
        // XCD's L2 under the workgroups that still stream through it.
        if (tid == 0 && t_done == (int)gridDim.x - 1) {
            p.ticket[0] = 0;
            p.ticket[1] = 0;
        }
    }
}

// ---------------------------------------------------------------------------------
// Layout-generic kernel: any combination of K-major / row-major A and C through element
// strides.  One workgroup (4 waves, 128 x 128 tile, 32-row steps) per work item in queue
// order, single-buffered.  Gathered A elements are fetched one by one with the lanes running
// along the kept-K list (for row-major A the 32 kept columns of a row sit within a few cache
// lines), staged as [m][k] so that an MFMA operand is a plain 16-byte LDS read.  This is the
// functional path for the layouts the pipelined K-major kernel does not take.
template <int DT>
__global__ void __launch_bounds__(256, 2) tw_gemm_generic_kernel(const GemmArgs p, int64_t sa_m,
                                                                  int64_t sa_k, int64_t sc_m,
                                                                  int64_t sc_n)
{
    constexpr int BM = 128, BK = 32, KP = BK + 8; // halfs per staged row (80 B)
    constexpr int PKS = kBlockK / kMfmaK;
    constexpr int CP = BM + 8;
    using E = Elem<DT>;
    __shared__ __align__(16) uint16_t smem[128 * CP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    const uint16_t *const A = reinterpret_cast<const uint16_t *>(p.A);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    const uint16_t *const Bp = reinterpret_cast<const uint16_t *>(p.Bp);
    const int item = blockIdx.x;

    if (item >= p.n_gemm_items) { // zero-fill item: pruned columns receive beta*C
        const int z = item - p.n_gemm_items;
        const int zt = z / p.n_mblk;
        const int m0 = (z - zt * p.n_mblk) * BM;
        const TileDev t = p.tiles[zt];
        for (int e = tid; e < t.n_pruned * BM; e += 256) {
            const int j = e % t.n_pruned, m = m0 + e / t.n_pruned;
            if (m < p.M) {
                const int c = t.col0 + p.pruned_n[t.pn_off + j];
                uint16_t *dst = C + (int64_t)m * sc_m + (int64_t)c * sc_n;
                const float old = p.beta != 0.0f ? p.beta * E::from_bits(*dst) : 0.0f;
                *dst = (uint16_t)E::to_bits(tw_finish(old, p.bias, c, p.act));
            }
        }
        return;
    }
    const int ui = item / p.n_mblk;
    const int m0 = (item - ui * p.n_mblk) * BM;
    const UnitDev u = p.units[ui];
    const int32_t *const klist = p.kept_k + u.kk_off;
    const int32_t *const nlist = p.kept_n + u.kn_off;
    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[mi][ni][r] = 0.0f;

    const int kk_l = tid & 31, m_l = tid >> 5; // this thread stages column kk_l of rows m_l + 8 i
    for (int s = 0; s < u.k_pad / BK; ++s) {
        const int kk = s * BK + kk_l;
        const bool k_ok = kk < u.k_kept;
        const int64_t koff = k_ok ? (int64_t)klist[kk] * sa_k : 0;
#pragma unroll 4
        for (int i = 0; i < BM / 8; ++i) {
            const int ml = m_l + 8 * i;
            uint16_t v = 0;
            if (k_ok && m0 + ml < p.M)
                v = A[(int64_t)(m0 + ml) * sa_m + koff];
            smem[ml * KP + kk_l] = v;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            u32x4 af[2], bf[2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
                af[mi] = *reinterpret_cast<const u32x4 *>(
                    smem + (wm * 64 + mi * 32 + (lane & 31)) * KP + ks * 16 + (lane >> 5) * 8);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const int nb = wn * 2 + ni;
                const int k16 = s * 2 + ks; // 16-row step; the weight is packed per kBlockK rows
                bf[ni] = *reinterpret_cast<const u32x4 *>(
                    Bp + u.b_off +
                    ((((int64_t)(k16 / PKS) * u.nblk + u.nb0 + (nb < u.nb_cnt ? nb : 0)) * PKS +
                      (k16 % PKS)) * 64 + lane) * 8);
            }
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
                    acc[mi][ni] = E::mfma(af[mi], bf[ni], acc[mi][ni]);
        }
        __syncthreads();
    }
    // epilogue: stage alpha*acc as fp32-rounded 16-bit [j][m], then strided stores
    float *const sF = reinterpret_cast<float *>(smem); // 64 columns x 128 rows of fp32 per half
    for (int half = 0; half < 2; ++half) {
        if (wn == half) {
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int jl = ni * 32 + (lane & 31);
                        const int ml = wm * 64 + mi * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                        sF[jl * (BM + 1) + ml] = acc[mi][ni][r];
                    }
        }
        __syncthreads();
        for (int e = tid; e < 64 * BM; e += 256) {
            const int jl = e & 63, ml = e >> 6;
            const int j = half * 64 + jl, m = m0 + ml;
            if (j < u.n_cnt && m < p.M) {
                const int c = u.col0 + nlist[j];
                uint16_t *dst = C + (int64_t)m * sc_m + (int64_t)c * sc_n;
                float v = p.alpha * sF[jl * (BM + 1) + ml];
                if (p.beta != 0.0f)
                    v += p.beta * E::from_bits(*dst);
                *dst = (uint16_t)E::to_bits(tw_finish(v, p.bias, c, p.act));
            }
        }
        __syncthreads();
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

// outputs above this size are written through to memory: the size of one XCD's L2
constexpr int64_t kStoreThroughBytes = 4 << 20;

static int env_int(const char *name, int dflt)
{
    const char *v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}

// Tile shapes: 0: 256 x 128 (8 waves of 64 x 64, one workgroup per CU), 1: 128 x 128 (4 waves,
// two per CU), 2: 512 x 64, 3: 256 x 64 (the two shapes for tiles of at most 64 kept columns),
// 4: 256 x 128 wave-specialised (the default for wider tiles; shape 0 remains for operands the
// 32-bit offsets of shape 4 cannot address).
struct Shape {
    int bm, wgs_per_cu;
};
static const Shape kShapes[5] = {{256, 1}, {128, 2}, {512, 1}, {256, 2}, {256, 1}};

template <int DT> static void launch_kmajor(int shape, const GemmArgs &a, int grid, hipStream_t s)
{
    switch (shape) {
    case 0:
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, 4, 2, 64, 2, 1>), dim3(grid), dim3(512), 0, s, a);
        break;
    case 1:
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, 2, 2, 32, 3, 2>), dim3(grid), dim3(256), 0, s, a);
        break;
    case 2:
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, 8, 1, 32, 2, 1>), dim3(grid), dim3(512), 0, s, a);
        break;
    case 3:
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, 4, 1, 32, 2, 2>), dim3(grid), dim3(256), 0, s, a);
        break;
    default: // 4: wave-specialised 256 x 128
        hipLaunchKernelGGL((tw_gemm_ws_kernel<DT>), dim3(grid), dim3(512), 0, s, a);
        break;
    }
}

} // namespace tw

using namespace tw;

extern "C" {

int tw_gemm(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C, int c_layout,
            int64_t ldc, int M, float alpha, float beta, int pruned_cols, void *stream)
{
    return tw_gemm_ex(plan, A, a_layout, lda, C, c_layout, ldc, M, alpha, beta, pruned_cols, nullptr,
                      stream);
}

int tw_gemm_ex(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C, int c_layout,
               int64_t ldc, int M, float alpha, float beta, int pruned_cols, const tw_epilogue *ep,
               void *stream)
{
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    if (ep && (ep->activation < TW_ACT_NONE || ep->activation > TW_ACT_TANH))
        return fail(TW_ERR_LAYOUT, "activation=%d: unknown", ep->activation);
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
    {
        // the plan's tables and packed weight live on the device it was built on
        int dev = -1;
        TW_HIP(hipGetDevice(&dev));
        if (dev != plan->device)
            return fail(TW_ERR_DEVICE, "the plan was built on device %d, the current device is %d",
                        plan->device, dev);
    }
    if (a_layout != TW_LAYOUT_KMAJOR || c_layout != TW_LAYOUT_KMAJOR) {
        // layout-generic path (element strides), 128-row blocks, one workgroup per item
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
        a.n_mblk = (M + 127) / 128;
        a.n_gemm_items = plan->n_units * a.n_mblk;
        a.n_pipe_items = plan->n_pipe_units * a.n_mblk;
        a.n_zero_tiles = pruned_cols == TW_PRUNED_ZERO ? plan->n_zero_tiles : 0;
        a.n_items = a.n_gemm_items + a.n_zero_tiles * a.n_mblk;
        a.alpha = alpha;
        a.beta = beta;
        a.ticket = nullptr;
        a.dbg = nullptr;
        a.n_arg_units = 0;
        a.bias = ep ? ep->bias : nullptr;
        a.act = ep ? ep->activation : TW_ACT_NONE;
        a.store_through = 0;
        if (a.n_items == 0)
            return TW_OK;
        const int64_t sa_m = a_layout == TW_LAYOUT_KMAJOR ? 1 : lda;
        const int64_t sa_k = a_layout == TW_LAYOUT_KMAJOR ? lda : 1;
        const int64_t sc_m = c_layout == TW_LAYOUT_KMAJOR ? 1 : ldc;
        const int64_t sc_n = c_layout == TW_LAYOUT_KMAJOR ? ldc : 1;
        if (plan->dtype == TW_F16)
            hipLaunchKernelGGL((tw_gemm_generic_kernel<TW_F16>), dim3(a.n_items), dim3(256), 0,
                               (hipStream_t)stream, a, sa_m, sa_k, sc_m, sc_n);
        else
            hipLaunchKernelGGL((tw_gemm_generic_kernel<TW_BF16>), dim3(a.n_items), dim3(256), 0,
                               (hipStream_t)stream, a, sa_m, sa_k, sc_m, sc_n);
        TW_HIP(hipGetLastError());
        return TW_OK;
    }

    // Shape choice: the large tile halves the weight traffic per row of A, but needs enough
    // work items to fill the chip; otherwise the small tile with two workgroups per CU.
    const bool narrow = plan->max_unit_n <= 64;
    // the wave-specialised kernel addresses A with 32-bit byte offsets
    const bool ws_ok = (uint64_t)plan->K * (uint64_t)lda * 2u < (1ull << 32);
    int shape = narrow ? 2 : (ws_ok ? 4 : 0);
    {
        const int forced = env_int("TWGEMM_SHAPE", -1);
        const int64_t big_items =
            (int64_t)plan->n_units * ((M + kShapes[shape].bm - 1) / kShapes[shape].bm);
        if (forced >= 0 && forced < 5 && (forced == 2 || forced == 3) == narrow && (forced != 4 || ws_ok))
            shape = forced;
        else if (big_items * 5 < 3 * (int64_t)plan->cu_count && (narrow || M <= 128))
            shape = narrow ? 3 : 1; // too few large items to occupy the chip (for wide tiles the
                                    // wave-specialised kernel still wins unless a 128-row block
                                    // holds all of M)
    }
    const int BM = kShapes[shape].bm;
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
    a.n_pipe_items = plan->n_pipe_units * a.n_mblk;
    const int per_cu = env_int("TWGEMM_WGS_PER_CU", kShapes[shape].wgs_per_cu);
    a.n_zero_tiles = pruned_cols == TW_PRUNED_ZERO ? plan->n_zero_tiles : 0;
    a.n_items = a.n_gemm_items + a.n_zero_tiles * a.n_mblk;
    a.alpha = alpha;
    a.beta = beta;
    a.bias = ep ? ep->bias : nullptr;
    a.act = ep ? ep->activation : TW_ACT_NONE;
    // an output larger than one L2 is written through (see store_chunk)
    a.store_through = (int64_t)M * plan->N * 2 > kStoreThroughBytes;
    if (a.n_items == 0)
        return TW_OK;
    const unsigned slot =
        __atomic_fetch_add(&plan->next_slot, 1u, __ATOMIC_RELAXED) % (unsigned)kTicketSlots;
    a.ticket = plan->d_tickets + 2 * slot;
    a.dbg = plan->d_tickets + 2 * kTicketSlots;
    a.n_arg_units = plan->n_units <= kMaxArgUnits ? plan->n_units : 0;
    for (int i = 0; i < a.n_arg_units; ++i)
        a.arg_units[i] = plan->h_units[i];

    const int grid = (int)std::min<int64_t>(a.n_items, (int64_t)plan->cu_count * per_cu);
    hipStream_t s = (hipStream_t)stream;
    if (plan->dtype == TW_F16)
        launch_kmajor<TW_F16>(shape, a, grid, s);
    else
        launch_kmajor<TW_BF16>(shape, a, grid, s);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

#ifdef TW_EXP_TIMING
int tw_exp_read_debug(const tw_plan *plan, void *host, int nbytes)
{
    return hipMemcpy(host, plan->d_tickets + 2 * kTicketSlots, nbytes, hipMemcpyDeviceToHost);
}
#endif

int tw_stream_gemm_nn(int M, int N, int K, int dtype, float alpha, const void *A, const void *B,
                      float beta, void *C, int block_num, const int32_t *N_cal,
                      const int32_t *K_cal, const int32_t *const *mask_n,
                      const int32_t *const *mask_k, const int64_t *off_B, const int64_t *off_C,
                      void *stream)
try {
    if (M > 0 && (M & 7))
        return fail(TW_ERR_ALIGNMENT, "M=%d must be a multiple of 8 here (lda = ldc = M)", M);
    tw_plan *plan = nullptr;
    int st = tw_plan_from_stream_operands(M, N, K, dtype, B, block_num, N_cal, K_cal, mask_n,
                                          mask_k, off_B, off_C, &plan);
    if (st)
        return st;
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
TW_CATCH_TO_STATUS

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
