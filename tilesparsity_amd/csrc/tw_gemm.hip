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
#include "tw_device.h"

#include <algorithm>
#include <atomic>
#include <mutex>
#include <type_traits>
#include <cstddef>
#include <cstdlib>

namespace tw {

// ---------------------------------------------------------------------------------
// Work queue (see GemmArgs): entry q of queue x names one item, or nothing past the end.
enum ItemKind { ITEM_PIPE = 0, ITEM_NOSTEP = 1, ITEM_ZERO = 2, ITEM_END = 3 };

struct Work {
    int kind; // ItemKind
    int u;    // column of the item matrix: piece of a unit, or n_gemm_u + tile to fill
    int m0;   // first row
    int rows; // rows [m0, m0 + rows) of A and C, cut at M by the caller
};

__device__ __forceinline__ int queue_length(const GemmArgs &p, int x)
{
    return p.n_own_items + (p.n_tail_items > x ? (p.n_tail_items - x + kXcd - 1) / kXcd : 0);
}

// (bm: rows of a row block of this launch)
__device__ __forceinline__ Work queue_entry(const GemmArgs &p, int x, int q, int bm)
{
    Work w;
    w.kind = ITEM_END;
    w.u = 0;
    w.m0 = 0;
    w.rows = bm;
    if (q < p.n_own_items) {
        const int i = q / p.n_all_u;
        w.u = q - i * p.n_all_u;
        w.m0 = (x * p.n_own + i) * bm;
    } else {
        const int j = (q - p.n_own_items) * kXcd + x;
        if (j >= p.n_tail_items)
            return w;
        if (p.n_bal > 0) {
            // columns with row blocks of their own height: column u owns the items
            // bal_first[u] .. bal_first[u + 1] - 1 of the list
            int u = 0;
#pragma unroll
            for (int i = 1; i < kBalColumns; ++i)
                u += i < p.n_bal && j >= p.bal_first[i];
            w.u = u;
            w.rows = p.bal_rows[u];
            w.m0 = (j - p.bal_first[u]) * w.rows;
        } else if (p.rb_major) {
            // all columns of a row block (heaviest first) before the next row block
            const int mb = j / p.n_all_u;
            w.u = j - mb * p.n_all_u;
            w.m0 = (kXcd * p.n_own + mb) * bm;
        } else {
            w.u = j / p.n_tail_mblk;
            w.m0 = (kXcd * p.n_own + (j - w.u * p.n_tail_mblk)) * bm;
        }
    }
    w.kind = w.u < p.n_pipe_u ? ITEM_PIPE : (w.u < p.n_gemm_u ? ITEM_NOSTEP : ITEM_ZERO);
    return w;
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
    // A ticket is an index into this workgroup's queue: GEMM items with at least one step,
    // GEMM items of units that keep no K row (their kept columns receive alpha*0 + beta*C)
    // and zero-fill items.  The workgroup always holds the ticket of its current and its next
    // item and has the atomic for the one after in flight, so a ticket's round trip is hidden
    // behind a whole item.
    const int qx = blockIdx.x % kXcd;
    const int qlen = queue_length(p, qx);
    // (an item is told by its column of the item matrix, compared with the bounds each time)
    struct Item {
        int col;
        int m0;
        UnitDev u; // col < n_gemm_u
    };
    auto make_item = [&](int ticket) {
        Item it;
        const Work w = queue_entry(p, qx, ticket, BM);
        it.col = w.kind == ITEM_END ? p.n_all_u : w.u;
        it.m0 = w.m0;
        if (it.col < p.n_gemm_u)
            it.u = load_unit(p, it.col);
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
    const int ticket_base = gridDim.x / kXcd; // workgroups per queue
    int t_pending = 0;   // thread 0: claim in flight
    bool closed = false; // thread 0: the queue is exhausted, no claim is in flight
    int t_done = -1;     // thread 0: workgroups counted as done before this one
    if (tid == 0) {
        if ((int)(blockIdx.x / kXcd) < qlen) {
            t_pending = atomicAdd(&p.ticket[qx], 1);
        } else { // nothing for this workgroup: it only counts itself as done
            closed = true;
            t_done = atomicAdd(&p.ticket[kXcd], 1);
        }
    }
    Item cur = make_item(blockIdx.x / kXcd);
    Item nxt = cur;
    bool have_next = false; // nxt is known for the current item
    // Publishes the claim in flight as the next item and starts the claim after it.  A ticket
    // past the end makes the current item the workgroup's last: all its claims have returned, so
    // it counts itself as done right away (the workgroup counted last re-arms the slot when it
    // leaves) and that count's round trip is over before the item ends.
    auto claim_next = [&]() {
        if (tid == 0) {
            const int t = closed ? qlen : ticket_base + t_pending;
            s_tk[0] = t;
            if (!closed) {
                if (t < qlen) {
                    t_pending = atomicAdd(&p.ticket[qx], 1);
                } else {
                    closed = true;
                    t_done = atomicAdd(&p.ticket[kXcd], 1);
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
    while (cur.col < p.n_all_u) {
        // the very first claim of a workgroup is published after the first item's loads have
        // been issued, so that its round trip overlaps with them
        if (!first || cur.col >= p.n_pipe_u)
            claim_next();
        first = false;
        if (cur.col >= p.n_gemm_u) {
            // ---- zero-fill item: pruned columns of one tile receive beta*C ----
            const int m = cur.m0 + chunk * 8;
            const TileDev t = p.tiles[cur.col - p.n_gemm_u];
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
                stage(s, a_ring[r], b_ring[r]);
                __syncthreads();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    frags(s, ks, af, bf);
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                        for (int mi = 0; mi < 2; ++mi)
                            acc[mi][ni] = E::mfma(af[mi], bf[ni], acc[mi][ni]);
                }
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
            if (!have_next)
                claim_next();
            int s0 = 0;
            // steady state: every iteration issues, stages and multiplies, no conditionals
            for (; s0 + R + D <= nsteps; s0 += R) {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    iteration(s0 + r, r, true);
            }
            // The next item's index words are fetched before the drain, so that its first row
            // loads can be issued right after this item's last step and fly over the epilogue.
            const bool chain = nxt.col < p.n_pipe_u;
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

        __syncthreads();
        cur = nxt;
        have_next = false;
    }

    // the workgroup counted last re-arms the ticket slot for the next launch: every workgroup's
    // claims had returned before it was counted.  Plain stores, made visible by the end of the
    // kernel; a device-scope fence here would write back and invalidate this XCD's L2 under the
    // workgroups that still stream through it.
    if (tid == 0 && t_done == (int)gridDim.x - 1) {
#pragma unroll
        for (int i = 0; i <= kXcd; ++i)
            p.ticket[i] = 0;
    }
}

// Scheduling hints for NMM MFMAs of one 16-row k step: each MFMA is followed by its share of
// the NRD LDS reads that fetch the operands of the next k step (none after the last step).
template <int NRD, int NMM, int I, bool READS> __device__ __forceinline__ void sched_mfma_with_reads()
{
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
    constexpr int n = NRD * (I + 1) / NMM - NRD * I / NMM;
    if constexpr (READS && n > 0)
        __builtin_amdgcn_sched_group_barrier(0x100, n, 0); // n LDS reads
    if constexpr (I + 1 < NMM)
        sched_mfma_with_reads<NRD, NMM, I + 1, READS>();
}

// ---------------------------------------------------------------------------------
// Wave-specialised BM x BN kernel.  Half of the waves only multiply: multiplying wave w owns
// rows [w * RW, (w + 1) * RW) of the row block and all BN compact columns (MI x NI MFMA blocks
// of 32 x 32).  The other half only move data: they gather the kept rows of A and the packed
// weight global -> registers -> LDS, R steps of 64 rows in flight.  Both halves meet at one
// barrier per step: while the multiplying waves read stage s & 1, the moving waves fill stage
// (s + 1) & 1, so LDS traffic, vector-memory traffic and MFMA work overlap instead of following
// each other.  One multiplying and one moving wave share a SIMD.
//   BM = 128: 2 + 2 waves, two or more workgroups per CU (one's start-up and epilogue hide
//             under the other's steps: the shape for items of few steps);
//   BM = 256: 4 + 4 waves, one workgroup per CU (half the weight traffic per row of A);
//   BM = 512: 4 + 4 waves, each multiplying wave 128 rows (tiles of at most 64 kept columns).
// The first loads of the next item are issued during the last step of the current one and
// fly over its epilogue.
template <int DT, int BM, int BN, int R, bool DMA = false>
__global__ void __launch_bounds__(BM == 128 ? 256 : 512, 2) tw_gemm_ws_kernel(const GemmArgs p)
{
    constexpr int NMW = BM == 128 ? 2 : 4;     // multiplying waves, and as many moving waves
    constexpr int NPM = 64 * NMW;              // threads of either half
    constexpr int NT = 2 * NPM;
    constexpr int BK = 64;
    constexpr int KS = BK / kMfmaK, PKS = kBlockK / kMfmaK;
    // (R register slots = steps of loads in flight per moving wave)
    constexpr int RW = BM / NMW;               // rows of a multiplying wave
    constexpr int MI = RW / 32, NI = BN / kMfmaN;
    constexpr int CPR = BM / 8;                // 16-byte chunks per staged A row / stored C column
    constexpr int RG = 64 / CPR;               // rows a moving wave covers with one load
    constexpr int RPW = BK / NMW;              // rows of a step per moving wave
    constexpr int PASSES = RPW / RG;           // A loads per moving thread and step
    constexpr int BPASS = BN * BK / 8 / NPM;   // weight loads per moving thread and step
    constexpr int PITCH = BM + TW_A_PAD;
    // DMA: the moving waves issue loads that write LDS directly.  A load of a wave (64 lanes x 16
    // bytes) lands as 1 KB in one piece, so a stage of A is 32 slots of two rows of the step (the
    // rows mw * 16 + ps and + 8 of moving wave mw's load ps: what one transposed read's lanes
    // 0 - 31 and 32 - 63 address), 64 bytes of padding behind each slot so that the four slots a
    // transposed read touches fall into four different groups of 16 banks; three stages, since a
    // stage is written by loads issued two steps ahead instead of passing through registers.
    constexpr int SLOTB = 1024 + 64; // bytes
    constexpr int NST = DMA ? 3 : 2;
    constexpr int ASTAGE = DMA ? (BK / 2) * SLOTB / 2 : BK * PITCH, BSTAGE = BN * BK;
    constexpr int CPITCH = BM + 4;
    constexpr int PIPE = NST * (ASTAGE + BSTAGE);
    // DMA: the stages lie one behind the other, each its rows of A followed by its weight, and the
    // C tile of an item is staged 64 columns at a time in the stage its last step was multiplied
    // from, so that the other two can already receive the first steps of the workgroup's next item
    constexpr int STG = ASTAGE + BSTAGE;
    constexpr int CROUNDS = DMA ? BN / 64 : 1;
    static_assert(!DMA || 64 * CPITCH <= STG, "64 columns of the C tile fit one stage");
    constexpr int SMEM = DMA ? PIPE : (PIPE > BN * CPITCH ? PIPE : BN * CPITCH);
    static_assert(!DMA || BM == 256, "the direct-to-LDS form is laid out for 256-row items");
    static_assert(BK == kBlockK && KS == PKS, "one packed weight step per main-loop step");
    static_assert(CPR <= 64 && PASSES % 4 == 0 && BPASS >= 1 && BN <= NPM, "tile shape");
    using E = Elem<DT>;

    __shared__ __align__(16) uint16_t smem[SMEM];
    __shared__ int s_tk[2];
    __shared__ int s_cols[BN];   // output columns of the current item's unit

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint16_t *const A = reinterpret_cast<const uint16_t *>(p.A);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    const uint16_t *const Bp = reinterpret_cast<const uint16_t *>(p.Bp);
    // (DMA: stage i holds its rows of A at sA + i * STG and its weight at sB + i * STG)
    uint16_t *const sA = smem;
    uint16_t *const sB = DMA ? smem + ASTAGE : smem + NST * ASTAGE;

    // this workgroup's queue
    const int qx = blockIdx.x % kXcd;
    const int qi = blockIdx.x / kXcd;        // position among the queue's workgroups
    const int qwg = gridDim.x / kXcd;        // workgroups per queue
    const int qlen = queue_length(p, qx);

    // An item is told by its column of the item matrix: below n_pipe_u a GEMM item with steps,
    // below n_gemm_u one without, below n_all_u a tile to fill, n_all_u past the end.  (The
    // tests below compare the column with these bounds each time, rather than a kind worked out
    // once: with the latter the compiler threads the item loop into copies that each keep their
    // own set of load registers.)
    struct Item {
        int col;
        int m0, m_end; // rows [m0, m_end) of A and C, at most BM of them
        UnitDev u;     // col < n_gemm_u
    };
    auto make_item = [&](int ticket) {
        Item it;
        const Work w = queue_entry(p, qx, ticket, BM);
        it.col = w.kind == ITEM_END ? p.n_all_u : w.u;
        it.m0 = w.m0;
        it.m_end = it.m0 + w.rows < p.M ? it.m0 + w.rows : p.M;
        if (it.col < p.n_gemm_u)
            it.u = load_unit(p, it.col);
        return it;
    };
    auto is_end = [&](const Item &it) { return it.col >= p.n_all_u; };
    auto has_steps = [&](const Item &it) { return it.col < p.n_pipe_u; };
    auto is_fill = [&](const Item &it) { return it.col >= p.n_gemm_u; };
    // Both halves of the workgroup walk the same item sequence and execute the same sequence
    // of barriers; thread 0 (a multiplying wave) owns the ticket counter.
    // The first two items of a workgroup are fixed (entries qi and qi + qwg of its queue), so
    // that no atomic's round trip sits between the start of the kernel and the first loads;
    // the queue's counter hands out the entries after those.
    const int ticket_base = 2 * qwg;
    int t_pending = 0;      // thread 0: result of the claim in flight
    int t_next = qi + qwg;  // thread 0: the next ticket once known, or -1
    bool closed = false;    // thread 0: no claim of this workgroup is in flight, none will follow
    bool announced = false; // thread 0: the workgroup has been counted as done with the counter
    int t_done = -1;        // thread 0: workgroups counted before this one (atomic's result)
    if (tid == 0) {
        if (qi < qlen) {
            t_pending = atomicAdd(&p.ticket[qx], 1);
        } else { // nothing for this workgroup: it only counts itself as done
            closed = true;
            announced = true;
            t_done = atomicAdd(&p.ticket[kXcd], 1);
        }
    }
    // Picks up the claim in flight and starts the one after it, unless the queue is exhausted.
    // Called before an item's output stores are issued: memory operations complete in order, so
    // waiting for an atomic issued after them (or overwriting its register) would wait for the
    // stores as well.
    auto pick_up = [&]() {
        if (tid == 0 && t_next < 0) {
            if (closed) {
                t_next = qlen;
            } else {
                t_next = ticket_base + t_pending;
                asm volatile("" : "+v"(t_next)); // here, not where it is published
                if (t_next < qlen)
                    t_pending = atomicAdd(&p.ticket[qx], 1);
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
        if (t_next >= qlen && !announced) {
            if (!closed) {
                // the second fixed item is already past the end: the first claim is in flight
                asm volatile("" ::"v"(t_pending));
                closed = true;
            }
            t_done = atomicAdd(&p.ticket[kXcd], 1);
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
        publish();
        TW_LDS_BARRIER();
        const Item it = published();
        TW_LDS_BARRIER();
        return it;
    };
    // zero-fill item: pruned columns of one tile receive beta*C (all threads, no barrier)
    auto zero_fill = [&](const Item &it) {
        const int m = it.m0 + (tid % CPR) * 8;
        const TileDev t = p.tiles[it.col - p.n_gemm_u];
        for (int j = tid / CPR; j < t.n_pruned; j += NT / CPR) {
            const int c = t.col0 + p.pruned_n[t.pn_off + j];
            uint16_t *dst = C + (int64_t)c * p.ldc + m;
            u32x4 v = {0u, 0u, 0u, 0u};
            if ((p.beta != 0.0f || p.bias || p.act) && m < it.m_end) {
                uint32_t w[4] = {0u, 0u, 0u, 0u};
                for (int e = 0; e < 8 && m + e < it.m_end; ++e) {
                    const float old = p.beta != 0.0f ? p.beta * E::from_bits(dst[e]) : 0.0f;
                    w[e >> 1] |= E::to_bits(tw_finish(old, p.bias, c, p.act)) << ((e & 1) * 16);
                }
                v.x = w[0];
                v.y = w[1];
                v.z = w[2];
                v.w = w[3];
            }
            store_chunk(dst, v, m, it.m_end, p.store_through != 0);
        }
    };
    // scatters the staged C tile (all threads): whole columns col0 + kept_n[j], 16-byte stores
    // (the output columns come from s_cols, filled by the first multiplying wave)
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

    // (DMA) the moving waves store this item's C tile during the next item's first time slot:
    // a full tile (no lane, no column to skip) followed by an item of two steps or more
    auto defer_stores = [&](const Item &it, const Item &next) {
        return it.u.n_cnt == BN && it.m_end - it.m0 == BM && has_steps(next) && next.u.k_pad >= 2 * BK;
    };
    // (DMA) scatters round rd of a C tile staged at `ctile`: 64 columns at most.  By the multiplying
    // waves alone where the moving waves are already loading the workgroup's next item (they must
    // not have stores among their loads), else by all waves.
    auto store_round = [&](const uint16_t *ctile, int rd, const UnitDev &u, int m0, int m_end, bool all) {
        const int m_st = m0 + (tid % CPR) * 8;
        const int jn = u.n_cnt - rd * 64 < 64 ? u.n_cnt - rd * 64 : 64;
        for (int j = tid / CPR; j < jn; j += (all ? NT : NPM) / CPR) {
            const int c = s_cols[rd * 64 + j];
            const u32x2 lo = *reinterpret_cast<const u32x2 *>(ctile + j * CPITCH + (tid % CPR) * 8);
            const u32x2 hi = *reinterpret_cast<const u32x2 *>(ctile + j * CPITCH + (tid % CPR) * 8 + 4);
            u32x4 v;
            v.x = lo.x;
            v.y = lo.y;
            v.z = hi.x;
            v.w = hi.y;
            store_chunk(C + (int64_t)c * p.ldc + m_st, v, m_st, m_end, p.store_through != 0);
        }
    };

    if (wave >= NMW && DMA) {
        // ================= moving waves, loads straight into LDS ===========================
        // Lane (g, chunk) of moving wave mw fetches chunk `chunk` (8 consecutive m) of the kept
        // rows mw * 16 + g * 8 + ps, ps = 0 .. 7, of a step: load ps of the wave fills slot
        // mw * 8 + ps of the stage.  A row past the tile's list, a chunk past the item's rows and
        // every load of a step past the item's last get an offset beyond the buffer and arrive
        // as zeros.  Step j + 1 is issued in time slot j (its stage was multiplied two slots
        // ago), step j is waited for at the slot's end: two steps in flight.  Every slot issues
        // the same loads in the same order, so the waits are exact counts: behind the loads of
        // step j are the two index loads and the twelve loads of the slot that follows.
        if constexpr (DMA) {
        constexpr uint32_t kGone = 0xFFFFFFF0u;
        const int chunk = lane % CPR, g = lane / CPR;
        const int mw = wave - NMW;
        const int row0 = mw * RPW + g * PASSES;
        const uint32_t lda_b = (uint32_t)p.lda * 2u;
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        struct Idx {
            i32x4 k[PASSES / 4];
        };
        const __amdgpu_buffer_rsrc_t a_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.A), 0, (int)p.a_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t b_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.Bp), 0, (int)p.b_bytes, 0x00020000);
        TW_LDS(unsigned char) const lds_a = (TW_LDS(unsigned char))sA + mw * (PASSES * SLOTB);
        TW_LDS(unsigned char) const lds_b = (TW_LDS(unsigned char))sB + mw * 1024;
        // what the loads of an item's steps need
        struct Ctx {
            const int32_t *k_list; // the tile's padded list of kept rows (uniform)
            const char *k_base;
            uint32_t m0b, b_pack_b;
            uint32_t b_blk[BPASS]; // weight block of load bp (a block beyond the unit reads block 0), bytes into Bp
            int k_left0, nsteps;
            bool m_ok;
        };
        auto ctx_of = [&](const Item &it) {
            Ctx c;
            c.k_list = p.kept_k + it.u.kk_off;
            c.k_base = reinterpret_cast<const char *>(c.k_list) + row0 * 4;
            c.m0b = (uint32_t)it.m0 * 2u;
            c.m_ok = it.m0 + chunk * 8 < it.m_end;
            c.k_left0 = it.u.k_kept - row0;
            c.nsteps = it.u.k_pad / BK;
#pragma unroll
            for (int bp = 0; bp < BPASS; ++bp)
                c.b_blk[bp] = (uint32_t)(it.u.b_off * 2) + (uint32_t)(it.u.nb0 + (bp < it.u.nb_cnt ? bp : 0)) * 4096u + mw * 1024u;
            c.b_pack_b = (uint32_t)it.u.nblk * (PKS * 64 * 8 * 2);
            return c;
        };
        auto load_idx = [&](const Ctx &c, int st, Idx &ix) { // (the list is padded: always in bounds)
#pragma unroll
            for (int i = 0; i < PASSES / 4; ++i)
                ix.k[i] = *reinterpret_cast<const i32x4 *>(c.k_base + (int64_t)st * (BK * 4) + 16 * i);
        };
        // The same words through the scalar cache (the wave's sixteen rows of the step, of which a
        // lane picks its eight): for the next item's first steps, whose index words are fetched
        // while this item's loads are in flight.  A vector load there would make the compiler wait
        // for all of those first (it cannot tell, around the loop over the items, that the
        // registers it is about to overwrite are no longer being loaded into).
        auto load_idx_scalar = [&](const Ctx &c, int st, Idx &ix) {
            const auto *kp = (const __attribute__((address_space(4))) int32_t *)(uintptr_t)(c.k_list + st * BK + mw * RPW);
#pragma unroll
            for (int e = 0; e < PASSES; ++e)
                ix.k[e >> 2][e & 3] = g ? kp[PASSES + e] : kp[e];
        };
        // the BPASS + PASSES loads of step st of an item into stage `stage`
        auto issue = [&](const Ctx &c, int st, int stage, const Idx &ix) {
            const bool real = st < c.nsteps;
            const uint32_t vb = real ? (uint32_t)lane * 16u : kGone;
            const uint32_t sb = (real ? (uint32_t)st : 0u) * c.b_pack_b;
#pragma unroll
            for (int bp = 0; bp < BPASS; ++bp)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (TW_LDS(void))(lds_b + stage * (STG * 2) + bp * 4096),
                                                         16, (int)vb, (int)(c.b_blk[bp] + sb), 0, 0);
            const int k_left = real ? c.k_left0 - st * BK : 0;
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const uint32_t off = (ps < k_left && c.m_ok) ? (uint32_t)ix.k[ps >> 2][ps & 3] * lda_b + (uint32_t)chunk * 16u : kGone;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (TW_LDS(void))(lds_a + stage * (STG * 2) + ps * SLOTB),
                                                         16, (int)off, (int)c.m0b, 0, 0);
            }
        };
        // A time slot: the index loads of the step after next, then the loads of the next step
        // into LDS (twelve at 128 columns), then the meeting, at which only those may still be
        // in flight: the step before them has landed.  The loads into LDS are never removed or
        // reordered among themselves; the index loads are kept ahead of them by a compiler barrier
        // and are not counted on (the compiler drops those whose result nobody reads).  These
        // waves issue no stores (a wave's loads and stores retire in order and share the counter).
        auto fence = [&]() { asm volatile("" ::: "memory"); };
        auto meet = [&]() { asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(BPASS + PASSES) : "memory"); };
        // Deferred stores.  Where a full C tile (every column kept, 256 rows) is followed by
        // another item of this workgroup, these waves take the staged tile out of LDS into
        // registers (8 x 16 bytes a lane and round) and store it during the next item's first
        // time slot, so that the multiplying waves go straight on: the chip's stores then run
        // beside the next item's products instead of between two items.  The stores come BEHIND
        // the slot's loads in the wave's queue: the meetings of that slot and the next count them
        // in (the step waited for is older than they are), and by the slot after, two steps
        // later, memory has acknowledged them.  Their number is fixed (a full tile has no lane
        // and no column to skip), so the counts stay exact.
        constexpr int NDS = 8 * CROUNDS; // stores a lane defers
        auto meet_wide = [&](bool wide) {
            if (wide)
                asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(BPASS + PASSES + NDS) : "memory");
            else
                meet();
        };
        u32x2 dlo[NDS], dhi[NDS]; // the deferred tile: column pt / CPR + 8 i of round r, 8 rows m from m_st on
        int dcol[NDS];
        uint16_t *d_c = C;        // C + the lane's first row of the deferred tile
        bool deferred = false;
        const int pt = tid - NPM;
        auto take_round = [&](const uint16_t *ctile, int rd) {
            // LDS reads in asm: a C++ read would make the compiler wait for every load into LDS
            // that is on its way (it cannot tell that those go to other stages)
            const uint32_t a0 = (uint32_t)(uintptr_t)(TW_LDS(const uint16_t))(ctile + (pt / CPR) * CPITCH + (pt % CPR) * 8);
            const uint32_t c0 = (uint32_t)(uintptr_t)(TW_LDS(const int))(s_cols + rd * 64 + pt / CPR);
#pragma unroll
            for (int i = 0; i < 8; i += 4) {
                asm volatile("ds_read_b64 %0, %8 offset:%9\n\tds_read_b64 %1, %8 offset:%10\n\t"
                             "ds_read_b64 %2, %8 offset:%11\n\tds_read_b64 %3, %8 offset:%12\n\t"
                             "ds_read_b64 %4, %8 offset:%13\n\tds_read_b64 %5, %8 offset:%14\n\t"
                             "ds_read_b64 %6, %8 offset:%15\n\tds_read_b64 %7, %8 offset:%16\n\t"
                             "s_waitcnt lgkmcnt(0)"
                             : "=&v"(dlo[rd * 8 + i]), "=&v"(dhi[rd * 8 + i]), "=&v"(dlo[rd * 8 + i + 1]), "=&v"(dhi[rd * 8 + i + 1]),
                               "=&v"(dlo[rd * 8 + i + 2]), "=&v"(dhi[rd * 8 + i + 2]), "=&v"(dlo[rd * 8 + i + 3]), "=&v"(dhi[rd * 8 + i + 3])
                             : "v"(a0), "n"((i + 0) * 8 * CPITCH * 2), "n"((i + 0) * 8 * CPITCH * 2 + 8),
                               "n"((i + 1) * 8 * CPITCH * 2), "n"((i + 1) * 8 * CPITCH * 2 + 8),
                               "n"((i + 2) * 8 * CPITCH * 2), "n"((i + 2) * 8 * CPITCH * 2 + 8),
                               "n"((i + 3) * 8 * CPITCH * 2), "n"((i + 3) * 8 * CPITCH * 2 + 8)
                             : "memory");
            }
            asm volatile("ds_read_b32 %0, %8\n\tds_read_b32 %1, %8 offset:32\n\tds_read_b32 %2, %8 offset:64\n\t"
                         "ds_read_b32 %3, %8 offset:96\n\tds_read_b32 %4, %8 offset:128\n\tds_read_b32 %5, %8 offset:160\n\t"
                         "ds_read_b32 %6, %8 offset:192\n\tds_read_b32 %7, %8 offset:224\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(dcol[rd * 8 + 0]), "=&v"(dcol[rd * 8 + 1]), "=&v"(dcol[rd * 8 + 2]), "=&v"(dcol[rd * 8 + 3]),
                           "=&v"(dcol[rd * 8 + 4]), "=&v"(dcol[rd * 8 + 5]), "=&v"(dcol[rd * 8 + 6]), "=&v"(dcol[rd * 8 + 7])
                         : "v"(c0)
                         : "memory");
        };
        auto store_deferred = [&]() {
#pragma unroll
            for (int i = 0; i < NDS; ++i) {
                u32x4 v;
                v.x = dlo[i].x;
                v.y = dlo[i].y;
                v.z = dhi[i].x;
                v.w = dhi[i].y;
                uint16_t *const dst = d_c + (int64_t)dcol[i] * p.ldc;
                if (p.store_through)
                    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
                else
                    asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
            }
        };
        Item cur = make_item(qi);
        Item nxt = cur;
        bool have_next = false;
        int gs = 0;          // stage of the current item's step 0 is gs % NST: the steps of all items count on
        bool primed = false; // the current item's steps 0 and 1 are already on their way (see below)
        Idx i0, i1, n0, n1;
        while (!is_end(cur)) {
            if (!has_steps(cur)) {
                nxt = claim();
                have_next = true;
            }
            if (is_fill(cur)) {
                zero_fill(cur);
            } else {
                const int nsteps = has_steps(cur) ? cur.u.k_pad / BK : 0;
                bool next_primed = false;
                if (nsteps > 0) {
                    const Ctx c = ctx_of(cur);
                    if (!primed) {
                        load_idx(c, 0, i0);
                        load_idx(c, 1, i1);
                        fence();
                        issue(c, 0, gs % NST, i0);
                        fence();
                        load_idx(c, 2, i0);
                        fence();
                        issue(c, 1, (gs + 1) % NST, i1);
                    }
                    if (deferred)
                        store_deferred();
                    meet_wide(deferred); // time slot 0: step 0 has landed
                    if (!have_next) {
                        nxt = published();
                        have_next = true;
                    }
                    // the next item's first index words, for the loads that the last time slot
                    // issues on its behalf: fetched now, so that nobody waits for them there
                    const bool chain = nsteps >= 2 && has_steps(nxt);
                    Ctx cn = c;
                    if (chain) {
                        cn = ctx_of(nxt);
                        load_idx_scalar(cn, 0, n0);
                        load_idx_scalar(cn, 1, n1);
                    }
                    // time slots 1 .. nsteps - 2 issue the steps 2 .. nsteps - 1 (odd slots out
                    // of i0, even ones out of i1)
                    int j = 1;
                    for (; j + 2 < nsteps; j += 2) {
                        load_idx(c, j + 2, i1);
                        fence();
                        issue(c, j + 1, (gs + j + 1) % NST, i0);
                        meet_wide(deferred && j == 1);
                        load_idx(c, j + 3, i0);
                        fence();
                        issue(c, j + 2, (gs + j + 2) % NST, i1);
                        meet();
                    }
                    if (j + 1 < nsteps) {
                        issue(c, j + 1, (gs + j + 1) % NST, i0);
                        meet_wide(deferred && j == 1);
                        ++j;
                    }
                    if (nsteps >= 2) {
                        // The last time slot has no step of this item left to issue.  If the next
                        // item has steps, its steps 0 and 1 go out now and after the last
                        // multiplication (the C tile is staged in the stage of this item's last
                        // step, the other two are free): they fly over the epilogue, and the next
                        // item finds itself as after its first loads.
                        if (chain) {
                            issue(cn, 0, (gs + nsteps) % NST, n0);
                            meet_wide(deferred && j == 1);
                            TW_LDS_BARRIER(); // end of the last time slot
                            load_idx(cn, 2, i0);
                            fence();
                            issue(cn, 1, (gs + nsteps + 1) % NST, n1);
                            next_primed = true;
                        } else {
                            asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory"); // the last step has landed
                            TW_LDS_BARRIER(); // end of the last time slot
                        }
                    } else {
                        TW_LDS_BARRIER(); // end of the last time slot
                    }
                } else {
                    TW_LDS_BARRIER(); // end of the last time slot
                }
                // the multiplying waves stage the C tile, 64 columns at a time; these waves help
                // to store it unless they are loading the next item
                const uint16_t *const ctile = smem + ((nsteps > 0 ? gs + nsteps - 1 : gs) % NST) * STG;
                deferred = next_primed && defer_stores(cur, nxt);
                if (deferred)
                    d_c = C + cur.m0 + (pt % CPR) * 8;
#pragma unroll
                for (int r = 0; r < CROUNDS; ++r) {
                    TW_LDS_BARRIER(); // staged
                    if (deferred)
                        take_round(ctile, r);
                    else if (!next_primed)
                        store_round(ctile, r, cur.u, cur.m0, cur.m_end, true);
                    TW_LDS_BARRIER(); // stored, or taken
                }
                gs += nsteps;
                primed = next_primed;
            }
            TW_LDS_BARRIER(); // LDS may be reused now
            cur = nxt;
            have_next = false;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // nothing on its way into LDS when the workgroup ends
        }
    } else if (wave >= NMW) {
        // ================= moving waves ===================================================
        // A load of a wave covers RG kept rows (CPR lanes of 16 bytes each per row); lane
        // (g, chunk) moves chunk `chunk` (8 consecutive m) of the rows
        // mw * RPW + g * PASSES + 0 .. PASSES - 1 of a step.  The lane fetches the indices of its
        // own rows (a 16-byte load per four rows, the lanes of a row group share the address)
        // R steps before the row loads that use them.  Row addresses are a uniform base plus a
        // 32-bit byte offset per lane.
        const int pt = tid - NPM;
        const int chunk = lane % CPR, g = lane / CPR;
        const int mw = wave - NMW;
        const int row0 = mw * RPW + g * PASSES;        // this lane's first row of a step
        const uint32_t lda_b = (uint32_t)p.lda * 2u;   // bytes; K * lda * 2 < 2^32 (host check)
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        struct Idx {
            i32x4 k[PASSES / 4];
        };
        const uint32_t v_idx = (uint32_t)row0 * 4u;    // byte offset of this lane's indices in a step
        const uint32_t v_b = (uint32_t)(pt & 255) * 16u; // ... of its 16-byte piece in a weight block
        // every address is a workgroup-uniform base plus a 32-bit byte offset per lane
        struct Thr {
            const char *k_base;     // the unit's kept-K list (bytes), uniform
            const char *a_base;     // A + m0 (bytes), uniform
            const char *b_base[BPASS]; // weight block of load bp in step 0, uniform
            int64_t b_pack_b;
            uint32_t v_chunk;       // byte offset of this lane's chunk inside a gathered row
            bool m_ok;
        };
        auto setup = [&](const Item &it) {
            Thr t;
            t.k_base = reinterpret_cast<const char *>(p.kept_k + it.u.kk_off); // padded past k_pad
            t.a_base = reinterpret_cast<const char *>(A + it.m0);
            t.m_ok = it.m0 + chunk * 8 < it.m_end;
            t.v_chunk = t.m_ok ? chunk * 16 : 0; // beyond the row block: re-read its first chunk
            // weight chunk c = pt + bp * NPM of a step is (nb = c / 256, k16 = (c / 64) % 4,
            // lane = c % 64), i.e. 16-byte piece c % 256 of block nb; a block beyond the unit
            // reads block 0 (its products are never stored)
#pragma unroll
            for (int bp = 0; bp < BPASS; ++bp) {
                const int nb = (bp * NPM) / 256 < it.u.nb_cnt ? (bp * NPM) / 256 : 0;
                t.b_base[bp] = reinterpret_cast<const char *>(Bp + it.u.b_off) +
                               ((int64_t)(it.u.nb0 + nb) * 256 + ((bp * NPM) & 255)) * 16;
            }
            t.b_pack_b = (int64_t)it.u.nblk * (PKS * 64 * 8 * 2);
            return t;
        };
        auto load_idx = [&](const Thr &t, int s, Idx &ix) {
#pragma unroll
            for (int i = 0; i < PASSES / 4; ++i)
                ix.k[i] = *reinterpret_cast<const i32x4 *>(t.k_base + (int64_t)s * (BK * 4) + 16 * i + v_idx);
        };
        // (`live` is all ones, or zero for a refill that fetches nothing: row 0, chunk 0)
        auto load_a = [&](const Thr &t, const Idx &ix, int ps, uint32_t live, uint32_t vc) {
            const uint32_t off = ((uint32_t)ix.k[ps >> 2][ps & 3] & live) * lda_b + vc;
            return *reinterpret_cast<const u32x4 *>(t.a_base + off);
        };
        auto load_b = [&](const Thr &t, int s, int bp, uint32_t vb) {
            return *reinterpret_cast<const u32x4 *>(t.b_base[bp] + (int64_t)s * t.b_pack_b + vb);
        };
        // The item loop is rotated: an iteration first starts the loads of its item, then finishes
        // the item before it (the two barriers around the staged C tile, this half's share of the
        // stores), then runs its item's time slots.  So the first loads of an item fly over the
        // epilogue of its predecessor, and the load registers live within one iteration only
        // (carried around the loop, the compiler keeps them in two register sets and copies one
        // into the other, waiting for the loads in flight).
        Item cur = make_item(qi);
        Item nxt = cur, prev = cur;
        bool have_next = false, have_prev = false;
        for (;;) {
            u32x4 a_ring[R][PASSES];
            u32x4 b_ring[R][BPASS];
            Idx ix_ring[R]; // row indices of the steps whose loads the next R slots issue
            const Thr tc = setup(cur);
            const int nsteps = has_steps(cur) ? cur.u.k_pad / BK : 0;
            if (nsteps > 0) {
                // First loads: weight and rows of steps 0 .. R - 1, the index loads R steps ahead,
                // in the order the time slots keep up.  All register slots are loaded whether or
                // not the item has that many steps (the index list is padded, the weight step is
                // clamped), like every slot below refills its registers whether or not a step is
                // left to fetch: the sequence of loads is then the same on every path and the
                // compiler can wait for exactly the loads a slot needs.
                Idx ix[R];
#pragma unroll
                for (int r = 0; r < R; ++r)
                    load_idx(tc, r, ix[r]);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    load_idx(tc, R + r, ix_ring[r]);
#pragma unroll
                    for (int bp = 0; bp < BPASS; ++bp)
                        b_ring[r][bp] = load_b(tc, r < nsteps ? r : nsteps - 1, bp, v_b);
#pragma unroll
                    for (int ps = 0; ps < PASSES; ++ps)
                        a_ring[r][ps] = load_a(tc, ix[r], ps, 0xFFFFFFFFu, tc.v_chunk);
                }
            }
            if (have_prev) {
                if (!is_fill(prev)) {
                    TW_LDS_BARRIER(); // end of the last time slot
                    TW_LDS_BARRIER(); // the C tile is staged
                    store_tile(prev.u, prev.m0, prev.m_end);
                }
                TW_LDS_BARRIER(); // LDS may be reused now
            }
            if (is_end(cur))
                break;
            if (!has_steps(cur)) { // no step, no pipeline barrier to ride on
                nxt = claim();
                have_next = true;
            }
            if (is_fill(cur)) {
                zero_fill(cur);
            } else if (nsteps > 0) {
                const UnitDev &u = cur.u;
                // time slot j: write step j (loaded R slots ago) into stage j & 1 and reuse its
                // registers for the loads of step j + R.  Every register is written to LDS and
                // refilled by its next load back to back, so that the LDS queue and the
                // vector-memory queue are fed at the same time.  When no step j + R is left, the
                // refill reads one fixed 16-byte piece with all lanes (a single cache line per
                // load, never used): no branch, and one copy of this code serves every slot.
                const int k_left0 = u.k_kept - row0; // kept rows from this lane's first row on
                auto slot = [&](int j, int r) {
                    uint16_t *const stA = sA + (j & 1) * ASTAGE;
                    uint16_t *const stB = sB + (j & 1) * BSTAGE;
                    const bool more = j + R < nsteps;
                    const uint32_t live = more ? 0xFFFFFFFFu : 0u;
                    // the indices of step j + R were fetched R slots ago; those of step j + 2 R
                    // are fetched now (the list is padded: always in bounds)
                    const Idx ix = ix_ring[r];
                    load_idx(tc, j + 2 * R, ix_ring[r]);
                    const int sb = more ? j + R : 0;
                    const uint32_t vb = v_b & live;
#pragma unroll
                    for (int bp = 0; bp < BPASS; ++bp) {
                        *reinterpret_cast<u32x4 *>(stB + (pt + bp * NPM) * 8) = b_ring[r][bp];
                        b_ring[r][bp] = load_b(tc, sb, bp, vb);
                    }
                    const uint32_t vc = tc.v_chunk & live;
                    const int k_left = k_left0 - j * BK;
#pragma unroll
                    for (int ps = 0; ps < PASSES; ++ps) {
                        // rows beyond K_t and chunks beyond M become zeros
                        const uint32_t keep = (ps < k_left && tc.m_ok) ? 0xFFFFFFFFu : 0u;
                        u32x4 v = a_ring[r][ps];
                        v.x &= keep;
                        v.y &= keep;
                        v.z &= keep;
                        v.w &= keep;
                        *reinterpret_cast<u32x4 *>(stA + (row0 + ps) * PITCH + chunk * 8) = v;
                        a_ring[r][ps] = load_a(tc, ix, ps, live, vc);
                    }
                    TW_LDS_BARRIER();
                    if (j == 0 && !have_next) {
                        nxt = published();
                        have_next = true;
                    }
                };
                for (int j = 0; j < nsteps;) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        if (j < nsteps) {
                            slot(j, r);
                            ++j;
                        }
                    }
                }
            } // (a unit without kept rows has no step: its columns receive beta * C)
            prev = cur;
            have_prev = true;
            cur = nxt;
            have_next = false;
        }
    } else {
        // ================= multiplying waves ==============================================
        Item cur = make_item(qi);
        Item nxt = cur;
        bool have_next = false;
        int gs = 0; // (DMA) stage of the current item's step 0 is gs % NST
        while (!is_end(cur)) {
            if (!has_steps(cur)) {
                nxt = claim();
                have_next = true;
            }
            if (is_fill(cur)) {
                zero_fill(cur);
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
                const bool w_active = m0 + wave * RW < cur.m_end;
                // output columns of this lane's compact columns and their bias: fetched now, used
                // in the epilogue (the wait for the first staged step covers their round trips)
                const int32_t *const nlist = p.kept_n + u.kn_off;
                int out_col[NI];
                float out_bias[NI];
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const int j = ni * 32 + (lane & 31);
                    out_col[ni] = u.col0 + nlist[j < u.n_cnt ? j : 0];
                }
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
                    out_bias[ni] = p.bias ? p.bias[out_col[ni]] : 0.0f;
                auto frags = [&](int s, int ks, u32x4(&af)[MI], u32x4(&bf)[NI]) {
                    const uint16_t *const stA = DMA ? sA + ((gs + s) % NST) * STG : sA + (s & 1) * ASTAGE;
                    const uint16_t *const stB = DMA ? sB + ((gs + s) % NST) * STG : sB + (s & 1) * BSTAGE;
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi) {
                        // ds_read_b64_tr_b16: 16 lanes read a 4(k) x 16(m) block; lane L addresses
                        // row L/4, columns 4*(L%4)..+3 and receives column L of the 4 rows.
                        const int L = lane & 15;
                        const int row = ks * 16 + (lane >> 5) * 8 + (L >> 2);
                        const int col = wave * RW + mi * 32 + ((lane >> 4) & 1) * 16 + (L & 3) * 4;
                        // (DMA: row (ks, lane >> 5, L >> 2) is half lane >> 5 of slot ks * 8 + (L >> 2))
                        constexpr int RSTEP = DMA ? SLOTB / 2 : PITCH; // from row r to row r + 1 of a group of eight
                        const uint16_t *q = DMA ? stA + (ks * 8 + (L >> 2)) * (SLOTB / 2) + (lane >> 5) * BM + col
                                                : stA + row * PITCH + col;
                        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))q);
                        s16x4 hi =
                            __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(q + 4 * RSTEP));
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
                        // Instruction order of the step, pinned: the operands of the first 16 k
                        // rows, then every MFMA of 16 k rows followed by its share of the LDS reads
                        // for the next 16.  (Left alone, the scheduler reads one operand at a time
                        // into the same registers and waits for each before the two MFMAs that
                        // use it: the LDS latency then shows 16 times per step.)
                        constexpr int NRD = 2 * MI + NI, NMM = MI * NI;
                        __builtin_amdgcn_sched_group_barrier(0x100, NRD, 0);
#pragma unroll
                        for (int ks = 0; ks + 1 < KS; ++ks)
                            sched_mfma_with_reads<NRD, NMM, 0, true>();
                        sched_mfma_with_reads<NRD, NMM, 0, false>();
                    }
                    TW_LDS_BARRIER();
                }

                // epilogue: alpha/beta in fp32, round, hand the tile over through LDS
                float scale = p.alpha;
                const bool fused = (p.bias || p.act) && p.beta == 0.0f;
                if (p.beta != 0.0f) {
                    // rare path: fold alpha, beta*C, the bias and the activation into the
                    // accumulators first (C is read on kept columns only)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int j = ni * 32 + (lane & 31);
                        const int col = out_col[ni];
                        const int64_t coff = (int64_t)col * p.ldc;
#pragma unroll
                        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int m = m0 + wave * RW + mi * 32 + (lane >> 5) * 4 + (r >> 2) * 8 + (r & 3);
                                float old = 0.0f;
                                if (p.beta != 0.0f && j < u.n_cnt && m < cur.m_end)
                                    old = E::from_bits(C[coff + m]);
                                acc[mi][ni][r] = tw_activate(
                                    p.alpha * acc[mi][ni][r] + p.beta * old + out_bias[ni], p.act);
                            }
                    }
                    scale = 1.0f;
                }
                // The C tile goes through LDS in CROUNDS rounds of RNI blocks of 32 columns: all of
                // it at once into the pipeline's stages, or (DMA) 64 columns at a time into the
                // stage of the item's last step.
                constexpr int RNI = NI / CROUNDS;
                uint16_t *const ctile = DMA ? smem + ((nsteps > 0 ? gs + nsteps - 1 : gs) % NST) * STG : smem;
                auto stage_round = [&](auto round_tag) {
                    constexpr int RD = decltype(round_tag)::value;
                    if (fused) {
                        // bias and activation in fp32, one rounding; the activation is a
                        // compile-time constant of each copy
                        auto stage_fused = [&](auto act_tag) {
                            constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
                            for (int ni = RD * RNI; ni < (RD + 1) * RNI; ++ni) {
                                const int j = (ni - RD * RNI) * 32 + (lane & 31);
                                const float bj = out_bias[ni];
#pragma unroll
                                for (int mi = 0; mi < MI; ++mi) {
                                    const int mloc = wave * RW + mi * 32 + (lane >> 5) * 4;
#pragma unroll
                                    for (int r4 = 0; r4 < 4; ++r4) {
                                        float v[4];
#pragma unroll
                                        for (int e = 0; e < 4; ++e)
                                            v[e] = tw_fp32_value(tw_activate(scale * acc[mi][ni][r4 * 4 + e] + bj, ACT));
                                        u32x2 pk;
                                        pk.x = E::to_bits(v[0]) | (E::to_bits(v[1]) << 16);
                                        pk.y = E::to_bits(v[2]) | (E::to_bits(v[3]) << 16);
                                        *reinterpret_cast<u32x2 *>(ctile + j * CPITCH + mloc + r4 * 8) = pk;
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
                        for (int ni = RD * RNI; ni < (RD + 1) * RNI; ++ni) {
                            const int j = (ni - RD * RNI) * 32 + (lane & 31); // compact column inside the round
#pragma unroll
                            for (int mi = 0; mi < MI; ++mi) {
                                const int mloc = wave * RW + mi * 32 + (lane >> 5) * 4;
#pragma unroll
                                for (int r4 = 0; r4 < 4; ++r4) {
                                    u32x2 pk;
                                    pk.x = E::to_bits(scale * acc[mi][ni][r4 * 4 + 0]) |
                                           (E::to_bits(scale * acc[mi][ni][r4 * 4 + 1]) << 16);
                                    pk.y = E::to_bits(scale * acc[mi][ni][r4 * 4 + 2]) |
                                           (E::to_bits(scale * acc[mi][ni][r4 * 4 + 3]) << 16);
                                    *reinterpret_cast<u32x2 *>(ctile + j * CPITCH + mloc + r4 * 8) = pk;
                                }
                            }
                        }
                    }
                };
                stage_round(std::integral_constant<int, 0>());
                if (wave == 0 && lane < 32) {
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni)
                        s_cols[ni * 32 + lane] = out_col[ni];
                }
                pick_up();
                if (tid == 0 && announced)
                    asm volatile("" : "+v"(t_done)); // the count has returned: read it before the stores
                TW_LDS_BARRIER(); // the C tile (its first round) is staged
                if constexpr (!DMA) {
                    store_tile(u, m0, cur.m_end);
                } else {
                    // (the moving waves help unless they are loading the next item already)
                    const bool chained = nsteps >= 2 && has_steps(nxt);
                    const bool all_store = !chained;
                    const bool deferred = chained && defer_stores(cur, nxt);
                    if (!deferred)
                        store_round(ctile, 0, u, m0, cur.m_end, all_store);
                    TW_LDS_BARRIER(); // stored (or taken by the moving waves): the stage may be written again
                    if constexpr (CROUNDS > 1) {
                        stage_round(std::integral_constant<int, CROUNDS - 1>());
                        TW_LDS_BARRIER(); // staged
                        if (!deferred)
                            store_round(ctile, 1, u, m0, cur.m_end, all_store);
                        TW_LDS_BARRIER(); // stored
                    }
                    static_assert(CROUNDS <= 2, "two rounds at most");
                    gs += nsteps;
                }
            }
            TW_LDS_BARRIER(); // LDS may be reused now
            cur = nxt;
            have_next = false;
        }
        // the workgroup counted last re-arms the ticket slot for the next launch: every
        // workgroup's claims had returned before it was counted.  Plain stores, made visible by
        // the end of the kernel; a device-scope fence here would write back and invalidate this
        // XCD's L2 under the workgroups that still stream through it.
        if (tid == 0 && t_done == (int)gridDim.x - 1) {
#pragma unroll
            for (int i = 0; i <= kXcd; ++i)
                p.ticket[i] = 0;
        }
    }
}

// ---------------------------------------------------------------------------------
// A-stationary kernel for a short K: a workgroup keeps a panel of A - every row k, BMS rows m -
// in LDS for its whole life and walks over its share of the plan with it.  The streaming kernels
// above pay a start-up chain (unit -> indices -> rows) and an epilogue per item, and with a
// short K an item is little else (BERT-base: three steps); here A is read once per workgroup
// with plain contiguous loads, the gather of a tile's kept rows happens inside LDS (a transposed
// read takes a row address per lane), the packed weight goes from memory straight into the MFMA
// operand registers of the one wave that uses it, and the waves never meet again after the
// panel is loaded: each wave takes blocks of 32 compact columns, multiplies BMS x 32, turns its
// product through its own piece of LDS and stores it.
//   panel: row k at k * 2 * BMS bytes; for BMS = 64 the two 64-byte halves of a row are swapped
//          in rows with bit 1 set, so that the four rows a transposed read touches (consecutive
//          kept rows are mostly a few rows apart) tend to fall into different bank groups
//   work:  block b of the plan (unit, 32-column block) belongs to group b % n_groups; workgroup
//          (row block, group); wave w takes every twelfth block of the group
//   loads: a block is cut into segments of two steps (8 groups of 16 k rows: per lane a 16-byte
//          weight fragment and a word with its two row numbers each).  A wave computes one
//          segment out of one register set while the loads of the next segment - of this block
//          or the next - fill the other.  Every segment issues the loads of all its 8 groups
//          (steps past the block's end fetch its last step again), so the number of loads in
//          flight behind a segment is the same on every path and the wait for it is an exact
//          count.
// Takes beta == 0 only (C is not read).  RM false: K-major A and C (32-bit row offsets into A).
// RM true: row-major A[M][lda] and C[M][ldc], the operands of the reference's Python operator
// (mask_dense, Pruning/BERT/utils/modeling.py:992-1007): the panel is transposed on its way into
// LDS (pieces of 16 rows m x 64 k, read along k and turned with the transposed LDS read), and
// the product goes out as 16-byte pieces of rows of C where a block's kept columns are
// neighbours in C in aligned groups of eight, else as 2-byte stores, a wave covering two rows
// of the block's 32 columns.
// Waves of a workgroup, steps of a segment, and waves that share a block of a 64-row panel (each
// then multiplies one 32-row half of it).  A wave's life is a chain of short dependent phases
// (loads, LDS reads, MFMAs, stage, stores), so more waves fill each other's gaps: twelve waves
// with two-step segments (157 registers of the 170 a wave may then have) run BERT-base in 14.2
// us, eight waves with four-step segments in 15.7; sixteen waves leave 128 registers, which
// only a 32-row product with one-step segments fits, and two such waves sharing a block of a
// 64-row panel load its weight fragments twice: 16.7 us.
constexpr int as_waves(int bms, bool rm) { return 12; }
constexpr int as_seg_steps(int bms, bool rm) { return 2; }
constexpr int as_split(int bms, bool rm) { return 1; }
constexpr int as_task_waves(int bms, bool rm) { return as_waves(bms, rm) / as_split(bms, rm); }

template <int DT, int BMS, bool RM>
__global__ void __launch_bounds__(64 * as_waves(BMS, RM), 1)
    tw_gemm_as_kernel(const GemmArgs p, const int32_t *__restrict__ blocks, int n_blocks, int n_groups,
                      int n_mblk, int k_rows, int blocks_per_unit)
{
    constexpr int kAsWaves = as_waves(BMS, RM), SPLIT = as_split(BMS, RM), TWV = kAsWaves / SPLIT;
    constexpr int NT = 64 * kAsWaves;
    constexpr int ROWB = BMS * 2; // bytes of a panel row
    constexpr int CH = BMS / 8;   // 16-byte chunks of a panel row
    constexpr int MI = BMS / 32 / SPLIT; // 32-row MFMA blocks of a wave
    constexpr int CP = 32 + 4;    // pitch of a wave's C stage: [32 columns][CP] elements, 32 rows at a time
    constexpr int DS = as_seg_steps(BMS, RM), GS = DS * 4;
    using E = Elem<DT>;
    extern __shared__ __align__(16) unsigned char as_smem[];
    unsigned char *const panel = as_smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int task = wave / SPLIT;           // which of the workgroup's block sequences
    const int mi0 = (wave % SPLIT) * MI;     // first 32-row block of the panel this wave multiplies
    const int mblk = blockIdx.x % n_mblk, group = blockIdx.x / n_mblk;
    const int m0 = mblk * BMS;
    const int m_end = m0 + BMS < p.M ? m0 + BMS : p.M;
    const uint16_t *const A = reinterpret_cast<const uint16_t *>(p.A);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    const unsigned char *const Bp = reinterpret_cast<const unsigned char *>(p.Bp);
    uint16_t *const cst = reinterpret_cast<uint16_t *>(as_smem + (size_t)(k_rows + 1) * ROWB) + wave * 32 * CP;

    const int L = lane & 15;
    // ---- the panel: 16-byte chunks, sixteen loads in flight per thread (the first segment's
    // loads of this wave are already on their way, see below)
    // Row-major A: a wave takes pieces of 16 rows m x 64 columns k.  It reads a piece with
    // 16-byte loads along k (eight lanes a row: whole 128-byte lines), puts it into its own stage
    // as it came, [m][k], and takes it out again with transposed reads: by the symmetry of that
    // instruction a lane then holds eight neighbouring m of one k, one 16-byte piece of a panel row.
    auto load_panel_row_major = [&]() {
        constexpr int MB = BMS / 16;  // pieces across the rows of the panel
        constexpr int TP = 144;       // bytes of a row of the piece in the stage (16 rows: the whole stage)
        static_assert(16 * TP <= 32 * CP * 2, "a piece has to fit the wave's stage");
        const int kchunks = (k_rows + 7) / 8;
        const int n_pieces = MB * ((k_rows + 63) / 64);
        unsigned char *const tmp = reinterpret_cast<unsigned char *>(cst);
        const int lrow = lane >> 3, lkc = lane & 7; // as a reader of A: row of the piece (and + 8), 16-byte chunk
        const int gq = lane >> 4;                   // as a writer of the panel: k = 16 gq + L of the piece
        TW_LDS(unsigned char) const tr_lane = (TW_LDS(unsigned char))tmp + (L >> 2) * TP + (gq * 16 + (L & 3) * 4) * 2;
        constexpr int PP = 4; // pieces in flight per wave
        for (int c0 = wave; c0 < n_pieces; c0 += kAsWaves * PP) {
            u32x4 v[PP][2];
#pragma unroll
            for (int q = 0; q < PP; ++q) {
                const int c = c0 + q * kAsWaves;
                const int mb = c % MB, kb = c / MB;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int m = m0 + mb * 16 + h * 8 + lrow, kc = kb * 8 + lkc;
                    v[q][h] = u32x4{0u, 0u, 0u, 0u};
                    if (c < n_pieces && m < p.M && kc < kchunks)
                        v[q][h] = *reinterpret_cast<const u32x4 *>(A + (int64_t)m * p.lda + kc * 8);
                }
            }
#pragma unroll
            for (int q = 0; q < PP; ++q) {
                const int c = c0 + q * kAsWaves;
                if (c < n_pieces) {
                    const int mb = c % MB, kb = c / MB;
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        *reinterpret_cast<u32x4 *>(tmp + (h * 8 + lrow) * TP + lkc * 16) = v[q][h];
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    const int k = kb * 64 + gq * 16 + L;
#pragma unroll
                    for (int cc = 0; cc < 2; ++cc) {
                        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(tr_lane + cc * 8 * TP));
                        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(tr_lane + (cc * 8 + 4) * TP));
                        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                        const int mch = mb * 2 + cc;
                        const int chs = BMS == 64 ? mch ^ (((k >> 1) & 1) << 2) : mch;
                        if (k < k_rows)
                            *reinterpret_cast<u32x4 *>(panel + k * ROWB + chs * 16) = u32x4{l2.x, l2.y, h2.x, h2.y};
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the stage is free for the next piece
                }
            }
        }
    };
    constexpr int PL = 128 / kAsWaves; // loads in flight per thread: 128 per SIMD lane of the unit
    const int panel_chunks = k_rows * CH;
    auto panel_fetch = [&](int base, u32x4 (&v)[PL]) {
        const uint32_t lda_b = (uint32_t)p.lda * 2u;
        const char *const a0 = reinterpret_cast<const char *>(A + m0);
#pragma unroll
        for (int q = 0; q < PL; ++q) {
            const int idx = base + q * NT;
            const int row = idx / CH, ch = idx % CH;
            v[q] = u32x4{0u, 0u, 0u, 0u};
            if (idx < panel_chunks && m0 + ch * 8 < p.M)
                v[q] = *reinterpret_cast<const u32x4 *>(a0 + (uint32_t)row * lda_b + ch * 16);
        }
    };
    auto panel_put = [&](int base, const u32x4 (&v)[PL]) {
#pragma unroll
        for (int q = 0; q < PL; ++q) {
            const int idx = base + q * NT;
            const int row = idx / CH, ch = idx % CH;
            const int chs = BMS == 64 ? ch ^ (((row >> 1) & 1) << 2) : ch;
            if (idx < panel_chunks)
                *reinterpret_cast<u32x4 *>(panel + row * ROWB + chs * 16) = v[q];
        }
    };

    // ---- this wave's blocks, segment by segment
    const int pair_e = (lane >> 5) * 4 + (L >> 2);            // this lane's word of a group's row pairs
    const int lane_b = ((lane >> 4) & 1) * 32 + (L & 3) * 8;  // its byte offset inside a 64-byte half row
    const int j = lane & 31;                                  // its compact column inside a block

    struct Cursor {    // one segment of one block; wave-uniform
        int b;         // block index in the plan's list, n_blocks or more: past the end
        int seg;       // segment of the block
        int nsteps;    // steps of the block
        int nb;        // 32-column block inside the unit
        int code_after; // list entry of the wave's block after this one, fetched a block ahead
        UnitDev u;
    };
    const int b_stride = n_groups * TWV;
    // entry b of the plan's list of blocks, unit * 4 + block of the unit: worked out where every
    // unit has the same number of blocks (no trip to memory before the first loads), else the
    // value fetched a block ahead
    auto block_code = [&](int b, int fetched) {
        if (blocks_per_unit) {
            const int ui = b / blocks_per_unit;
            return ui * 4 + (b - ui * blocks_per_unit);
        }
        return __builtin_amdgcn_readfirstlane(fetched);
    };
    auto open_block = [&](int b, int code) {
        Cursor c;
        c.b = b;
        c.seg = 0;
        c.nsteps = 0;
        c.nb = 0;
        c.code_after = 0;
        if (b < n_blocks) {
            if (!blocks_per_unit)
                c.code_after = blocks[b + b_stride < n_blocks ? b + b_stride : b];
            c.u = load_unit(p, code >> 2);
            c.nb = code & 3;
            c.nsteps = c.u.k_pad / kBlockK;
        }
        return c;
    };
    auto valid = [&](const Cursor &c) { return c.b < n_blocks; };
    auto last_segment = [&](const Cursor &c) { return (c.seg + 1) * DS >= c.nsteps; };
    auto advance = [&](const Cursor &c) {
        if (!last_segment(c)) {
            Cursor n = c;
            n.seg = c.seg + 1;
            return n;
        }
        return open_block(c.b + b_stride, block_code(c.b + b_stride, c.code_after));
    };
    struct Seg {
        u32x4 bq[GS];
        u32x4 rows[DS]; // per step: the two rows this lane addresses in each of its four groups, 16 bits each
        int out_n;      // this lane's compact column of the block as a column of the tile
    };
    // all loads of a segment (a block without steps has only its column numbers)
    auto issue = [&](const Cursor &c, Seg &g) {
        g.out_n = p.kept_n[c.u.kn_off + c.nb * 32 + (j < c.u.n_cnt - c.nb * 32 ? j : 0)];
        if (c.nsteps == 0)
            return;
        const uint32_t *const klist = p.kept_pairs + (c.u.kk_off >> 1) + pair_e * 4;
        const unsigned char *const bsrc = Bp + c.u.b_off * 2 + (int64_t)(c.u.nb0 + c.nb) * 4096 + lane * 16;
        const int64_t step_b = (int64_t)c.u.nblk * 4096;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int s = c.seg * DS + ds < c.nsteps ? c.seg * DS + ds : c.nsteps - 1;
            g.rows[ds] = *reinterpret_cast<const u32x4 *>(klist + s * (kBlockK / 2));
#pragma unroll
            for (int k16 = 0; k16 < 4; ++k16)
                g.bq[ds * 4 + k16] = *reinterpret_cast<const u32x4 *>(bsrc + s * step_b + k16 * 1024);
        }
    };
    f32x16 acc[MI];
    auto clear = [&]() {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[mi][r] = 0.0f;
    };
    float out_bias = 0.0f; // bias of this lane's column of the block being computed
    int out_col = 0;
    auto compute = [&](const Cursor &c, const Seg &g) {
        const int steps = min(DS, c.nsteps - c.seg * DS);
        if (last_segment(c)) { // the column numbers have landed with the segment: the bias follows
            out_col = c.u.col0 + g.out_n;
            out_bias = p.bias ? p.bias[out_col] : 0.0f;
        }
        TW_LDS(unsigned char) lds_lane = (TW_LDS(unsigned char))panel + lane_b;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            if (ds < steps) {
#pragma unroll
                for (int k16 = 0; k16 < 4; ++k16) {
                    const uint32_t r_lo = g.rows[ds][k16] & 0xFFFFu, r_hi = g.rows[ds][k16] >> 16;
                    // row r at r * ROWB; for BMS = 64 its halves are swapped when bit 1 of r is set
                    const uint32_t o_lo = r_lo * ROWB + (BMS == 64 ? (r_lo & 2u) << 5 : 0u);
                    const uint32_t o_hi = r_hi * ROWB + (BMS == 64 ? (r_hi & 2u) << 5 : 0u);
#pragma unroll
                    for (int mi = 0; mi < MI; ++mi) {
                        TW_LDS(unsigned char) qlo = lds_lane + (o_lo ^ (uint32_t)((mi0 + mi) * 64));
                        TW_LDS(unsigned char) qhi = lds_lane + (o_hi ^ (uint32_t)((mi0 + mi) * 64));
                        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))qlo);
                        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))qhi);
                        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                        acc[mi] = E::mfma(u32x4{l2.x, l2.y, h2.x, h2.y}, g.bq[ds * 4 + k16], acc[mi]);
                    }
                }
            }
        }
    };
    // after a block's last segment: alpha, bias, activation, one rounding; 32 rows at a time
    // through this wave's stage; 16-byte stores
    auto finish = [&](const Cursor &c) {
        if (!last_segment(c))
            return;
        const int cnt = min(32, c.u.n_cnt - c.nb * 32);
        if (RM) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                float v[16];
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    v[r] = p.alpha * acc[mi][r] + out_bias;
                tw_activate_all(v, p.act);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[mi][r] = tw_fp32_value(v[r]);
            }
            // Where the block's compact columns are neighbours in C in aligned groups of eight
            // (no column of the tile pruned, or whole groups), the product is turned through
            // the wave's stage, [row][column], and leaves as 16-byte pieces of rows of C.
            const int prev_col = __shfl_up(out_col, 1);
            const bool octets = cnt % 8 == 0 &&
                                __all(j >= cnt || ((j & 7) ? out_col == prev_col + 1 : (out_col & 7) == 0));
            if (octets) {
                const int r = lane >> 2, ch = lane & 3;
                const int col = __shfl(out_col, ch * 8);
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        uint16_t *const dst = cst + ((lane >> 5) * 4 + r4 * 8) * CP + j;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            dst[e * CP] = (uint16_t)E::to_bits(acc[mi][r4 * 4 + e]);
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const int row = r + q * 16;
                        const u32x2 lo = *reinterpret_cast<const u32x2 *>(cst + row * CP + ch * 8);
                        const u32x2 hi = *reinterpret_cast<const u32x2 *>(cst + row * CP + ch * 8 + 4);
                        const int m = m0 + (mi0 + mi) * 32 + row;
                        if (ch * 8 < cnt && m < m_end)
                            *reinterpret_cast<u32x4 *>(C + (int64_t)m * p.ldc + col) = u32x4{lo.x, lo.y, hi.x, hi.y};
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the stage is free again
                }
                clear();
                return;
            }
            // rows m_lane + 8 * g + e, g = 0 .. 4 MI - 1, e = 0 .. 3: a running pointer, so that
            // the 16 MI addresses are not all worked out (and kept in registers) ahead
            const int m_lane = m0 + mi0 * 32 + (lane >> 5) * 4;
            uint16_t *cp = C + (int64_t)m_lane * p.ldc + out_col;
#pragma unroll
            for (int g = 0; g < 4 * MI; ++g) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint16_t h = (uint16_t)E::to_bits(acc[g >> 2][(g & 3) * 4 + e]);
                    if (j < cnt && m_lane + g * 8 + e < m_end)
                        cp[(int64_t)e * p.ldc] = h;
                }
                cp += 8 * p.ldc;
                asm volatile("" : "+v"(cp));
            }
            clear();
            return;
        }
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const int mloc = (lane >> 5) * 4;
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; ++r)
                v[r] = p.alpha * acc[mi][r] + out_bias;
            tw_activate_all(v, p.act); // the test of the activation outside the loop over the elements
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                uint32_t h[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    h[e] = E::to_bits(tw_fp32_value(v[r4 * 4 + e]));
                u32x2 pk;
                pk.x = h[0] | (h[1] << 16);
                pk.y = h[2] | (h[3] << 16);
                *reinterpret_cast<u32x2 *>(cst + j * CP + mloc + r4 * 8) = pk;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int q = 0; q < 2; ++q) { // 32 columns x 4 chunks of 8 rows
                const int idx = lane + q * 64;
                const int jj = idx >> 2, ch = idx & 3;
                const int col = __shfl(out_col, jj);
                const u32x2 lo = *reinterpret_cast<const u32x2 *>(cst + jj * CP + ch * 8);
                const u32x2 hi = *reinterpret_cast<const u32x2 *>(cst + jj * CP + ch * 8 + 4);
                const int m = m0 + (mi0 + mi) * 32 + ch * 8;
                if (jj < cnt)
                    store_chunk(C + (int64_t)col * p.ldc + m, u32x4{lo.x, lo.y, hi.x, hi.y}, m, m_end,
                                p.store_through != 0);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the stage is free again
        }
        clear();
    };

    clear();
    Seg g0, g1;
    const int b_first = group + n_groups * task;
    Cursor cur_first;
    if (RM) {
        Cursor first = open_block(b_first, b_first < n_blocks ? block_code(b_first, blocks_per_unit ? 0 : blocks[b_first]) : 0);
        if (valid(first))
            issue(first, g0); // weight and row numbers do not wait for the panel
        load_panel_row_major();
        cur_first = first;
    } else {
        // the panel's first loads leave before anything else is known: the unit of the wave's
        // first block and that block's loads follow them while they are on their way
        u32x4 pv[PL];
        panel_fetch(tid, pv);
        Cursor first = open_block(b_first, b_first < n_blocks ? block_code(b_first, blocks_per_unit ? 0 : blocks[b_first]) : 0);
        if (valid(first))
            issue(first, g0);
        panel_put(tid, pv);
        for (int base = tid + NT * PL; base < panel_chunks; base += NT * PL) {
            panel_fetch(base, pv);
            panel_put(base, pv);
        }
        cur_first = first;
    }
    Cursor cur = cur_first;
    // the row of zeros behind the panel: the padding of every list of kept rows points at it
    if (tid < CH)
        *reinterpret_cast<u32x4 *>(panel + (size_t)k_rows * ROWB + tid * 16) = u32x4{0u, 0u, 0u, 0u};
    __syncthreads();
    if (valid(cur)) {
        for (;;) {
            Cursor nxt = advance(cur);
            if (valid(nxt))
                issue(nxt, g1);
            compute(cur, g0);
            finish(cur);
            if (!valid(nxt))
                break;
            cur = advance(nxt);
            if (valid(cur))
                issue(cur, g0);
            compute(nxt, g1);
            finish(nxt);
            if (!valid(cur))
                break;
        }
    }

    // ---- TW_PRUNED_ZERO: the pruned columns of this group's tiles receive act(bias)
    for (int z = p.n_gemm_u + group; z < p.n_all_u; z += n_groups) {
        const TileDev t = p.tiles[z - p.n_gemm_u];
        if (RM) {
            for (int i = tid; i < t.n_pruned * BMS; i += NT) {
                const int m = m0 + i / t.n_pruned;
                const int c = t.col0 + p.pruned_n[t.pn_off + i % t.n_pruned];
                if (m < m_end)
                    C[(int64_t)m * p.ldc + c] = (uint16_t)E::to_bits(tw_finish(0.0f, p.bias, c, p.act));
            }
            continue;
        }
        for (int i = tid; i < t.n_pruned * CH; i += NT) {
            const int jz = i / CH, ch = i % CH;
            const int c = t.col0 + p.pruned_n[t.pn_off + jz];
            const uint32_t hb = E::to_bits(tw_finish(0.0f, p.bias, c, p.act));
            const uint32_t w = hb | (hb << 16);
            store_chunk(C + (int64_t)c * p.ldc + m0 + ch * 8, u32x4{w, w, w, w}, m0 + ch * 8, m_end,
                        p.store_through != 0);
        }
    }
}

// ---------------------------------------------------------------------------------
// Skinny kernel for a handful of rows of A (one time step of a recurrent cell: M = 128): the
// launch is then a chain of dependent trips to memory on an almost empty chip, and the streaming
// kernels walk a tile's kept rows 64 at a time, one trip per step.  Here a workgroup takes
// 32 rows m of one half of a unit (up to 64 compact columns) and its four waves split the kept
// rows between them: wave w takes the steps w, w + 4, ... of 64 kept rows, two at a time: it
// fetches their row numbers, then their 8 KB of A and 16 KB of weight fragments in one go, turns
// A through its own piece of LDS (no barrier: nobody else reads it) and multiplies.  The four
// partial products meet in LDS once, are added in wave order (so the result does not depend on
// timing) and leave through one rounding.  A tile of 512 kept rows is one trip to memory for the
// numbers and one for the operands.
//   work:  workgroup (x, y): die x % 8, unit (x / 16) * 8 + die, half (x / 8) % 2, row block y
//          (a plan without units wider than 64 columns is launched without second halves);
//          the unit comes from the kernel arguments at an offset that depends on the workgroup
//          number alone, so that it arrives with the other arguments; the halves and row blocks
//          of a unit sit on one die and share its rows of A in that L2; workgroups of a half the
//          unit does not have fill pruned columns (TW_PRUNED_ZERO) or leave
//   stage: per wave 2 x 64 rows k of 32 rows m (64 bytes each), then reused for the wave's
//          partial product [64 columns][32 + 4 rows m] in fp32
// K-major A and C; any beta.  The sum over k runs in four slices, so the result can differ from
// the streaming kernels' in the last bit of fp32 before the rounding to 16 bits.
constexpr int kSkWaves = 4;
constexpr int kSkRows = 32;                            // rows m of a workgroup
constexpr int kSkCols = 64;                            // compact columns of a workgroup
constexpr int kSkPitch = kSkRows + 4;                  // floats per column of a partial product
constexpr int kSkStage = kSkCols * kSkPitch * 4;       // 9216 bytes >= 2 * 64 * 64
constexpr int kSkLdsBytes = kSkWaves * kSkStage;

template <int DT>
__global__ void __launch_bounds__(64 * kSkWaves, 1) tw_gemm_skinny_kernel(const GemmArgs p, int n_units, int halves)
{
    constexpr int NT = 64 * kSkWaves;
    using E = Elem<DT>;
    __shared__ __align__(16) unsigned char sk_smem[kSkLdsBytes];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int die = blockIdx.x % kXcd, rest = blockIdx.x / kXcd;
    // (halves: 2, or 1 for a plan whose units all have at most 64 compact columns)
    const int half = halves == 2 ? rest & 1 : 0, ui = (halves == 2 ? rest >> 1 : rest) * kXcd + die;
    // the arguments the first loads need, asked for together with the unit
    // (as integers: a pointer that has been through an asm statement is no longer known to
    // point to global memory)
    uintptr_t A_i = (uintptr_t)p.A, kk_i = (uintptr_t)p.kept_k, kn_i = (uintptr_t)p.kept_n, Bp_i = (uintptr_t)p.Bp;
    int64_t lda = p.lda, ldc = p.ldc;
    int M = p.M;
    const bool in_range = ui < n_units;
    const int m0 = blockIdx.y * kSkRows;
    // the unit: asked for from the kernel arguments before anything else has arrived
    UnitDev u;
    {
        const auto *ka = (const __attribute__((address_space(4))) int32_t *)__builtin_amdgcn_kernarg_segment_ptr();
        const int ua = ui < kMaxArgUnits ? ui : 0;
        int32_t w[12];
#pragma unroll
        for (int i = 0; i < 12; ++i)
            w[i] = ka[offsetof(GemmArgs, arg_units) / 4 + ua * 12 + i];
        const int n_arg_units = p.n_arg_units;
#pragma unroll
        for (int i = 0; i < 12; ++i)
            asm volatile("" : "+s"(w[i])); // asked for here, not behind the test below
        asm volatile("" : "+s"(A_i), "+s"(kk_i), "+s"(kn_i), "+s"(Bp_i), "+s"(lda), "+s"(ldc), "+s"(M));
        if (!n_arg_units) {
            const auto *gu = (const __attribute__((address_space(4))) int32_t *)(uintptr_t)(p.units + (in_range ? ui : 0));
#pragma unroll
            for (int i = 0; i < 12; ++i)
                w[i] = gu[i];
        }
#pragma unroll
        for (int i = 0; i < 12; ++i)
            w[i] = __builtin_amdgcn_readfirstlane(w[i]);
        __builtin_memcpy(&u, w, sizeof(UnitDev));
    }
    const int m_end = m0 + kSkRows < M ? m0 + kSkRows : M;
    TW_GLOBAL(const uint16_t) const A = (TW_GLOBAL(const uint16_t))A_i;
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);
    TW_GLOBAL(const int32_t) const kept_k = (TW_GLOBAL(const int32_t))kk_i;
    TW_GLOBAL(const int32_t) const kept_n = (TW_GLOBAL(const int32_t))kn_i;
    TW_GLOBAL(const unsigned char) const Bp = (TW_GLOBAL(const unsigned char))Bp_i;

    if (in_range && half * 2 < u.nb_cnt) {
        const int nsteps = u.k_pad / kBlockK;
        const bool two_blocks = half * 2 + 1 < u.nb_cnt;
        unsigned char *const stage = sk_smem + wave * kSkStage;
        // the reducing role of this lane: column jj of the half, rows m8 .. m8 + 7
        const int jj = wave * 16 + (lane >> 2), m8 = (lane & 3) * 8;
        const int cnt = min(kSkCols, u.n_cnt - half * kSkCols);

        struct Numbers {
            int row[2][4]; // rows of A this lane fetches a chunk of: kept row i * 16 + lane / 4 of step t
        };
        struct Loads {
            u32x4 a[2][4], b[2][2][4];
        };
        TW_GLOBAL(const unsigned char) const bsrc = Bp + u.b_off * 2 +
                                          (int64_t)(u.nb0 + half * 2) * 4096 + lane * 16;
        const int64_t step_b = (int64_t)u.nblk * 4096;
        const int ch = lane & 3, row16 = lane >> 2;
        // Nothing on the way to the operands is conditional, so that the waits between the loads
        // are exact counts: a chunk of rows past M is fetched from the row block's first chunk
        // instead (those rows of the product are never stored), a second step past the end and a
        // second block the half does not have repeat the first (and are not multiplied, or not
        // stored).
        TW_GLOBAL(const uint16_t) const a_lane = A + m0 + (m0 + ch * 8 < M ? ch * 8 : 0);
        const int cb_off = two_blocks ? 4096 : 0;
        // a pair of steps: s and s + kSkWaves (the second may be past the end)
        auto numbers = [&](int s) {
            Numbers n;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int st = s + t * kSkWaves < nsteps ? s + t * kSkWaves : s;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    n.row[t][i] = kept_k[u.kk_off + st * kBlockK + i * 16 + row16];
            }
            return n;
        };
        // (the weight fragments first: they do not wait for the row numbers, so on a wave's
        // first pair they travel while the numbers are still on their way)
        auto issue = [&](int s, const Numbers &n, Loads &l) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int st = s + t * kSkWaves < nsteps ? s + t * kSkWaves : s;
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                    for (int k16 = 0; k16 < 4; ++k16)
                        l.b[t][cb][k16] =
                            *(TW_GLOBAL(const u32x4))(bsrc + st * step_b + cb * cb_off + k16 * 1024);
            }
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    l.a[t][i] = *(TW_GLOBAL(const u32x4))(a_lane + (int64_t)n.row[t][i] * lda);
        };
        f32x16 acc[2];
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[cb][r] = 0.0f;
        const int L = lane & 15;
        const int pair_e = (lane >> 5) * 4 + (L >> 2);
        const int lane_b = ((lane >> 4) & 1) * 32 + (L & 3) * 8;
        const uint32_t r_first = (uint32_t)((pair_e >> 2) * 8 + (pair_e & 3));

        // the steps of the pair at s out of one register set: A through the stage, the products
        // (the tile's list of kept rows is padded to whole steps with row 0: what was fetched for
        // the padding is replaced by zeros here, so that no value of a row the tile does not keep,
        // finite or not, ever reaches a product)
        const int k_lim = u.k_kept - row16;
        auto multiply = [&](int s, const Loads &l) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int k0 = (s + t * kSkWaves) * kBlockK;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t keep = k0 + i * 16 < k_lim ? 0xFFFFFFFFu : 0u;
                    const u32x4 v = l.a[t][i];
                    *reinterpret_cast<u32x4 *>(stage + (t * 64 + i * 16 + row16) * 64 + ch * 16) =
                        u32x4{v.x & keep, v.y & keep, v.z & keep, v.w & keep};
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the rows are in the stage
            TW_LDS(unsigned char) lds_lane = (TW_LDS(unsigned char))stage + lane_b;
#pragma unroll
            for (int t = 0; t < 2; ++t)
                if (s + t * kSkWaves < nsteps) {
#pragma unroll
                    for (int k16 = 0; k16 < 4; ++k16) {
                        const uint32_t r_lo = t * 64 + r_first + k16 * 16, r_hi = r_lo + 4;
                        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(lds_lane + r_lo * 64));
                        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(lds_lane + r_hi * 64));
                        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                        const u32x4 af = u32x4{l2.x, l2.y, h2.x, h2.y};
                        acc[0] = E::mfma(af, l.b[t][0][k16], acc[0]);
                        acc[1] = E::mfma(af, l.b[t][1][k16], acc[1]);
                    }
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read before the next steps overwrite it
        };
        // One pair is multiplied out of one register set while the operands of the wave's next
        // pair fill the other and the row numbers of the pair after that are on their way.
        constexpr int kPair = 2 * kSkWaves;
        int s = wave;
        int out_col = 0;
        float out_bias = 0.0f;
        Loads l0, l1;
        Numbers n;
        if (s < nsteps) {
            n = numbers(s);
            issue(s, n, l0);
            if (s + kPair < nsteps)
                n = numbers(s + kPair);
        }
        // behind the first operands on their way: where this lane's sums go
        out_col = u.col0 + kept_n[u.kn_off + half * kSkCols + (jj < cnt ? jj : 0)];
        while (s < nsteps) {
            if (s + kPair < nsteps) {
                issue(s + kPair, n, l1);
                if (s + 2 * kPair < nsteps)
                    n = numbers(s + 2 * kPair);
            }
            multiply(s, l0);
            s += kPair;
            if (s >= nsteps)
                break;
            if (s + kPair < nsteps) {
                issue(s + kPair, n, l0);
                if (s + 2 * kPair < nsteps)
                    n = numbers(s + 2 * kPair);
            }
            multiply(s, l1);
            s += kPair;
        }
        if (p.bias)
            out_bias = p.bias[out_col];
        // the partial product of this wave: column cb * 32 + lane % 32, rows r4 * 8 + (lane / 32) * 4 + e
        float *const part = reinterpret_cast<float *>(stage);
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                float *const dst = part + (cb * 32 + (lane & 31)) * kSkPitch + r4 * 8 + (lane >> 5) * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    dst[e] = acc[cb][r4 * 4 + e];
            }
        __syncthreads();
        // (a wave without steps has written zeros)
        float sum[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
            sum[e] = 0.0f;
#pragma unroll
        for (int w = 0; w < kSkWaves; ++w) {
            const float *const src = reinterpret_cast<const float *>(sk_smem + w * kSkStage) + jj * kSkPitch + m8;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                sum[e] += src[e];
        }
        if (jj < cnt && m0 + m8 < m_end) {
            uint16_t *const dst = C + (int64_t)out_col * ldc + m0 + m8;
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e)
                v[e] = p.alpha * sum[e];
            if (p.beta != 0.0f) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (m0 + m8 + e < m_end)
                        v[e] += p.beta * E::from_bits(dst[e]);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e)
                v[e] += out_bias;
            tw_activate_all(v, p.act);
            uint32_t h[8];
#pragma unroll
            for (int e = 0; e < 8; ++e)
                h[e] = E::to_bits(tw_fp32_value(v[e]));
            store_chunk(dst, u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)},
                        m0 + m8, m_end, false);
        }
    }

    // ---- TW_PRUNED_ZERO: pruned columns receive act(beta * C + bias); shared out over the
    // workgroups of a row block
    if (in_range) {
        for (int z = p.n_gemm_u + ui * halves + half; z < p.n_all_u; z += n_units * halves) {
            const TileDev t = p.tiles[z - p.n_gemm_u];
            for (int i = tid; i < t.n_pruned * 4; i += NT) {
                const int jz = i >> 2, m = m0 + (i & 3) * 8;
                const int c = t.col0 + p.pruned_n[t.pn_off + jz];
                uint16_t *const dst = C + (int64_t)c * ldc + m;
                uint32_t w[4] = {0u, 0u, 0u, 0u};
                for (int e = 0; e < 8 && m + e < m_end; ++e) {
                    const float old = p.beta != 0.0f ? p.beta * E::from_bits(dst[e]) : 0.0f;
                    w[e >> 1] |= E::to_bits(tw_finish(old, p.bias, c, p.act)) << ((e & 1) * 16);
                }
                store_chunk(dst, u32x4{w[0], w[1], w[2], w[3]}, m, m_end, false);
            }
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
    // one workgroup per item, unit after unit (the queues are not used here: n_split == 1)
    const int item = blockIdx.x;

    if (item >= p.n_gemm_u * p.n_mblk) { // zero-fill item: pruned columns receive beta*C
        const int z = item - p.n_gemm_u * p.n_mblk;
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
    // strict bound (the reference's `idx > n` writes one element too many); grid-stride, so any n
    // fits a launch
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = dtype == TW_BF16 ? (uint16_t)Elem<TW_BF16>::to_bits(src[i])
                                  : (uint16_t)Elem<TW_F16>::to_bits(src[i]);
}

__global__ void delete_row_kernel(const uint16_t *matrix, uint16_t *matrix_2, int rows, int columns,
                                  const int32_t *mask)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < columns)
        for (int i = blockIdx.y; i < rows; i += gridDim.y) // any row count fits a launch
            matrix_2[(int64_t)i * columns + j] = matrix[(int64_t)(i + mask[i]) * columns + j];
}

__global__ void insert_row_kernel(uint16_t *matrix, const uint16_t *matrix_2, int rows, int columns,
                                  const int32_t *mask)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < columns)
        for (int i = blockIdx.y; i < rows; i += gridDim.y)
            matrix[(int64_t)(i + mask[i]) * columns + j] = matrix_2[(int64_t)i * columns + j];
}

// outputs above this size are written through to memory: the size of one XCD's L2
constexpr int64_t kStoreThroughBytes = 4 << 20;

// Kernel shapes: rows of a work item, widest unit piece taken, workgroups meant to share a CU.
// SHAPE_WIDE is tw_gemm_kmajor_kernel (64-bit addressing, for operands the 32-bit row offsets of
// the wave-specialised kernel cannot reach); all others are tw_gemm_ws_kernel<BM, BN>.
struct Shape {
    int bm, bn, wgs_per_cu;
};
static const Shape kShapes[TW_N_SHAPES] = {
    {256, 128, 1}, // TW_SHAPE_WIDE
    {128, 128, 2}, // TW_SHAPE_128x128
    {512, 64, 1},  // TW_SHAPE_512x64
    {128, 64, 2},  // TW_SHAPE_128x64
    {256, 128, 1}, // TW_SHAPE_256x128
    {128, 32, 2},  // TW_SHAPE_128x32
    {256, 64, 1},  // TW_SHAPE_256x64
    {64, 128, 1},  // TW_SHAPE_AS64
    {32, 128, 1},  // TW_SHAPE_AS32
    {32, 128, 1},  // TW_SHAPE_SKINNY
    {64, 128, 3},  // TW_SHAPE_BS
};

// LDS of the A-stationary kernel: the panel (all K rows, BMS rows m) and a C stage per wave
constexpr int kLdsBytes = 160 * 1024;
// (and a row of zeros behind the panel)
static int64_t as_lds_bytes(int K, int bms) { return (int64_t)(K + 1) * bms * 2 + as_waves(bms, false) * 32 * 36 * 2; }
static bool is_as_shape(int shape) { return shape == TW_SHAPE_AS64 || shape == TW_SHAPE_AS32; }
// shapes that walk the plan's units themselves: no work queue, no unit pieces
static bool is_queueless_shape(int shape)
{
    return is_as_shape(shape) || shape == TW_SHAPE_SKINNY || shape == TW_SHAPE_BS;
}

// Steps of loads a moving wave keeps in flight, per shape (bounded by its 256 registers: a step
// takes 4 * (A loads + weight loads per thread) of them).  Measured on the benchmark shapes: two
// steps in flight are as fast as three or four, or faster.
#ifndef TW_R_256x128
#define TW_R_256x128 2
#endif
#ifndef TW_R_128x128
#define TW_R_128x128 2
#endif
#ifndef TW_R_512x64
#define TW_R_512x64 2
#endif
#ifndef TW_R_128x64
#define TW_R_128x64 2
#endif
#ifndef TW_R_256x64
#define TW_R_256x64 3
#endif
#ifndef TW_R_128x32
#define TW_R_128x32 2
#endif

template <int DT> static void launch_kmajor(int shape, const GemmArgs &a, int grid, hipStream_t s)
{
    switch (shape) {
    case TW_SHAPE_WIDE:
        hipLaunchKernelGGL((tw_gemm_kmajor_kernel<DT, 4, 2, 64, 2, 1>), dim3(grid), dim3(512), 0, s, a);
        break;
    case TW_SHAPE_128x128:
        hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 128, 128, TW_R_128x128>), dim3(grid), dim3(256), 0, s, a);
        break;
    case TW_SHAPE_512x64:
        hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 512, 64, TW_R_512x64>), dim3(grid), dim3(512), 0, s, a);
        break;
    case TW_SHAPE_128x64:
        hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 128, 64, TW_R_128x64>), dim3(grid), dim3(256), 0, s, a);
        break;
    case TW_SHAPE_128x32:
        hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 128, 32, TW_R_128x32>), dim3(grid), dim3(256), 0, s, a);
        break;
    case TW_SHAPE_256x64:
        if (a.lds_dma)
            hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 256, 64, TW_R_256x64, true>), dim3(grid), dim3(512), 0, s, a);
        else
            hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 256, 64, TW_R_256x64>), dim3(grid), dim3(512), 0, s, a);
        break;
    default: // TW_SHAPE_256x128
        if (a.lds_dma)
            hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 256, 128, TW_R_256x128, true>), dim3(grid), dim3(512), 0, s, a);
        else
            hipLaunchKernelGGL((tw_gemm_ws_kernel<DT, 256, 128, TW_R_256x128>), dim3(grid), dim3(512), 0, s, a);
        break;
    }
}

// Process-wide tuning switches (tw_set_option); -1 = automatic.  The environment variables
// named in kOptEnv give their initial values and are read once.
static std::atomic<int> g_opt[TW_N_OPTIONS];
static std::once_flag g_opt_once;
static const char *const kOptEnv[TW_N_OPTIONS] = {"TWGEMM_SHAPE", "TWGEMM_WGS_PER_CU", "TWGEMM_PIECE",
                                                  "TWGEMM_XCD_QUEUES", "TWGEMM_SPIN_LIMIT", "TWGEMM_BALANCE",
                                                  "TWGEMM_LDS_DMA", "TWGEMM_LSTM_LOOK"};

static bool option_in_range(int option, int value)
{
    if (value == -1)
        return true;
    switch (option) {
    case TW_OPT_SHAPE:
        return value >= 0 && value < TW_N_SHAPES;
    case TW_OPT_WGS_PER_CU:
        return value >= 1 && value <= 8;
    case TW_OPT_PIECE:
        return value == 32 || value == 64 || value == 128;
    case TW_OPT_XCD_QUEUES:
        return value >= 0 && value <= 2;
    case TW_OPT_SPIN_LIMIT:
        return value >= 0;
    case TW_OPT_BALANCE:
    case TW_OPT_LDS_DMA:
    case TW_OPT_LSTM_LOOK:
        return value == 0 || value == 1;
    }
    return false;
}

static void init_options()
{
    std::call_once(g_opt_once, [] {
        for (int o = 0; o < TW_N_OPTIONS; ++o) {
            const char *v = getenv(kOptEnv[o]);
            const int x = v && *v ? atoi(v) : -1;
            g_opt[o].store(option_in_range(o, x) ? x : -1, std::memory_order_relaxed);
        }
    });
}

static int option(int o)
{
    init_options();
    return g_opt[o].load(std::memory_order_relaxed);
}

int get_option(int option_id) { return option(option_id); }

static int round_up32(int v) { return (v + 31) / 32 * 32; }

// What a launch runs with: kernel shape, columns of a unit piece, workgroups per CU.
struct Choice {
    int shape, piece, per_cu;
    bool xcd;
};

// Picks the shape from the plan and M.  Wide tiles run 256-row items (half the weight traffic
// per row of A of 128-row items).  Launches with too few items for the chip (skinny M) hand a
// unit out in pieces of 64 or 32 columns.  One queue per die is an option, not the default: the
// workgroups of a die then share the rows of A in their L2 (measured on the 0 %-sparse plan of
// the headline shape: a third of the reads from memory), but no benchmark shape ran faster for
// it and the stress shape, whose 512-row block of A fills an L2, ran 13 % slower.
static Choice choose_shape(const tw_plan *plan, int M, int64_t lda, int64_t ldc, bool reads_c)
{
    Choice c;
    const int width = std::max(32, round_up32(plan->max_unit_n)); // 32, 64, 96 or 128
    const int cu = plan->cu_count;
    const bool ws_ok = (uint64_t)plan->K * (uint64_t)lda * 2u < (1ull << 32);
    const int64_t units = std::max(1, plan->n_pipe_units);
    auto items = [&](int bm, int piece) {
        return units * ((width + piece - 1) / piece) * ((M + bm - 1) / bm);
    };
    // one queue per die where the tiles share their rows (a 0 %-sparse plan reads A once per die
    // then instead of once per tile); no sparse plan gained from it, see below
    c.xcd = option(TW_OPT_XCD_QUEUES) == 1 || (option(TW_OPT_XCD_QUEUES) == -1 && plan->rows_shared);
    c.piece = 128;
    // The A-stationary kernel (K short enough for a panel of A in LDS, C not read).  Measured on a
    // grid of M 128 .. 16384, K 512 .. 2048, N 512 .. 4096, tiles of 64 and 128 columns, 25 and
    // 50 % of the rows kept, against every streaming shape: wherever a 64-row panel fits it is
    // the fastest shape or within 8 % of it (tiles of 64 columns: by 5 - 50 %; BERT-base 14.2
    // against 18.2 us, BERT-large FFN1 at 50 / 75 / 90 %: 52 / 33 / 24 against 55 / 38 / 30);
    // 32-row panels below about a thousand rows of A, 64-row panels above.
    auto as_ok = [&](int shape) {
        return ws_ok && !reads_c && plan->n_blocks > 0 && plan->d_kept_pairs &&
               as_lds_bytes(plan->K, kShapes[shape].bm) <= kLdsBytes;
    };
    // The skinny kernel where it gives a compute unit at most two workgroups: the launch is then
    // a chain of trips to memory, which it keeps shortest (measured on M 16 .. 512 of the grid
    // above, replayed from a graph: 1.6 - 3 x faster up to one workgroup per unit, 1.1 - 1.5 x
    // up to two).
    const bool skinny_ok = plan->n_units > 0 && (M + 31) / 32 <= 65535; // its grid: units x row blocks
    // (not beyond 1024 rows: M 2048, N 512 would still be two workgroups per unit, but each then
    // walks a whole tile's kept rows for 32 rows of A: 10 - 24 us against 6 - 15)
    const bool skinny = skinny_ok && M <= 1024 && (int64_t)plan->n_halves * ((M + 31) / 32) <= 2 * (int64_t)cu;
    // The weight-stationary kernel where a tile keeps at most 192 rows under many rows of A, tiles
    // wider than 64 columns.  Measured on M 512 .. 16384, K 768 / 1024 / 4096, N 1024 / 4096 with
    // 64 .. 192 kept rows a tile against the choice below: from 2048 rows of A on it takes 0.58 -
    // 1.05 of the time (median 0.79 - 0.86; most where K is too long for a panel of A in LDS),
    // below that, and on tiles of 64 columns, it is as often slower as faster.
    // Its workgroups (unit x range of rows) have to fill the chip's slots evenly: BERT-base's 24
    // units give 384 workgroups for 512 slots, and the kernel is then 1 us slower than the
    // A-stationary one (15 against 14), where 32 units (BERT-large FFN1 at 90 %) gain 12 %.
    // With K = 512 the panel of A is small and the A-stationary kernel stays ahead (M 16384, N 4096:
    // 43 against 49 - 54 us), so the kernel is taken from K = 1024 on.
    const bool bs = bs_takes(plan, lda, ldc, reads_c) && width > 64 && M >= 2048 && plan->K >= 1024 && bs_fill(plan, M) >= 0.9;
    // Tiles of six steps and more on average, wide, with 256-row items for three quarters of the
    // chip: the streaming 256 x 128 kernel, whose loads write LDS directly, is ahead of the panel
    // (M 8192, K 1024, N 2048, half the rows kept: 28.4 against 33.2 us; BERT-large FFN1 at 50 %
    // 47 against 55; at four steps the two are level: BERT-large FFN1 at 75 % 34 against 34 - 37,
    // random tiles of K 1024 with a quarter of the rows kept 39 against 36)
    // (only where the 256-row items come out even over the workgroups: 600 items on 256 are three
    // rounds for 2.3 rounds of work, and the panel kernel wins: M 12800, K 768, N 3072 with 12 tiles
    // of 384 kept rows 28.3 against 32.2 us)
    const int64_t it256 = items(256, 128);
    const bool long_tiles = ws_ok && width > 64 && plan->pipe_steps >= 6 * units && it256 * 4 >= 3 * cu &&
                            it256 * 10 >= (it256 + cu - 1) / cu * cu * 9;
    if (skinny) {
        c.shape = TW_SHAPE_SKINNY;
    } else if (bs) {
        c.shape = TW_SHAPE_BS;
    } else if (!ws_ok) {
        c.shape = TW_SHAPE_WIDE;
    } else if (as_ok(TW_SHAPE_AS64) && (M > 128 || plan->n_blocks >= 96) &&
               (!plan->rows_shared || width <= 64 || items(256, 128) * 2 <= 3 * cu) && !long_tiles) {
        // (a 0 %-sparse plan with many 256-row items is better off streaming with one queue per
        // die: M 12800, K 768, N 3072: 87 against 96 us)
        // 64-row panels where they still give three quarters of the compute units a workgroup
        const int mblk64 = (M + 63) / 64;
        constexpr int tw64 = as_task_waves(64, false);
        const int groups64 = std::min(std::max(1, cu / mblk64), (plan->n_blocks + tw64 - 1) / tw64);
        c.shape = (int64_t)mblk64 * groups64 * 4 >= (int64_t)cu * 3 ? TW_SHAPE_AS64 : TW_SHAPE_AS32;
    } else if (!as_ok(TW_SHAPE_AS64) && as_ok(TW_SHAPE_AS32) && M > 128 &&
               (M <= 512 || (M <= 1024 && plan->n_blocks <= as_task_waves(32, false) * std::max(1, cu / ((M + 31) / 32))))) {
        // (up to 1024 rows where every wave still has at most one block: M 1024, K 2048, N 2048:
        // 12.3 - 15.8 us against 14.4 - 20.2)
        c.shape = TW_SHAPE_AS32;
    } else if (width > 64) {
        if (items(128, 128) * 2 < cu) { // skinny: split the units until half the chip has work
            c.piece = items(128, 64) * 2 >= cu ? 64 : 32;
            c.shape = c.piece == 64 ? TW_SHAPE_128x64 : TW_SHAPE_128x32;
        } else if (items(256, 128) * 4 <= cu) {
            // 256-row items for a quarter of the chip at most: 128-row items of 64 columns
            // (M 512, K 4096, N 4096: 30.2 against 36.4 us)
            c.piece = 64;
            c.shape = TW_SHAPE_128x64;
        } else {
            // (128 x 128 on two workgroups per CU fills more of the chip when 256-row items are
            // few, and is slower all the same: 17.8 against 12.4 us and 36.6 against 26.9 us on the
            // reference driver's first two shapes, 150 items each)
            c.shape = TW_SHAPE_256x128;
        }
    } else if (width > 32) {
        c.piece = 64;
        // (256-row items, whose loads write LDS directly, are ahead of 512-row items wherever
        // both fill the chip - M 2048, K 4096, N 4096, half the rows kept: 50 against 66 us; the
        // stress shape 363 against 385 - and of 128-row items from a quarter of a chip of items on)
        if (items(256, 64) * 4 >= cu) {
            c.shape = TW_SHAPE_256x64;
        } else if (items(128, 64) * 2 >= cu) {
            c.shape = TW_SHAPE_128x64;
        } else {
            c.piece = 32;
            c.shape = TW_SHAPE_128x32;
        }
    } else {
        c.piece = 32;
        c.shape = TW_SHAPE_128x32;
    }
    // forced choices, where they fit the plan: a shape takes pieces up to its width
    const int f_piece = option(TW_OPT_PIECE), f_shape = option(TW_OPT_SHAPE);
    if (f_shape >= 0 && is_as_shape(f_shape)) {
        if (as_ok(f_shape))
            c.shape = f_shape;
    } else if (f_shape == TW_SHAPE_SKINNY) {
        if (skinny_ok)
            c.shape = f_shape;
    } else if (f_shape == TW_SHAPE_BS) {
        if (bs_takes(plan, lda, ldc, reads_c))
            c.shape = f_shape;
    } else if (f_shape >= 0 && (f_shape != TW_SHAPE_WIDE ? ws_ok : true)) {
        const int piece = f_piece > 0 ? f_piece : std::min(128, kShapes[f_shape].bn);
        if (std::min(piece, width) <= kShapes[f_shape].bn) {
            c.shape = f_shape;
            c.piece = piece;
        }
    } else if (f_piece > 0 && std::min(f_piece, width) <= kShapes[c.shape].bn) {
        c.piece = f_piece;
    }
    if (c.shape == TW_SHAPE_WIDE || is_queueless_shape(c.shape))
        c.piece = 128;
    c.per_cu = option(TW_OPT_WGS_PER_CU) > 0 ? option(TW_OPT_WGS_PER_CU) : kShapes[c.shape].wgs_per_cu;
    return c;
}

// the A-stationary kernel: one workgroup per (row block, group of blocks); no work queue
bool takes_row_major_directly(const tw_plan *plan, float beta)
{
    return beta == 0.0f && plan->d_kept_pairs && plan->n_blocks > 0 && as_lds_bytes(plan->K, 32) <= kLdsBytes;
}

template <int DT, int BMS, bool RM> static int launch_as(const tw_plan *plan, const GemmArgs &a, int M, hipStream_t s)
{
    const int pst = prepare_device();
    if (pst != TW_OK)
        return pst;
    const int n_mblk = (M + BMS - 1) / BMS;
    // as many groups as keep every compute unit at one workgroup, each wave with a block or more
    const int per_wg = as_task_waves(BMS, RM);
    int n_groups = std::max(1, plan->cu_count / n_mblk);
    n_groups = std::min(n_groups, std::max(1, (plan->n_blocks + per_wg - 1) / per_wg));
    if ((int64_t)n_mblk * n_groups > (int64_t)0x7fffffff)
        return fail(TW_ERR_SHAPE, "%lld workgroups (M=%d): a launch takes at most %lld",
                    (long long)n_mblk * n_groups, M, (long long)(int64_t)0x7fffffff);
    hipLaunchKernelGGL((tw_gemm_as_kernel<DT, BMS, RM>), dim3((unsigned)(n_mblk * n_groups)),
                       dim3(64 * as_waves(BMS, RM)), (size_t)as_lds_bytes(plan->K, BMS), s, a, plan->d_blocks, plan->n_blocks, n_groups,
                       n_mblk, plan->K, plan->blocks_per_unit);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

// the skinny kernel: one workgroup per (half of a unit, 32-row block)
template <int DT> static int launch_skinny(const tw_plan *plan, const GemmArgs &a, hipStream_t s)
{
    const int halves = plan->max_unit_n > kSkCols ? 2 : 1;
    const int64_t gx = ((int64_t)plan->n_units + kXcd - 1) / kXcd * kXcd * halves;
    const int64_t gy = (a.M + kSkRows - 1) / kSkRows;
    if (gx > (int64_t)0x7fffffff || gy > 65535)
        return fail(TW_ERR_SHAPE, "%lld x %lld workgroups (M=%d): the skinny kernel takes at most 65535 row blocks",
                    (long long)gx, (long long)gy, a.M);
    hipLaunchKernelGGL((tw_gemm_skinny_kernel<DT>), dim3((unsigned)gx, (unsigned)gy), dim3(64 * kSkWaves), 0, s, a,
                       plan->n_units, halves);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

} // namespace tw

using namespace tw;

// Launch-time scratch of tw_gemm_static: the work-queue counters of one launch.  One copy per
// GPU, held until the process ends; every tw_gemm_static call on a GPU uses it.
constexpr int kStaticScratchInts = 64; // 256 bytes, of which kTicketInts counters are used
static_assert(kStaticScratchInts >= kTicketInts, "the counters of a launch fit the static scratch");
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];

namespace tw {

namespace {
constexpr int kMaxDevices = 64;
int32_t *g_scratch_ptr[kMaxDevices] = {};
} // namespace

// Once per device: the set-up a launch needs that may not run while a stream is being captured
// (symbol look-up, function attributes).  Every plan runs it when it is built, so a caller that
// records launches into a graph has it behind them; the launch paths call it again for the
// devices no plan was built on, where it costs one flag load.
int prepare_device()
{
    static std::mutex mu;
    static std::atomic<bool> ready[kMaxDevices];
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(TW_ERR_DEVICE, "device %d: the library serves devices 0..%d", dev, kMaxDevices - 1);
    if (ready[dev].load(std::memory_order_acquire))
        return TW_OK;
    std::lock_guard<std::mutex> lock(mu);
    if (ready[dev].load(std::memory_order_relaxed))
        return TW_OK;
    const void *as_kernels[] = {
        (const void *)tw_gemm_as_kernel<TW_F16, 64, false>,  (const void *)tw_gemm_as_kernel<TW_F16, 32, false>,
        (const void *)tw_gemm_as_kernel<TW_F16, 64, true>,   (const void *)tw_gemm_as_kernel<TW_F16, 32, true>,
        (const void *)tw_gemm_as_kernel<TW_BF16, 64, false>, (const void *)tw_gemm_as_kernel<TW_BF16, 32, false>,
        (const void *)tw_gemm_as_kernel<TW_BF16, 64, true>,  (const void *)tw_gemm_as_kernel<TW_BF16, 32, true>,
    };
    for (const void *k : as_kernels)
        TW_HIP(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
    void *p = nullptr;
    TW_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = static_cast<int32_t *>(p);
    ready[dev].store(true, std::memory_order_release);
    return TW_OK;
}

} // namespace tw

extern "C" {

int tw_set_option(int option_id, int value)
{
    if (option_id < 0 || option_id >= TW_N_OPTIONS)
        return fail(TW_ERR_LAYOUT, "option %d: unknown", option_id);
    if (!option_in_range(option_id, value))
        return fail(TW_ERR_LAYOUT, "option %d: value %d is out of range", option_id, value);
    init_options();
    g_opt[option_id].store(value, std::memory_order_relaxed);
    return TW_OK;
}

int tw_gemm(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C, int c_layout,
            int64_t ldc, int M, float alpha, float beta, int pruned_cols, void *stream)
{
    return tw_gemm_ex(plan, A, a_layout, lda, C, c_layout, ldc, M, alpha, beta, pruned_cols, nullptr,
                      stream);
}

namespace {

// argument checks shared by the launching entry points; TW_OK with *run == false: nothing to do
int check_gemm_args(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C,
                    int c_layout, int64_t ldc, int M, int pruned_cols, const tw_epilogue *ep,
                    bool *run)
{
    *run = false;
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
    // the plan's tables and packed weight live on the device it was built on
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    if (dev != plan->device)
        return fail(TW_ERR_DEVICE, "the plan was built on device %d, the current device is %d",
                    plan->device, dev);
    *run = true;
    return TW_OK;
}

void fill_common(GemmArgs &a, const tw_plan *plan, const void *A, int64_t lda, void *C, int64_t ldc,
                 int M, float alpha, float beta, const tw_epilogue *ep)
{
    a.units = plan->d_units;
    a.tiles = plan->d_tiles;
    a.kept_k = plan->d_kept_k_pad;
    a.kept_pairs = plan->d_kept_pairs;
    a.kept_n = plan->d_kept_n;
    a.pruned_n = plan->d_pruned_n;
    a.Bp = plan->d_Bp;
    a.A = A;
    a.C = C;
    a.lda = lda;
    a.ldc = ldc;
    a.M = M;
    a.alpha = alpha;
    a.beta = beta;
    a.bias = ep ? ep->bias : nullptr;
    a.act = ep ? ep->activation : TW_ACT_NONE;
    a.store_through = 0;
    a.ticket = nullptr;
    a.n_bal = 0;
    a.rb_major = 0;
    a.lds_dma = 0;
    a.a_bytes = a.b_bytes = 0;
    a.n_arg_units = 0;
}

// work items of a launch are counted in 32-bit integers
constexpr int64_t kMaxItems = 0x7fffffff;

// item matrix and queues of a launch with `bm`-row items and unit pieces of `piece` columns
void fill_queues(GemmArgs &a, const tw_plan *plan, int M, int bm, int piece, int pruned_cols, bool xcd)
{
    const int width = std::max(32, round_up32(plan->max_unit_n));
    a.n_split = (std::min(width, 128) + piece - 1) / piece;
    a.piece_nb = piece / kMfmaN;
    a.n_mblk = (M + bm - 1) / bm;
    a.n_pipe_u = plan->n_pipe_units * a.n_split;
    a.n_gemm_u = plan->n_units * a.n_split;
    a.n_all_u = a.n_gemm_u + (pruned_cols == TW_PRUNED_ZERO ? plan->n_zero_tiles : 0);
    a.n_own = xcd ? a.n_mblk / kXcd : 0;
    a.n_own_items = a.n_own * a.n_all_u;
    a.n_tail_mblk = a.n_mblk - kXcd * a.n_own;
    a.n_tail_items = a.n_tail_mblk * a.n_all_u;
}

// Row blocks sized per column of the item matrix, for launches whose items do not fill the chip
// once: with whole row blocks the launch lasts as long as an item of the tile with the most kept
// rows, next to idle compute units and to items that end early.  Column u gets row blocks of
// h_u rows, a multiple of 64 (whole 128-byte lines of a K-major row of 16-bit elements, whole
// multiplying waves) of at most bm, so that steps_u * h_u is as even as the items allow while
// all of them still fit the chip at once.  Returns false (and leaves `a` alone) where that gains
// nothing: one column, every column at full height, more items than workgroups.
bool balance_items(GemmArgs &a, const tw_plan *plan, int M, int bm, int64_t wgs)
{
    if (a.n_split != 1 || a.n_own != 0 || a.n_all_u > kBalColumns || a.n_pipe_u < 2 || bm < 128)
        return false;
    int steps[kBalColumns];
    for (int u = 0; u < a.n_all_u; ++u)
        steps[u] = u < a.n_pipe_u ? plan->h_units[u].k_pad / kBlockK : 0;
    auto items_at = [&](int64_t cost, int32_t *rows) {
        int64_t n = 0;
        for (int u = 0; u < a.n_all_u; ++u) {
            int h = bm;
            if (steps[u] > 0)
                h = (int)std::min<int64_t>(bm, std::max<int64_t>(64, cost / steps[u] / 64 * 64));
            rows[u] = h;
            n += (M + h - 1) / h;
        }
        return n;
    };
    // candidate costs: every steps_u * h; the smallest whose items fit
    int64_t best = 0;
    int32_t rows[kBalColumns], best_rows[kBalColumns];
    for (int u = 0; u < a.n_pipe_u; ++u)
        for (int h = 64; h <= bm; h += 64) {
            const int64_t cost = (int64_t)steps[u] * h;
            if ((best == 0 || cost < best) && items_at(cost, rows) <= wgs) {
                best = cost;
                std::copy(rows, rows + a.n_all_u, best_rows);
            }
        }
    if (best == 0)
        return false;
    bool shorter = false;
    for (int u = 0; u < a.n_pipe_u; ++u)
        shorter |= best_rows[u] < bm;
    if (!shorter)
        return false;
    a.n_bal = a.n_all_u;
    int32_t first = 0;
    for (int u = 0; u < a.n_all_u; ++u) {
        a.bal_first[u] = first;
        a.bal_rows[u] = best_rows[u];
        first += (M + best_rows[u] - 1) / best_rows[u];
    }
    for (int u = a.n_all_u; u <= kBalColumns; ++u)
        a.bal_first[u] = first;
    a.n_tail_items = first;
    return true;
}

// launches the K-major kernels with the counters at `ticket` (kTicketInts zeros)
int launch_gemm(const tw_plan *plan, GemmArgs &a, const Choice &c, int32_t *ticket, hipStream_t s)
{
    if (a.n_all_u == 0)
        return TW_OK;
    a.ticket = ticket;
    a.n_arg_units = plan->n_units <= kMaxArgUnits ? plan->n_units : 0;
    for (int i = 0; i < a.n_arg_units; ++i)
        a.arg_units[i] = plan->h_units[i];
    if (is_as_shape(c.shape)) {
        if (plan->dtype == TW_F16)
            return c.shape == TW_SHAPE_AS64 ? launch_as<TW_F16, 64, false>(plan, a, a.M, s)
                                            : launch_as<TW_F16, 32, false>(plan, a, a.M, s);
        return c.shape == TW_SHAPE_AS64 ? launch_as<TW_BF16, 64, false>(plan, a, a.M, s)
                                        : launch_as<TW_BF16, 32, false>(plan, a, a.M, s);
    }
    if (c.shape == TW_SHAPE_SKINNY)
        return plan->dtype == TW_F16 ? launch_skinny<TW_F16>(plan, a, s) : launch_skinny<TW_BF16>(plan, a, s);
    if (c.shape == TW_SHAPE_BS)
        return launch_bs(plan, a, option(TW_OPT_WGS_PER_CU), s);
    // queue 0 is the longest: one workgroup per entry, up to the chip's share of a queue
    const int64_t qlen0 = (int64_t)a.n_own_items + (a.n_tail_items + kXcd - 1) / kXcd;
    const int64_t per_queue = std::max<int64_t>(1, (int64_t)plan->cu_count * c.per_cu / kXcd);
    const int grid = (int)(kXcd * std::min(qlen0, per_queue));
    if (plan->dtype == TW_F16)
        launch_kmajor<TW_F16>(c.shape, a, grid, s);
    else
        launch_kmajor<TW_BF16>(c.shape, a, grid, s);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

__global__ void clear_counters_kernel(int32_t *counters)
{
    if (threadIdx.x < kTicketInts)
        counters[threadIdx.x] = 0;
}

__global__ void clear_all_slots_kernel(int32_t *tickets)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < kTicketSlots * kTicketInts)
        tickets[i] = 0;
}

// Device address of `scratch` on the current device (the array's name is only a host-side
// stand-in; every GPU holds its own copy at its own address), looked up by prepare_device.
int static_scratch(int32_t **out)
{
    const int st = prepare_device();
    if (st != TW_OK)
        return st;
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    *out = g_scratch_ptr[dev];
    return TW_OK;
}

// tw_gemm_ex and tw_gemm_static: the latter brings the counters (the library's `scratch` array),
// cleared on the stream before the launch; the former takes a ticket slot of the plan.
int gemm_impl(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C, int c_layout,
              int64_t ldc, int M, float alpha, float beta, int pruned_cols, const tw_epilogue *ep,
              void *stream, bool use_static)
{
    bool run = false;
    const int st = check_gemm_args(plan, A, a_layout, lda, C, c_layout, ldc, M, pruned_cols, ep, &run);
    if (st != TW_OK || !run)
        return st;
    GemmArgs a;
    fill_common(a, plan, A, lda, C, ldc, M, alpha, beta, ep);
    if (a_layout == TW_LAYOUT_ROWMAJOR && c_layout == TW_LAYOUT_ROWMAJOR && takes_row_major_directly(plan, beta)) {
        // both operands row-major, K short enough for a panel of A in LDS, C not read: the
        // A-stationary kernel in its row-major form (64-row panels where they fit and still give
        // three quarters of the compute units a workgroup)
        fill_queues(a, plan, M, 64, 128, pruned_cols, false);
        a.n_arg_units = plan->n_units <= kMaxArgUnits ? plan->n_units : 0;
        for (int i = 0; i < a.n_arg_units; ++i)
            a.arg_units[i] = plan->h_units[i];
        const int mblk64 = (M + 63) / 64;
        const int groups64 =
            std::min(std::max(1, plan->cu_count / mblk64), (plan->n_blocks + as_task_waves(64, true) - 1) / as_task_waves(64, true));
        const bool b64 = as_lds_bytes(plan->K, 64) <= kLdsBytes &&
                         (int64_t)mblk64 * groups64 * 4 >= (int64_t)plan->cu_count * 3;
        hipStream_t s = (hipStream_t)stream;
        if (plan->dtype == TW_F16)
            return b64 ? launch_as<TW_F16, 64, true>(plan, a, M, s) : launch_as<TW_F16, 32, true>(plan, a, M, s);
        return b64 ? launch_as<TW_BF16, 64, true>(plan, a, M, s) : launch_as<TW_BF16, 32, true>(plan, a, M, s);
    }
    if (a_layout != TW_LAYOUT_KMAJOR || c_layout != TW_LAYOUT_KMAJOR) {
        // layout-generic path (element strides), 128-row blocks, one workgroup per item
        fill_queues(a, plan, M, 128, 128, pruned_cols, false);
        const int64_t n_items = (int64_t)a.n_all_u * a.n_mblk;
        if (n_items == 0)
            return TW_OK;
        if (n_items > kMaxItems)
            return fail(TW_ERR_SHAPE, "%lld work items (M=%d): a launch takes at most %lld",
                        (long long)n_items, M, (long long)kMaxItems);
        const int64_t sa_m = a_layout == TW_LAYOUT_KMAJOR ? 1 : lda;
        const int64_t sa_k = a_layout == TW_LAYOUT_KMAJOR ? lda : 1;
        const int64_t sc_m = c_layout == TW_LAYOUT_KMAJOR ? 1 : ldc;
        const int64_t sc_n = c_layout == TW_LAYOUT_KMAJOR ? ldc : 1;
        if (plan->dtype == TW_F16)
            hipLaunchKernelGGL((tw_gemm_generic_kernel<TW_F16>), dim3((unsigned)n_items), dim3(256), 0,
                               (hipStream_t)stream, a, sa_m, sa_k, sc_m, sc_n);
        else
            hipLaunchKernelGGL((tw_gemm_generic_kernel<TW_BF16>), dim3((unsigned)n_items), dim3(256), 0,
                               (hipStream_t)stream, a, sa_m, sa_k, sc_m, sc_n);
        TW_HIP(hipGetLastError());
        return TW_OK;
    }

    const Choice c = choose_shape(plan, M, lda, ldc, beta != 0.0f);
    fill_queues(a, plan, M, kShapes[c.shape].bm, c.piece, pruned_cols, c.xcd);
    a.rb_major = option(TW_OPT_XCD_QUEUES) == 2;
    // 256-row items whose loads write LDS directly (measured faster on every shape tried, with
    // one item per workgroup and with several)
    if ((c.shape == TW_SHAPE_256x128 || c.shape == TW_SHAPE_256x64) && option(TW_OPT_LDS_DMA) != 0 && (uint64_t)plan->packed_elems * 2u < (1ull << 32)) {
        a.lds_dma = 1;
        a.a_bytes = (uint32_t)((uint64_t)plan->K * (uint64_t)lda * 2u); // (a chunk that holds row K - 1's last elements is read whole)
        a.b_bytes = (uint32_t)((uint64_t)plan->packed_elems * 2u);
    }
    // (a tuning switch, off unless asked for: measured on the benchmark shapes it changes nothing,
    // a step of an item takes as long at 192 rows as at 256)
    if (c.shape != TW_SHAPE_WIDE && !is_queueless_shape(c.shape) && option(TW_OPT_BALANCE) == 1)
        balance_items(a, plan, M, kShapes[c.shape].bm, (int64_t)plan->cu_count * c.per_cu);
    if ((int64_t)a.n_all_u * a.n_mblk > kMaxItems)
        return fail(TW_ERR_SHAPE, "%lld work items (M=%d): a launch takes at most %lld",
                    (long long)a.n_all_u * a.n_mblk, M, (long long)kMaxItems);
    // an output larger than one L2 is written through (see store_chunk)
    a.store_through = (int64_t)M * plan->N * 2 > kStoreThroughBytes;
    // Ticket slot of this launch.  A launch recorded into a HIP graph keeps its slot for every
    // replay, so recorded launches draw from a range of their own that eager launches never use.
    hipStream_t s = (hipStream_t)stream;
    if (use_static) {
        // the counters must start at zero: cleared with a kernel (a launch can then be recorded
        // into a graph), whatever the last call on this GPU left in them
        int32_t *counters = nullptr;
        const int sst = static_scratch(&counters);
        if (sst != TW_OK)
            return sst;
        if (a.n_all_u == 0)
            return TW_OK;
        hipLaunchKernelGGL(clear_counters_kernel, dim3(1), dim3(64), 0, s, counters);
        TW_HIP(hipGetLastError());
        return launch_gemm(plan, a, c, counters, s);
    }
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusNone;
    }
    unsigned slot;
    if (cap == hipStreamCaptureStatusActive)
        slot = kEagerSlots + __atomic_fetch_add(&plan->next_capture_slot, 1u, __ATOMIC_RELAXED) %
                                 (unsigned)(kTicketSlots - kEagerSlots);
    else
        slot = __atomic_fetch_add(&plan->next_slot, 1u, __ATOMIC_RELAXED) % (unsigned)kEagerSlots;
    return launch_gemm(plan, a, c, plan->d_tickets + kTicketInts * slot, s);
}

} // namespace

int tw_gemm_ex(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C, int c_layout,
               int64_t ldc, int M, float alpha, float beta, int pruned_cols, const tw_epilogue *ep,
               void *stream)
{
    return gemm_impl(plan, A, a_layout, lda, C, c_layout, ldc, M, alpha, beta, pruned_cols, ep, stream,
                     false);
}

int tw_gemm_choice(const tw_plan *plan, int M, int64_t lda, int64_t ldc, float beta, int32_t *choice)
{
    if (!plan || !choice)
        return fail(TW_ERR_NULL, "plan or choice is NULL");
    if (M < 0)
        return fail(TW_ERR_SHAPE, "M=%d is negative", M);
    const Choice c = choose_shape(plan, M, lda, ldc, beta != 0.0f);
    choice[0] = c.shape;
    choice[1] = c.piece;
    choice[2] = c.per_cu;
    choice[3] = c.xcd ? 1 : 0;
    return TW_OK;
}

int tw_plan_reset(tw_plan *plan, void *stream)
{
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    if (dev != plan->device)
        return fail(TW_ERR_DEVICE, "the plan was built on device %d, the current device is %d", plan->device, dev);
    if (!plan->d_tickets)
        return TW_OK;
    // a kernel, not a memset: the call may be recorded into a graph
    hipLaunchKernelGGL(clear_all_slots_kernel, dim3((kTicketSlots * kTicketInts + 255) / 256), dim3(256), 0,
                       (hipStream_t)stream, plan->d_tickets);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int tw_gemm_static(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C,
                   int c_layout, int64_t ldc, int M, float alpha, float beta, int pruned_cols,
                   const tw_epilogue *ep, void *stream)
{
    return gemm_impl(plan, A, a_layout, lda, C, c_layout, ldc, M, alpha, beta, pruned_cols, ep, stream,
                     true);
}

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
    hipLaunchKernelGGL(cast_f32_kernel, dim3((unsigned)std::min<int64_t>((n + 255) / 256, 1 << 20)), dim3(256), 0,
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
    hipLaunchKernelGGL(delete_row_kernel, dim3((columns + 255) / 256, std::min(rows, 65535)), dim3(256), 0,
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
    hipLaunchKernelGGL(insert_row_kernel, dim3((columns + 255) / 256, std::min(rows, 65535)), dim3(256), 0,
                       (hipStream_t)stream, (uint16_t *)matrix, (const uint16_t *)matrix_2, rows,
                       columns, mask);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

} // extern "C"
