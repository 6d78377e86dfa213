// Weight-stationary kernel of the tile-wise-sparse GEMM (TW_SHAPE_BS), for tiles that keep few
// rows (at most 192) under many rows of A: BERT-like layers at 75 % sparsity and more.
//
// A workgroup takes one unit (up to 128 compact columns of a tile) and a range of rows of A.  Its
// four multiplying waves own one block of 32 compact columns each and keep that block's packed
// weight - every kept row of it - in registers for the whole range, so the weight is read once
// per workgroup and the steady state moves nothing but A in and C out.  A fifth wave only loads:
// it gathers the tile's kept rows of A, 64 rows m at a time, with loads that write straight into
// LDS (buffer_load_dwordx4 ... lds: no registers, no LDS write instructions), a step of 64 kept
// rows per stage of a ring of four, two steps ahead of the multiplying waves.  Its waits for a
// step count exactly the loads issued behind it.  (It issues no store: memory operations of a
// wave complete in order, and a store in front of a load keeps that load's completion back
// until memory has acknowledged the store; measured with the stores of C moved into this wave:
// 27 us on a problem that takes 13.)  Both sides meet at one barrier per step.  The reference's
// counterpart is the masked main loop (cutlass/gemm/gemm_mainloop.h:230-338) with its gathered
// global -> shared stage (cutlass/tile_iterator.h:786-816), which re-reads the weight tile for
// every 128 rows of A.
//
//   stage:  64 kept rows k x 64 rows m, row k at k * 128 bytes, no padding (a load writes 1 KiB
//           of consecutive LDS: 8 rows); the two 64-byte halves of a row are swapped in rows
//           with bit 1 set, so that the four rows a transposed read touches fall into four
//           different bank groups.  The swap happens on the global side: lane l of a load
//           fetches chunk (l % 8) ^ 4 of such a row.
//   edges:  A is addressed through a buffer descriptor; a lane's offset names its row k and
//           16-byte piece, the scalar offset the block's first row m.  A list of kept rows is
//           padded to whole steps: the padding gets an offset beyond the buffer, for which the
//           hardware delivers zeros, so that nothing of a row the tile does not keep ever
//           reaches a product.  Rows m beyond M fetch whatever follows (or zeros); the rows of
//           the product they feed are never stored.
//   ranges: the rows of A are cut into n_ranges ranges on 32-row boundaries; the workgroups of a
//           range run on one die (workgroup b runs on die b % 8), so that the units of a range
//           share its rows of A in that die's L2.
//   output: a wave turns its 64 x 32 product through its own piece of LDS (no barrier) and
//           stores 16-byte pieces of whole columns, as the other kernels do; same order of
//           summation, so the same bits.
// Takes a K-major A below 4 GiB, a K-major C, and beta == 0 (C is not read).
#include "tw_device.h"

#include <algorithm>

namespace tw {

constexpr int kBsRows = 64;                       // rows of A per block of a range
constexpr int kBsMulWaves = 4;
constexpr int kBsLoadWave = kBsMulWaves;
constexpr int kBsWaves = kBsMulWaves + 1;
constexpr int kBsRing = 4;                        // stages
constexpr int kBsAhead = 2;                       // steps of loads in flight ahead of the multiplying waves
constexpr int kBsStage = kBlockK * kBsRows * 2;   // 8 KiB
constexpr int kBsCPitch = kBsRows + 4;            // elements per column of a wave's C stage
constexpr int kBsCStage = 32 * kBsCPitch * 2;     // bytes
constexpr int kBsPerCu = 2;                       // workgroups meant to share a compute unit
constexpr int kBsRsrcFlags = 0x00020000;          // word 3 of a raw buffer descriptor of this target
static_assert(kBsRing >= kBsAhead + 2, "a stage is refilled only after the step before last has been multiplied");
static_assert(kBsAhead == 2, "the loading wave's waits are written out for two steps ahead");
constexpr int kBsMaxSteps = 3;                    // steps of 64 kept rows the widest instantiation holds in registers
                                                  // (four: 64 more registers than a wave of four a SIMD has)

// the loading wave: waits until at most N of its loads are outstanding, then meets the other waves
template <int N> __device__ __forceinline__ void bs_wait_loads_and_meet()
{
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// (at most 128 registers: the first SIMD of a compute unit holds two waves of each of its two
// workgroups; a third workgroup's five waves find no room on it)
template <int DT, int NS>
__global__ void __launch_bounds__(64 * kBsWaves, 4)
    tw_gemm_bs_kernel(const GemmArgs p, int n_units, int n_ranges, int row_units, int affine, uint32_t a_bytes,
                      uint32_t)
{
    using E = Elem<DT>;
    static_assert(NS >= 1 && NS <= kBsMaxSteps, "steps in registers");
    __shared__ __align__(1024) unsigned char ring[kBsRing * kBsStage];
    __shared__ __align__(16) unsigned char cstage[kBsMulWaves * kBsCStage];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // workgroup -> (unit, range); with `affine` the ranges r = die (mod 8) sit on one die
    int ui, r;
    if (affine) {
        const int die = blockIdx.x % kXcd, i = blockIdx.x / kXcd;
        ui = i % n_units;
        r = die + kXcd * (i / n_units);
    } else {
        r = blockIdx.x % n_ranges;
        ui = blockIdx.x / n_ranges;
    }
    if (r >= n_ranges)
        return;
    const int m_lo = (int)((int64_t)r * row_units / n_ranges) * 32;
    const int m_hi = min((int)((int64_t)(r + 1) * row_units / n_ranges) * 32, p.M);
    if (m_lo >= m_hi)
        return;
    const UnitDev u = load_unit(p, ui);
    const int nsteps = u.k_pad / kBlockK; // <= NS (host check)
    const int n_mb = (m_hi - m_lo + kBsRows - 1) / kBsRows;
    const int total = n_mb * nsteps; // steps, and barriers, of the workgroup

    if (wave == kBsLoadWave) {
        // ================= the loading wave =================================================
        if (nsteps == 0)
            return;
        const int rr = lane >> 3, pos = lane & 7;
        const uint32_t lda_b = (uint32_t)p.lda * 2u;
        const __amdgpu_buffer_rsrc_t a_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p.A), 0, (int)a_bytes, kBsRsrcFlags);
        // Load j of a step covers its kept rows 8 j .. 8 j + 7; lane l fetches 16 bytes of row
        // 8 j + l / 8 into LDS position l % 8 of that row.
        uint32_t off[NS][8];
        {
            // the row numbers: one load per step for the whole wave (lane l asks for row l of the
            // step; a step the unit does not have asks for its last one again), all in flight
            // together, then handed to the lanes that fetch the row
            int knum[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s)
                knum[s] = p.kept_k[u.kk_off + (s < nsteps ? s : nsteps - 1) * kBlockK + lane]; // the list is padded: in bounds
#pragma unroll
            for (int s = 0; s < NS; ++s) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int row = j * 8 + rr; // kept row of the step
                    const int chunk = pos ^ (((row >> 1) & 1) << 2);
                    const uint32_t k = (uint32_t)__shfl(knum[s], row);
                    off[s][j] = s * kBlockK + row < u.k_kept ? k * lda_b + (uint32_t)chunk * 16u : 0xFFFFFFF0u;
                }
            }
        }
        TW_LDS(unsigned char) const lds0 = (TW_LDS(unsigned char))ring;
        // Step gi is issued, then step gi - 2 handed over: behind its loads are those of the steps
        // issued since (two, fewer at the end of the range).
        int s_cur = 0, mb_cur = 0;
        for (int gi = 0; gi < total + kBsAhead; ++gi) {
            if (gi < total) {
                const int m0b = (m_lo + mb_cur * kBsRows) * 2;
                TW_LDS(unsigned char) const dst = lds0 + (gi % kBsRing) * kBsStage;
#define TW_BS_ISSUE(S)                                                                                      \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) __builtin_amdgcn_raw_ptr_buffer_load_lds(                 \
        a_rsrc, (TW_LDS(void))(dst + j * 1024), 16, (int)off[(S) < NS ? (S) : 0][j], m0b, 0, 0)
                switch (s_cur) { // (the offsets of a step sit in registers: one copy of the loads per step)
                case 0:
                    TW_BS_ISSUE(0);
                    break;
                case 1:
                    TW_BS_ISSUE(1);
                    break;
                default:
                    TW_BS_ISSUE(2);
                    break;
                }
#undef TW_BS_ISSUE
                if (++s_cur == nsteps) {
                    s_cur = 0;
                    ++mb_cur;
                }
            }
            if (gi >= kBsAhead) {
                const int behind = min(gi, total - 1) - (gi - kBsAhead); // steps issued behind the one handed over
                if (behind >= 2)
                    bs_wait_loads_and_meet<16>();
                else if (behind == 1)
                    bs_wait_loads_and_meet<8>();
                else
                    bs_wait_loads_and_meet<0>();
            }
        }
        return;
    }

    // ================= multiplying waves ====================================================
    // A unit of at most 64 compact columns has two blocks: its four waves then take a block and
    // one 32-row half of the 64 rows each, instead of two waves taking a block and two idling.
    const bool narrow = u.nb_cnt <= 2;
    const int half = wave >> 1;
    const bool active = (narrow ? wave & 1 : wave) < u.nb_cnt;
    const int nb = active ? (narrow ? wave & 1 : wave) : 0;
    const int cnt = min(32, u.n_cnt - nb * 32); // compact columns of this wave's block
    const int L = lane & 15;
    const int j = lane & 31;
    // weight fragments of the block: every kept row, in registers
    u32x4 bq[NS][4];
    {
        const unsigned char *const bsrc = reinterpret_cast<const unsigned char *>(p.Bp) +
                                          (nsteps ? u.b_off * 2 + (int64_t)(u.nb0 + nb) * 4096 : 0) + lane * 16;
        const int64_t step_b = (int64_t)u.nblk * 4096;
        // (no branches: a step the unit does not have fetches its last one again and is never used;
        // a unit without kept rows owns no weight: it fetches the plan's first fragments)
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int sc = s < nsteps ? s : max(nsteps - 1, 0);
#pragma unroll
            for (int k16 = 0; k16 < 4; ++k16)
                bq[s][k16] = *reinterpret_cast<const u32x4 *>(bsrc + sc * step_b + k16 * 1024);
        }
    }
    int out_col = u.col0 + p.kept_n[u.kn_off + nb * 32 + (j < cnt ? j : 0)];
    float out_bias = p.bias ? p.bias[out_col] : 0.0f;
    // Everything fetched so far is waited for here, before the loop over the range: inside it
    // the only memory operations of these waves are the output stores, and a wait placed there
    // for one of these loads would wait for the stores of the block before as well.
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int k16 = 0; k16 < 4; ++k16)
            asm volatile("" : "+v"(bq[s][k16]));
    asm volatile("" : "+v"(out_col), "+v"(out_bias));
    // this lane's address inside a stage for the transposed reads: row (lane / 32) * 8 + L / 4 of a
    // group of 16 kept rows, 8 bytes at m = (lane / 16 % 2) * 16 + (L % 4) * 4 of a 32-row half;
    // the halves of a row are swapped where bit 1 of the row is set
    const uint32_t swap = (uint32_t)((L >> 3) & 1);
    const uint32_t lane_row = (uint32_t)((lane >> 5) * 8 + (L >> 2)) * 128u + (uint32_t)(((lane >> 4) & 1) * 32 + (L & 3) * 8);
    const uint32_t lane_a[2] = {lane_row + swap * 64u, lane_row + (1u - swap) * 64u};
    TW_LDS(unsigned char) const lds0 = (TW_LDS(unsigned char))ring;
    uint16_t *const cst = reinterpret_cast<uint16_t *>(cstage + wave * kBsCStage);
    uint16_t *const C = reinterpret_cast<uint16_t *>(p.C);

    int g = 0; // flat step
    for (int mb = 0; mb < n_mb; ++mb) {
        f32x16 acc[2];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[mi][e] = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (s < nsteps) {
                TW_LDS_BARRIER(); // the step is in its stage (and this wave's reads of the step before are over)
                if (active) {
                    TW_LDS(unsigned char) const st = lds0 + (g % kBsRing) * kBsStage;
#pragma unroll
                    for (int k16 = 0; k16 < 4; ++k16) {
#pragma unroll
                        for (int mi = 0; mi < 2; ++mi) {
                            if (narrow && mi != half)
                                continue;
                            TW_LDS(unsigned char) const q = st + lane_a[mi] + k16 * 2048;
                            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))q);
                            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(q + 512));
                            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                            acc[mi] = E::mfma(u32x4{l2.x, l2.y, h2.x, h2.y}, bq[s][k16], acc[mi]);
                        }
                    }
                }
                ++g;
            }
        }
        if (!active)
            continue;
        // ---- the block's 64 x 32 product: alpha, bias, activation, one rounding; through the
        // wave's stage as [column][row m]; 16-byte stores of whole columns
        const int m0 = m_lo + mb * kBsRows;
        const int m_end = min(m0 + kBsRows, m_hi);
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[mi][e] = p.alpha * acc[mi][e] + out_bias;
        }
        if (p.act != TW_ACT_NONE) { // (tested once per block, not per element)
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) {
                float v[16];
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    v[e] = acc[mi][e];
                tw_activate_all(v, p.act);
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[mi][e] = v[e];
            }
        }
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                uint32_t h[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    h[e] = E::to_bits(tw_fp32_value(acc[mi][r4 * 4 + e]));
                u32x2 pk;
                pk.x = h[0] | (h[1] << 16);
                pk.y = h[2] | (h[3] << 16);
                *reinterpret_cast<u32x2 *>(cst + j * kBsCPitch + mi * 32 + (lane >> 5) * 4 + r4 * 8) = pk;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // (what follows is worked out from the lane number anew in every block: kept across the
        // loop, these few values cost registers the widest instantiation does not have, and a
        // value parked in scratch memory comes back behind a wait for every store in flight)
        int ln = lane;
        asm volatile("" : "+v"(ln));
#pragma unroll
        for (int q = 0; q < 4; ++q) { // 32 columns x 8 chunks of 8 rows
            const int idx = ln + q * 64;
            const int jj = idx >> 3, ch = idx & 7;
            const int col = __shfl(out_col, jj);
            const u32x2 lo = *reinterpret_cast<const u32x2 *>(cst + jj * kBsCPitch + ch * 8);
            const u32x2 hi = *reinterpret_cast<const u32x2 *>(cst + jj * kBsCPitch + ch * 8 + 4);
            const int m = m0 + ch * 8;
            if (jj < cnt && (!narrow || (ch >> 2) == half))
                store_chunk(C + (int64_t)col * p.ldc + m, u32x4{lo.x, lo.y, hi.x, hi.y}, m, m_end,
                            p.store_through != 0);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the stage is free again
    }

    // ---- TW_PRUNED_ZERO: the pruned columns of this unit's share of the tiles receive act(bias)
    // on the range's rows
    for (int z = p.n_gemm_u + ui; z < p.n_all_u; z += n_units) {
        const TileDev t = p.tiles[z - p.n_gemm_u];
        const int chunks = (m_hi - m_lo + 7) / 8;
        for (int i = tid; i < t.n_pruned * chunks; i += 64 * kBsMulWaves) {
            const int jz = i / chunks, ch = i - jz * chunks;
            const int c = t.col0 + p.pruned_n[t.pn_off + jz];
            const uint32_t hb = E::to_bits(tw_finish(0.0f, p.bias, c, p.act));
            const uint32_t w = hb | (hb << 16);
            store_chunk(C + (int64_t)c * p.ldc + m_lo + ch * 8, u32x4{w, w, w, w}, m_lo + ch * 8, m_hi,
                        p.store_through != 0);
        }
    }
}

bool bs_takes(const tw_plan *plan, int64_t lda, int64_t ldc, bool reads_c)
{
    if (reads_c || plan->n_units == 0 || plan->n_pipe_units == 0)
        return false;
    // A is addressed through a buffer descriptor with 32-bit offsets
    if ((uint64_t)plan->K * (uint64_t)lda * 2u >= (1ull << 32))
        return false;
    (void)ldc;
    return plan->max_k_pad <= kBsMaxSteps * kBlockK;
}

// ranges of rows of A a launch is cut into: as many as give every compute unit `per_cu`
// workgroups, a multiple of the number of dies (a range then lives on one die) or a divisor of it
int bs_ranges(const tw_plan *plan, int M, int per_cu)
{
    if (per_cu <= 0)
        per_cu = kBsPerCu;
    const int row_units = (M + 31) / 32;
    int r = std::max(1, plan->cu_count * per_cu / std::max(1, plan->n_units));
    r = std::min(r, std::max(1, row_units / 2)); // at least 64 rows a range
    if (r >= kXcd)
        r = r / kXcd * kXcd;
    else
        r = r >= 4 ? 4 : (r >= 2 ? 2 : 1);
    return r;
}

// share of the compute units' workgroup slots the launch fills, over a whole number of rounds
double bs_fill(const tw_plan *plan, int M)
{
    const int64_t wgs = (int64_t)plan->n_units * bs_ranges(plan, M, 0);
    const int64_t slots = (int64_t)plan->cu_count * kBsPerCu;
    const int64_t rounds = (wgs + slots - 1) / slots;
    return (double)wgs / (double)(rounds * slots);
}

template <int DT, int NS> static int launch_bs_t(const tw_plan *plan, const GemmArgs &a, int per_cu, hipStream_t s)
{
    const int n_ranges = bs_ranges(plan, a.M, per_cu);
    const int affine = n_ranges >= kXcd;
    const int64_t grid = affine ? (int64_t)kXcd * plan->n_units * (n_ranges / kXcd) : (int64_t)n_ranges * plan->n_units;
    if (grid > (int64_t)0x7fffffff)
        return fail(TW_ERR_SHAPE, "%lld workgroups (M=%d): a launch takes at most %lld", (long long)grid, a.M,
                    (long long)(int64_t)0x7fffffff);
    hipLaunchKernelGGL((tw_gemm_bs_kernel<DT, NS>), dim3((unsigned)grid), dim3(64 * kBsWaves), 0, s, a, plan->n_units,
                       n_ranges, (a.M + 31) / 32, affine, (uint32_t)((uint64_t)plan->K * (uint64_t)a.lda * 2u), 0u);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

int launch_bs(const tw_plan *plan, const GemmArgs &a, int per_cu, hipStream_t s)
{
    // (per_cu <= 0: as many workgroups per compute unit as the kernel is built for)
    const int ns = std::max(1, plan->max_k_pad / kBlockK);
    const int pc = per_cu > 0 ? per_cu : kBsPerCu;
    if (plan->dtype == TW_F16) {
        switch (ns) {
        case 1:
        case 2:
            return launch_bs_t<TW_F16, 2>(plan, a, pc, s);
        default:
            return launch_bs_t<TW_F16, 3>(plan, a, pc, s);
        }
    }
    switch (ns) {
    case 1:
    case 2:
        return launch_bs_t<TW_BF16, 2>(plan, a, pc, s);
    default:
        return launch_bs_t<TW_BF16, 3>(plan, a, pc, s);
    }
}

} // namespace tw
