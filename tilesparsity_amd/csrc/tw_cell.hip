// LSTM gate arithmetic behind the TW GEMM of the NMT configuration: the gate pre-activations
// come out of tw_gemm(_ex) as a K-major [4H][M] matrix, the new hidden state goes straight into
// the K-major A of the next time step.  Elementwise, 18 bytes per (unit, row): at the sizes of a time step (M = 128, H = 1024: 2.4 MB)
// the launch itself is most of its time.
#include "tw_internal.h"

#include <cstddef>
#include <cstring>

namespace tw {
namespace {

__device__ __forceinline__ float from16(uint16_t b, int dtype)
{
    if (dtype == TW_F16)
        return (float)__builtin_bit_cast(_Float16, b);
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}

__device__ __forceinline__ uint16_t to16(float f, int dtype)
{
    if (dtype == TW_F16)
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)((u >> 16) | 0x40u); // NaN stays NaN
    u += 0x7FFFu + ((u >> 16) & 1u);          // round to nearest even
    return (uint16_t)(u >> 16);
}

// sigmoid and tanh through the hardware exponential and reciprocal (about 1 ulp each): exact
// limits at +-inf, ~1e-6 relative error in between, far below the 16-bit rounding of h
__device__ __forceinline__ float sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float tanh_fast(float x)
{
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * x) + 1.0f);
}

// One thread per EPT consecutive rows m of one hidden unit n.  The two paths (a full group of
// EPT rows: vector loads and stores; the ragged end of M: one row at a time) share no arrays:
// with common staging arrays and a run-time row count the compiled kernel took four times as long.
constexpr int EPT = 4;

__device__ __forceinline__ void cell_update(float i, float j, float f, float o, float forget_bias,
                                            float &c, float &h)
{
    c = c * sigmoidf(f + forget_bias) + sigmoidf(i) * tanh_fast(j);
    h = tanh_fast(c) * sigmoidf(o);
}

__global__ void __launch_bounds__(256)
    lstm_gates_kernel(int M, int H, int dtype, const uint16_t *gates, int64_t ldg, float forget_bias,
                      const float *c_prev, int64_t ldcp, float *c_new, int64_t ldcn, uint16_t *h_new,
                      int64_t ldh)
{
    const int cpr = (M + EPT - 1) / EPT;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)H * cpr)
        return;
    const int n = (int)(idx / cpr);
    const int m0 = (int)(idx - (int64_t)n * cpr) * EPT;
    const uint16_t *const g0 = gates + (int64_t)n * ldg + m0;
    const int64_t gate_stride = (int64_t)H * ldg;
    if (m0 + EPT <= M) {
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const u16x4 gi = *reinterpret_cast<const u16x4 *>(g0);
        const u16x4 gj = *reinterpret_cast<const u16x4 *>(g0 + gate_stride);
        const u16x4 gf = *reinterpret_cast<const u16x4 *>(g0 + 2 * gate_stride);
        const u16x4 go = *reinterpret_cast<const u16x4 *>(g0 + 3 * gate_stride);
        f32x4 c = *reinterpret_cast<const f32x4 *>(c_prev + (int64_t)n * ldcp + m0);
        u16x4 h;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            float ce = c[e], he;
            cell_update(from16(gi[e], dtype), from16(gj[e], dtype), from16(gf[e], dtype),
                        from16(go[e], dtype), forget_bias, ce, he);
            c[e] = ce;
            h[e] = to16(he, dtype);
        }
        *reinterpret_cast<f32x4 *>(c_new + (int64_t)n * ldcn + m0) = c;
        *reinterpret_cast<u16x4 *>(h_new + (int64_t)n * ldh + m0) = h;
    } else {
        for (int e = 0; m0 + e < M; ++e) {
            float ce = c_prev[(int64_t)n * ldcp + m0 + e], he;
            cell_update(from16(g0[e], dtype), from16(g0[gate_stride + e], dtype),
                        from16(g0[2 * gate_stride + e], dtype), from16(g0[3 * gate_stride + e], dtype),
                        forget_bias, ce, he);
            c_new[(int64_t)n * ldcn + m0 + e] = ce;
            h_new[(int64_t)n * ldh + m0 + e] = to16(he, dtype);
        }
    }
}

// ---------------------------------------------------------------------------------
// One LSTM time step in one launch: the gate GEMM of a tile-wise plan and the cell arithmetic,
// for a handful of rows (the batch of a decoding step).  The i, j, f, o pre-activations of a
// hidden unit are columns h, H + h, 2H + h, 3H + h of the GEMM, four different tiles with four
// kept-row lists, so a workgroup takes 32 hidden units x 32 rows m and runs four K loops side
// by side: wave w multiplies gate w / 2 and every second step of 64 kept rows (w % 2), two steps
// at a time out of one register set, A turned through the wave's own piece of LDS as in the
// skinny GEMM kernel.  The eight partial products meet in LDS; a thread then owns two rows of
// one hidden unit, adds its 4 x 2 partial sums in a fixed order, adds the bias and applies the
// cell in fp32: the gate matrix never goes to memory and is never rounded to 16 bits.
//   work:  workgroup (x, y): hidden units 32 x .. 32 x + 31, rows 32 y .. 32 y + 31
//   table: entry 4 x + gate of the kernel arguments describes the 32-column block of that gate
//          (its offset depends on the workgroup and wave numbers alone, so it arrives with the
//          other arguments)
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
#define TW_LDS(T) __attribute__((address_space(3))) T *
#define TW_GLOBAL(T) __attribute__((address_space(1))) T *

template <int DT> __device__ __forceinline__ f32x16 mfma16(u32x4 a, u32x4 b, f32x16 c)
{
    if (DT == TW_F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

struct LstmBlk {
    int32_t kk_off;      // the tile's kept-K list in the padded array
    int32_t k_kept;      // kept rows of the tile (steps of 64: rounded up)
    int64_t b_first;     // byte offset of the block's first weight fragment
    int64_t step_b;      // bytes from one step's fragments to the next
};
constexpr int kLstmMaxBlks = 128;        // 4 gates x 32 blocks of 32 hidden units: H <= 1024
constexpr int kLstmWaves = 8;
constexpr int kLstmStage = 2 * 64 * 64;  // bytes per wave: two steps of 64 rows k x 32 rows m
constexpr int kLstmPitch = 36;           // floats per column of a partial product
static_assert(32 * kLstmPitch * 4 <= kLstmStage, "a partial product reuses the wave's stage");

struct LstmArgs {
    const void *A;
    const int32_t *kept_k;
    const void *Bp;
    const float *bias;
    const float *c_prev;
    float *c_new;
    void *h_new;
    int64_t lda, ldcp, ldcn, ldh;
    int32_t M, H;
    float forget_bias;
    int32_t pad_;
    LstmBlk blk[kLstmMaxBlks];
};
static_assert(sizeof(LstmArgs) <= 4096, "kernel arguments");

template <int DT>
__global__ void __launch_bounds__(64 * kLstmWaves, 1) tw_lstm_step_kernel(const LstmArgs p)
{
    __shared__ __align__(16) unsigned char smem[kLstmWaves * kLstmStage];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int gate = wave >> 1, kh = wave & 1;
    const int hb = blockIdx.x, m0 = blockIdx.y * 32;
    // the block of this wave's gate, and the arguments the first loads need, asked for at once
    uintptr_t A_i = (uintptr_t)p.A, kk_i = (uintptr_t)p.kept_k, Bp_i = (uintptr_t)p.Bp;
    int64_t lda = p.lda;
    int M = p.M;
    LstmBlk blk;
    {
        const auto *ka = (const __attribute__((address_space(4))) int32_t *)__builtin_amdgcn_kernarg_segment_ptr();
        int32_t w[6];
#pragma unroll
        for (int i = 0; i < 6; ++i)
            w[i] = ka[offsetof(LstmArgs, blk) / 4 + (hb * 4 + gate) * 6 + i];
#pragma unroll
        for (int i = 0; i < 6; ++i)
            asm volatile("" : "+s"(w[i]));
        asm volatile("" : "+s"(A_i), "+s"(kk_i), "+s"(Bp_i), "+s"(lda), "+s"(M));
        __builtin_memcpy(&blk, w, sizeof(LstmBlk));
    }
    static_assert(sizeof(LstmBlk) == 24, "LstmBlk is read as 6 words");
    TW_GLOBAL(const uint16_t) const A = (TW_GLOBAL(const uint16_t))A_i;
    TW_GLOBAL(const int32_t) const kept_k = (TW_GLOBAL(const int32_t))kk_i;
    TW_GLOBAL(const unsigned char) const Bp = (TW_GLOBAL(const unsigned char))Bp_i;
    const int nsteps = (blk.k_kept + kBlockK - 1) / kBlockK;
    unsigned char *const stage = smem + wave * kLstmStage;

    struct Numbers {
        int row[2][4];
    };
    struct Loads {
        u32x4 a[2][4], b[2][4];
    };
    TW_GLOBAL(const unsigned char) const bsrc = Bp + blk.b_first + lane * 16;
    const int ch = lane & 3, row16 = lane >> 2;
    // nothing on the way to the operands is conditional (exact wait counts): a chunk of rows past
    // M is fetched from the row block's first chunk, a second step past the end repeats the first
    TW_GLOBAL(const uint16_t) const a_lane = A + m0 + (m0 + ch * 8 < M ? ch * 8 : 0);
    constexpr int kStride = 2;           // this wave's steps: kh, kh + 2, ...
    constexpr int kPair = 2 * kStride;   // a pair: steps s and s + 2
    auto numbers = [&](int s) {
        Numbers n;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int st = s + t * kStride < nsteps ? s + t * kStride : s;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                n.row[t][i] = kept_k[blk.kk_off + st * kBlockK + i * 16 + row16];
        }
        return n;
    };
    auto issue = [&](int s, const Numbers &n, Loads &l) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int st = s + t * kStride < nsteps ? s + t * kStride : s;
#pragma unroll
            for (int k16 = 0; k16 < 4; ++k16)
                l.b[t][k16] = *(TW_GLOBAL(const u32x4))(bsrc + st * blk.step_b + k16 * 1024);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                l.a[t][i] = *(TW_GLOBAL(const u32x4))(a_lane + (int64_t)n.row[t][i] * lda);
    };
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        acc[r] = 0.0f;
    const int L = lane & 15;
    const int pair_e = (lane >> 5) * 4 + (L >> 2);
    const int lane_b = ((lane >> 4) & 1) * 32 + (L & 3) * 8;
    const uint32_t r_first = (uint32_t)((pair_e >> 2) * 8 + (pair_e & 3));
    // (a list of kept rows is padded to whole steps with row 0: what was fetched for the padding
    // is replaced by zeros here, so that no value of a row the tile does not keep reaches a product)
    const int k_lim = blk.k_kept - row16;
    auto multiply = [&](int s, const Loads &l) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int k0 = (s + t * kStride) * kBlockK;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t keep = k0 + i * 16 < k_lim ? 0xFFFFFFFFu : 0u;
                const u32x4 v = l.a[t][i];
                *reinterpret_cast<u32x4 *>(stage + (t * 64 + i * 16 + row16) * 64 + ch * 16) =
                    u32x4{v.x & keep, v.y & keep, v.z & keep, v.w & keep};
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        TW_LDS(unsigned char) lds_lane = (TW_LDS(unsigned char))stage + lane_b;
#pragma unroll
        for (int t = 0; t < 2; ++t)
            if (s + t * kStride < nsteps) {
#pragma unroll
                for (int k16 = 0; k16 < 4; ++k16) {
                    const uint32_t r_lo = t * 64 + r_first + k16 * 16, r_hi = r_lo + 4;
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(lds_lane + r_lo * 64));
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(lds_lane + r_hi * 64));
                    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                    acc = mfma16<DT>(u32x4{l2.x, l2.y, h2.x, h2.y}, l.b[t][k16], acc);
                }
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read before the next steps overwrite it
    };
    int s = kh;
    Loads l0, l1;
    Numbers n;
    if (s < nsteps) {
        n = numbers(s);
        issue(s, n, l0);
        if (s + kPair < nsteps)
            n = numbers(s + kPair);
    }
    // behind the first operands on their way: what the cell needs of this thread's two rows of
    // hidden unit hb * 32 + tid / 16
    const int ju = tid >> 4, m2 = (tid & 15) * 2;
    const int hu = hb * 32 + ju;
    const bool row_ok = m0 + m2 < p.M;
    float bias4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (p.bias) {
        TW_GLOBAL(const float) const gb = (TW_GLOBAL(const float))(uintptr_t)p.bias;
#pragma unroll
        for (int g = 0; g < 4; ++g)
            bias4[g] = gb[g * p.H + hu];
    }
    f32x2 c_old = f32x2{0.0f, 0.0f};
    if (row_ok)
        c_old = *(TW_GLOBAL(const f32x2))(uintptr_t)(p.c_prev + (int64_t)hu * p.ldcp + m0 + m2);
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
    // the partial product of this wave: column lane % 32, rows r4 * 8 + (lane / 32) * 4 + e
    float *const part = reinterpret_cast<float *>(stage);
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        float *const dst = part + (lane & 31) * kLstmPitch + r4 * 8 + (lane >> 5) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            dst[e] = acc[r4 * 4 + e];
    }
    __syncthreads();
    if (!row_ok)
        return;
    float pre[4][2];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const float *const lo = reinterpret_cast<const float *>(smem + (2 * g) * kLstmStage) + ju * kLstmPitch + m2;
        const float *const hi = reinterpret_cast<const float *>(smem + (2 * g + 1) * kLstmStage) + ju * kLstmPitch + m2;
#pragma unroll
        for (int e = 0; e < 2; ++e)
            pre[g][e] = (lo[e] + hi[e]) + bias4[g];
    }
    float c2[2] = {c_old.x, c_old.y}, h2[2];
#pragma unroll
    for (int e = 0; e < 2; ++e)
        cell_update(pre[0][e], pre[1][e], pre[2][e], pre[3][e], p.forget_bias, c2[e], h2[e]);
    float *const cdst = p.c_new + (int64_t)hu * p.ldcn + m0 + m2;
    uint16_t *const hdst = reinterpret_cast<uint16_t *>(p.h_new) + (int64_t)hu * p.ldh + m0 + m2;
    if (m0 + m2 + 1 < p.M) {
        *reinterpret_cast<f32x2 *>(cdst) = f32x2{c2[0], c2[1]};
        *reinterpret_cast<uint32_t *>(hdst) = (uint32_t)to16(h2[0], DT) | ((uint32_t)to16(h2[1], DT) << 16);
    } else {
        cdst[0] = c2[0];
        hdst[0] = to16(h2[0], DT);
    }
}


// ---------------------------------------------------------------------------------
// T time steps of the LSTM in one launch (tw_lstm_steps): the recurrence of the NMT cells
// (Pruning/NMT/nmt/model_helper.py:400-402 builds the cell once and dynamic_rnn applies it step
// after step with the same kernel) as a persistent kernel.  Same decomposition as the single
// step above (workgroup = 32 hidden units x 32 rows, wave = one gate and every second step of 64
// kept rows), but the weight fragments, the row offsets, the bias and the cell state of a
// workgroup are fetched once and stay in registers for all T steps; per step a workgroup reads
// its rows of A_t = [x_t ; h_(t-1)], multiplies, applies the cell and writes its piece of h_t into
// the rows of A_(t+1).  No barrier between the steps: the data is its own flag.
//   hand-over: a launch before this one fills the rows of h of A_1 .. A_(T-1) (rows m below M)
//           with the 16-bit pattern 0xFFFF, which no step ever stores (a NaN of that pattern is
//           stored as 0xFFFE).  A wave that needs rows of h loads them and looks at what came: a
//           piece that still shows the pattern has not been written yet, and the wave loads its
//           rows again.  So a step costs one store's way to memory and one load's way back, not
//           the round trips of a counter on top of them.  The rows of x of A_(t+1) do not wait:
//           the steps of a tile's kept rows that hold nothing else are fetched with the rows of h
//           of A_t and multiplied before the wave looks for h_t.
//   coherence: h crosses from one die to another between two steps.  Its stores write through
//           (sc0 sc1) and the loads of steps that hold rows of h bypass the die's L2 (sc0 sc1), so
//           no cache is written back or invalidated inside the launch.
//   bounds: the number of loads a wave spends on one step's rows is bounded.  A wave that runs out
//           (the launch does not fit the chip next to whatever else runs there, so some
//           workgroup never started) sets the status word, stops looking and runs its remaining
//           steps on whatever it reads; the host reports the launch as failed.
//   edges:  A_t is addressed through a buffer descriptor; the padding of a list of kept rows and
//           rows m beyond M get an offset beyond the buffer, for which the hardware delivers
//           zeros.  Elements m >= M inside a 16-byte piece are the caller's and are not looked at.
constexpr int kSeqSteps = 4; // steps of 64 kept rows a wave holds in registers: tiles of at most 512 kept rows
constexpr int kSeqRsrcFlags = 0x00020000;
constexpr int kSeqAuxCoherent = 1 | 16; // sc0 sc1
constexpr uint32_t kSeqUnwritten = 0xFFFFu; // 16-bit fill pattern of rows of h that no step has stored yet

struct LstmSeqArgs {
    const void *A;
    const int32_t *kept_k;
    const void *Bp;
    const float *bias;
    float *c;
    int32_t *status; // set to 1 by a wave that gave up
    int64_t lda, a_step, ldc;
    int32_t M, H, K, T;
    float forget_bias;
    int32_t spin_limit;
    uint32_t a_bytes; // K * lda * 2
    int32_t pad_;
    LstmBlk blk[kLstmMaxBlks];
};
static_assert(sizeof(LstmSeqArgs) <= 4096, "kernel arguments");

// RB rows m of A per workgroup (32 is what the launch uses).  LOOK false: without the first look at
// one word per writing workgroup (the fall-back path alone; TW_OPT_LSTM_LOOK = 0).
template <int DT, int RB, bool LOOK>
__global__ void __launch_bounds__(64 * kLstmWaves, 1) tw_lstm_steps_kernel(const LstmSeqArgs p)
{
    static_assert(RB == 32 || RB == 16, "rows of a workgroup");
    constexpr int LPS = RB / 8;       // 16-byte loads per lane and step of 64 kept rows
    constexpr int RPL = kBlockK / LPS; // kept rows a load of the wave covers
    constexpr int PITCH = RB * 2;     // bytes of a staged row
    constexpr int STEPB = kBlockK * PITCH;
    constexpr int RPT = RB / 16;      // rows of a hidden unit a thread applies the cell to
    __shared__ __align__(16) unsigned char smem[kLstmWaves * kLstmStage];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int gate = wave >> 1, kh = wave & 1;
    const int hb = blockIdx.x, m0 = blockIdx.y * RB;
    const LstmBlk blk = p.blk[hb * 4 + gate];
    const int nsteps = (blk.k_kept + kBlockK - 1) / kBlockK;
    unsigned char *const stage = smem + wave * kLstmStage;

    // ---- what stays for all T steps: weight fragments and row offsets of this wave's steps
    // kh, kh + 2, ... (a step the tile does not have repeats the tile's first and is skipped)
    const int ch = lane % LPS, rowl = lane / LPS; // this lane's 16-byte chunk of a row, its row of a load
    const bool m_ok = m0 + ch * 8 < p.M;
    u32x4 bq[kSeqSteps][4];
    uint32_t voff[kSeqSteps][LPS];
    uint32_t h_loads = 0; // bit i * LPS + r: load r of step i fetches a row of h
    {
        TW_GLOBAL(const unsigned char) const bsrc = (TW_GLOBAL(const unsigned char))p.Bp + blk.b_first + lane * 16;
        int rows[kSeqSteps][LPS];
#pragma unroll
        for (int i = 0; i < kSeqSteps; ++i) {
            const int s = kh + 2 * i, sc = s < nsteps ? s : 0;
#pragma unroll
            for (int k16 = 0; k16 < 4; ++k16)
                bq[i][k16] = *(TW_GLOBAL(const u32x4))(bsrc + sc * blk.step_b + k16 * 1024);
#pragma unroll
            for (int r = 0; r < LPS; ++r)
                rows[i][r] = p.kept_k[blk.kk_off + sc * kBlockK + r * RPL + rowl]; // the list is padded: in bounds
        }
#pragma unroll
        for (int i = 0; i < kSeqSteps; ++i)
#pragma unroll
            for (int r = 0; r < LPS; ++r) {
                const int kk = (kh + 2 * i) * kBlockK + r * RPL + rowl;
                voff[i][r] = (kk < blk.k_kept && m_ok)
                                 ? (uint32_t)rows[i][r] * ((uint32_t)p.lda * 2u) + (uint32_t)(m0 + ch * 8) * 2u
                                 : 0xFFFFFFF0u;
                if (kk < blk.k_kept && m_ok && rows[i][r] >= p.K - p.H)
                    h_loads |= 1u << (i * LPS + r);
            }
    }
    // the elements of this lane's 16-byte piece that lie below M, as masks of its four words
    uint32_t below_m[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const int m = m0 + ch * 8 + 2 * d;
        below_m[d] = (m < p.M ? 0xFFFFu : 0u) | (m + 1 < p.M ? 0xFFFF0000u : 0u);
    }
    const int my_steps = nsteps > kh ? (nsteps - kh + 1) / 2 : 0; // <= kSeqSteps (host check)
    // The first n_pre of this wave's steps hold rows of x only (a list of kept rows ascends, and
    // the rows of x come first in A): they do not depend on the step before, so they are fetched
    // and multiplied while the workgroup waits at the barrier.
    int n_pre = 0;
#pragma unroll
    for (int i = 0; i < kSeqSteps; ++i) {
        const int s = kh + 2 * i;
        if (s < nsteps) {
            const int last = min(s * kBlockK + kBlockK - 1, blk.k_kept - 1);
            if (n_pre == i && p.kept_k[blk.kk_off + last] < p.K - p.H)
                n_pre = i + 1;
        }
    }
    n_pre = __builtin_amdgcn_readfirstlane(n_pre);
    // the cell's share of this thread: RPT rows of hidden unit hb * 32 + tid / 16
    const int ju = tid >> 4, mt = (tid & 15) * RPT;
    const int hu = hb * 32 + ju;
    bool row_ok[RPT];
#pragma unroll
    for (int e = 0; e < RPT; ++e)
        row_ok[e] = m0 + mt + e < p.M;
    float bias4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (p.bias) {
#pragma unroll
        for (int g = 0; g < 4; ++g)
            bias4[g] = p.bias[g * p.H + hu];
    }
    float c2[RPT];
#pragma unroll
    for (int e = 0; e < RPT; ++e)
        c2[e] = row_ok[e] ? p.c[(int64_t)hu * p.ldc + m0 + mt + e] : 0.0f;

    // this lane's place in a staged step for the transposed reads: row (lane / 32) * 8 + L / 4 of a
    // group of 16 kept rows, 8 bytes at row m (lane / 16 % 2) * 16 + (L % 4) * 4; with 16 rows m
    // the lanes of the upper 16 read what the lower 16 read (their products are never used)
    const int L = lane & 15;
    const int pair_e = (lane >> 5) * 4 + (L >> 2);
    const int lane_b = (RB == 32 ? ((lane >> 4) & 1) * 32 : 0) + (L & 3) * 8;
    const uint32_t r_first = (uint32_t)((pair_e >> 2) * 8 + (pair_e & 3));
    float *const part = reinterpret_cast<float *>(stage);
    const uint16_t *const A0 = reinterpret_cast<const uint16_t *>(p.A);

    u32x4 av[kSeqSteps][LPS];
    f32x16 acc;
    auto clear = [&]() {
#pragma unroll
        for (int e = 0; e < 16; ++e)
            acc[e] = 0.0f;
    };
    // the rows of this wave's steps [lo, hi) of A_t; `coherent`: past the die's L2
    auto load_steps = [&](int t, int lo, int hi, bool coherent) {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t *>(A0 + (int64_t)t * p.a_step), 0, (int)p.a_bytes, kSeqRsrcFlags);
#pragma unroll
        for (int i = 0; i < kSeqSteps; ++i)
            if (i >= lo && i < hi) {
#pragma unroll
                for (int r = 0; r < LPS; ++r)
                    av[i][r] = coherent ? __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff[i][r], 0, kSeqAuxCoherent))
                                        : __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff[i][r], 0, 0));
            }
    };
    // multiplies them: a step through one half of the wave's stage (the halves in turn, so that a
    // step's rows are written while the step before is still being read)
    auto multiply_steps = [&](int lo, int hi) {
#pragma unroll
        for (int i = 0; i < kSeqSteps; ++i)
            if (i >= lo && i < hi) {
                unsigned char *const half = stage + (i & 1) * STEPB;
#pragma unroll
                for (int r = 0; r < LPS; ++r)
                    *reinterpret_cast<u32x4 *>(half + (r * RPL + rowl) * PITCH + ch * 16) = av[i][r];
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                TW_LDS(unsigned char) lds_lane = (TW_LDS(unsigned char))half + lane_b;
#pragma unroll
                for (int k16 = 0; k16 < 4; ++k16) {
                    const uint32_t r_lo = r_first + k16 * 16, r_hi = r_lo + 4;
                    const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(lds_lane + r_lo * PITCH));
                    const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TW_LDS(s16x4))(lds_lane + r_hi * PITCH));
                    const u32x2 l2 = __builtin_bit_cast(u32x2, lo4), h2 = __builtin_bit_cast(u32x2, hi4);
                    acc = mfma16<DT>(u32x4{l2.x, l2.y, h2.x, h2.y}, bq[i][k16], acc);
                }
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };

    // the word lane l looks at before it fetches rows of h: the last one workgroup (l, this row
    // block) stores, hidden unit 32 l + 31, the last two rows m of the block below M
    const int probe_m = m0 + ((min(p.M - m0, RB) - 1) & ~1);
    const uint32_t probe_off = lane < (int)gridDim.x
                                   ? (uint32_t)(p.K - p.H + 32 * lane + 31) * ((uint32_t)p.lda * 2u) + (uint32_t)probe_m * 2u
                                   : 0xFFFFFFF0u; // (beyond the buffer: zeros)
    const uint32_t probe_mask = probe_m + 1 < p.M ? 0xFFFFFFFFu : 0xFFFFu;
    // whether a piece of this wave's rows of h of a step still shows the fill pattern
    auto unwritten = [&]() {
        uint32_t bad = 0;
#pragma unroll
        for (int i = 0; i < kSeqSteps; ++i)
            if (i >= n_pre && i < my_steps) {
#pragma unroll
            for (int r = 0; r < LPS; ++r) {
                const uint32_t w[4] = {av[i][r].x, av[i][r].y, av[i][r].z, av[i][r].w};
                uint32_t hit = 0;
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t x = ~(w[d] & below_m[d]); // a 16-bit half of zeros: all ones below M
                    hit |= (x - 0x00010001u) & ~x & 0x80008000u;
                }
                bad |= (h_loads >> (i * LPS + r)) & 1u ? hit : 0u;
            }
            }
        return __builtin_amdgcn_ballot_w64(bad != 0) != 0;
    };

    clear();
    load_steps(0, 0, n_pre, false);
    multiply_steps(0, n_pre);
    bool gave_up = false;
    for (int t = 0; t < p.T; ++t) {
        // ---- the steps that hold rows of h (of the step before).  For t > 0 the wave
        // first looks at one word of every workgroup that writes rows it needs (the last one
        // each of them stores, past the caches) until none shows the fill pattern, then fetches
        // its rows through the L2 like any others (the 16 workgroups of a die ask for the same
        // lines), and falls back to loads past the L2 for what still shows the pattern: a line
        // another workgroup of the die fetched too early.
        bool look = t > 0 && !gave_up && h_loads != 0; // (A_0 holds the caller's h)
        int left = p.spin_limit;
        if (look && LOOK) {
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint16_t *>(A0 + (int64_t)t * p.a_step), 0, (int)p.a_bytes, kSeqRsrcFlags);
            for (;;) {
                if (left <= 0)
                    break;
                --left;
                const uint32_t w = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)probe_off, 0, kSeqAuxCoherent);
                const uint32_t x = ~(w & probe_mask);
                const bool fresh = ((x - 0x00010001u) & ~x & 0x80008000u) != 0;
                if (__builtin_amdgcn_ballot_w64(fresh) == 0)
                    break;
                __builtin_amdgcn_s_sleep(1);
            }
        }
        load_steps(t, n_pre, my_steps, !LOOK && look); // (without the first look: past the caches at once)
        if (look) {
            for (;;) {
                if (left <= 0) {
                    gave_up = true;
                    if (lane == 0)
                        __hip_atomic_store(p.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                if (!unwritten())
                    break;
                --left;
                __builtin_amdgcn_s_sleep(1);
                load_steps(t, n_pre, my_steps, true);
            }
        }
        // the next step's rows of x leave now: they travel while this step is multiplied and
        // the cell applied (together with the rows of h they would only hold those up)
        if (t + 1 < p.T)
            load_steps(t + 1, 0, n_pre, false);
        multiply_steps(n_pre, my_steps);
        // the partial product of this wave: column lane % 32, rows r4 * 8 + (lane / 32) * 4 + e
        // (four rows at a time: they are neighbours in the column, 16-byte aligned)
        typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int r4 = 0; r4 < RB / 8; ++r4)
            *reinterpret_cast<f32x4 *>(part + (lane & 31) * kLstmPitch + r4 * 8 + (lane >> 5) * 4) =
                f32x4{acc[r4 * 4], acc[r4 * 4 + 1], acc[r4 * 4 + 2], acc[r4 * 4 + 3]};
        __syncthreads();
        {
            float pre[4][RPT];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float *const lo = reinterpret_cast<const float *>(smem + (2 * g) * kLstmStage) + ju * kLstmPitch + mt;
                const float *const hi = reinterpret_cast<const float *>(smem + (2 * g + 1) * kLstmStage) + ju * kLstmPitch + mt;
#pragma unroll
                for (int e = 0; e < RPT; ++e)
                    pre[g][e] = (lo[e] + hi[e]) + bias4[g];
            }
            float h2[RPT];
#pragma unroll
            for (int e = 0; e < RPT; ++e)
                cell_update(pre[0][e], pre[1][e], pre[2][e], pre[3][e], p.forget_bias, c2[e], h2[e]);
            // h_t into the rows of A_(t+1) that hold h; written through, for the other dies.  The
            // fill pattern is never stored: it would read as "not written yet".
            uint16_t *const hdst = const_cast<uint16_t *>(A0) + (int64_t)(t + 1) * p.a_step +
                                   (int64_t)(p.K - p.H + hu) * p.lda + m0 + mt;
            uint32_t h16[RPT];
#pragma unroll
            for (int e = 0; e < RPT; ++e) {
                h16[e] = to16(h2[e], DT);
                h16[e] = h16[e] == kSeqUnwritten ? kSeqUnwritten - 1u : h16[e];
            }
            if (RPT == 2 && row_ok[RPT - 1]) {
                const uint32_t w = h16[0] | (h16[RPT - 1] << 16);
                asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"(hdst), "v"(w) : "memory");
            } else if (row_ok[0]) {
                const uint32_t w = h16[0];
                asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(hdst), "v"(w) : "memory");
            }
        }
        if (t + 1 == p.T)
            break;
        // ---- the next step's rows of x, multiplied while h_t travels
        clear();
        __syncthreads(); // the partial sums have been read: the stages may be written again
        multiply_steps(0, n_pre);
    }
#pragma unroll
    for (int e = 0; e < RPT; ++e)
        if (row_ok[e])
            p.c[(int64_t)hu * p.ldc + m0 + mt + e] = c2[e];
}

// Fills the rows of h of A_1 .. A_(T-1), rows m below M, with the pattern tw_lstm_steps_kernel
// takes for "not written yet".  One thread per 16-byte piece (8 rows m) of a row.
__global__ void lstm_mark_unwritten_kernel(uint16_t *A, int64_t lda, int64_t a_step, int M, int H, int K, int T)
{
    const int pieces = (M + 7) / 8;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)(T - 1) * H * pieces)
        return;
    const int pc = (int)(i % pieces);
    const int64_t row = i / pieces;
    uint16_t *const dst = A + (row / H + 1) * a_step + (int64_t)(K - H + row % H) * lda + pc * 8;
    if (pc * 8 + 8 <= M) {
        const uint32_t w = kSeqUnwritten | (kSeqUnwritten << 16);
        *reinterpret_cast<u32x4 *>(dst) = u32x4{w, w, w, w};
    } else {
        for (int e = 0; pc * 8 + e < M; ++e)
            dst[e] = (uint16_t)kSeqUnwritten;
    }
}

// what tw_lstm_step and tw_lstm_steps have in common: whether the fused kernels take the plan
bool lstm_fused_plan(const tw_plan *plan, int H)
{
    bool fused = H % 32 == 0 && H / 32 * 4 <= kLstmMaxBlks && plan->n_units == plan->n_tiles;
    for (int t = 0; t < plan->n_tiles && fused; ++t)
        fused = plan->tile_col0[t] % 32 == 0 && plan->tile_width[t] % 32 == 0 &&
                plan->kept_n_ptr[t + 1] - plan->kept_n_ptr[t] == plan->tile_width[t];
    return fused;
}

void lstm_fill_blocks(const tw_plan *plan, int H, LstmBlk *blk)
{
    for (const UnitDev &u : plan->h_units) {
        // the unit's blocks: columns col0 + 32 nb of C, i.e. gate (col / H), hidden block (col % H) / 32
        for (int nb = 0; nb < u.nb_cnt; ++nb) {
            const int col = u.col0 + 32 * nb;
            LstmBlk &b = blk[(col % H) / 32 * 4 + col / H];
            b.kk_off = u.kk_off;
            b.k_kept = u.k_pad ? u.k_kept : 0;
            b.b_first = u.b_off * 2 + (int64_t)(u.nb0 + nb) * 4096;
            b.step_b = (int64_t)u.nblk * 4096;
        }
    }
}
} // namespace
} // namespace tw

using namespace tw;

extern "C" int tw_lstm_step(const tw_plan *plan, const void *A, int64_t lda, int M, const float *bias,
                            float forget_bias, const float *c_prev, int64_t ldc_prev, float *c_new,
                            int64_t ldc_new, void *h_new, int64_t ldh, void *gates_ws, int64_t ldg,
                            void *stream)
{
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    if (M < 0)
        return fail(TW_ERR_SHAPE, "M=%d", M);
    if (plan->N % 4)
        return fail(TW_ERR_SHAPE, "N=%d is not four gates wide", plan->N);
    const int H = plan->N / 4;
    if (M == 0)
        return TW_OK;
    if (!A || !c_prev || !c_new || !h_new)
        return fail(TW_ERR_NULL, "A, c_prev, c_new or h_new is NULL");
    // what the fused kernel takes: every column kept, tiles that are whole blocks of 32 columns and
    // one work item each, at most 128 blocks in all
    const bool fused = lstm_fused_plan(plan, H);
    if (!fused) {
        if (!gates_ws)
            return fail(TW_ERR_LAYOUT, "this plan needs the two-kernel form (pruned columns, tiles that are no "
                                       "multiple of 32 columns, or H > 1024): pass a gate matrix of 4H x ldg elements");
        tw_epilogue ep;
        ep.bias = bias;
        ep.activation = TW_ACT_NONE;
        int rc = tw_gemm_ex(plan, A, TW_LAYOUT_KMAJOR, lda, gates_ws, TW_LAYOUT_KMAJOR, ldg, M, 1.0f, 0.0f,
                            TW_PRUNED_ZERO, &ep, stream);
        if (rc != TW_OK)
            return rc;
        return tw_lstm_gates(M, H, plan->dtype, gates_ws, ldg, forget_bias, c_prev, ldc_prev, c_new, ldc_new,
                             h_new, ldh, stream);
    }
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    if (dev != plan->device)
        return fail(TW_ERR_DEVICE, "the plan was built on device %d, the current device is %d", plan->device, dev);
    if (lda < M || ldc_prev < M || ldc_new < M || ldh < M)
        return fail(TW_ERR_SHAPE, "leading dimensions %lld %lld %lld %lld must be >= M=%d", (long long)lda,
                    (long long)ldc_prev, (long long)ldc_new, (long long)ldh, M);
    if ((lda & 7) || (ldh & 7) || (ldc_prev & 3) || (ldc_new & 3))
        return fail(TW_ERR_ALIGNMENT, "lda and ldh must be multiples of 8 elements, ldc_prev and ldc_new of 4");
    if (((uintptr_t)A & 15) || ((uintptr_t)h_new & 15) || ((uintptr_t)c_prev & 15) || ((uintptr_t)c_new & 15))
        return fail(TW_ERR_ALIGNMENT, "all buffers must be 16-byte aligned");
    const int64_t row_blocks = ((int64_t)M + 31) / 32;
    if (row_blocks > 65535)
        return fail(TW_ERR_SHAPE, "M=%d: the fused step takes at most %d rows", M, 65535 * 32);
    LstmArgs a;
    std::memset(&a, 0, sizeof a);
    a.A = A;
    a.kept_k = plan->d_kept_k_pad;
    a.Bp = plan->d_Bp;
    a.bias = bias;
    a.c_prev = c_prev;
    a.c_new = c_new;
    a.h_new = h_new;
    a.lda = lda;
    a.ldcp = ldc_prev;
    a.ldcn = ldc_new;
    a.ldh = ldh;
    a.M = M;
    a.H = H;
    a.forget_bias = forget_bias;
    a.pad_ = 0;
    lstm_fill_blocks(plan, H, a.blk);
    if (plan->dtype == TW_F16)
        hipLaunchKernelGGL((tw_lstm_step_kernel<TW_F16>), dim3((unsigned)(H / 32), (unsigned)row_blocks),
                           dim3(64 * kLstmWaves), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((tw_lstm_step_kernel<TW_BF16>), dim3((unsigned)(H / 32), (unsigned)row_blocks),
                           dim3(64 * kLstmWaves), 0, (hipStream_t)stream, a);
    TW_HIP(hipGetLastError());
    return TW_OK;
}

extern "C" int tw_lstm_steps(const tw_plan *plan, int T, void *A, int64_t lda, int64_t a_step, int M,
                             const float *bias, float forget_bias, float *c, int64_t ldc, void *gates_ws,
                             int64_t ldg, void *stream)
{
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    if (T < 0 || M < 0)
        return fail(TW_ERR_SHAPE, "T=%d M=%d", T, M);
    if (plan->N % 4)
        return fail(TW_ERR_SHAPE, "N=%d is not four gates wide", plan->N);
    const int H = plan->N / 4, K = plan->K;
    if (H > K)
        return fail(TW_ERR_SHAPE, "K=%d has no room for the H=%d rows of h", K, H);
    if (T == 0 || M == 0)
        return TW_OK;
    if (!A || !c)
        return fail(TW_ERR_NULL, "A or c is NULL");
    if (lda < M || ldc < M)
        return fail(TW_ERR_SHAPE, "lda=%lld ldc=%lld must be >= M=%d", (long long)lda, (long long)ldc, M);
    if (a_step < (int64_t)K * lda)
        return fail(TW_ERR_SHAPE, "a_step=%lld: consecutive steps' A (K x lda = %lld elements) overlap", (long long)a_step,
                    (long long)K * lda);
    if ((lda & 7) || (a_step & 7) || (ldc & 3))
        return fail(TW_ERR_ALIGNMENT, "lda and a_step must be multiples of 8 elements, ldc of 4");
    if (((uintptr_t)A & 15) || ((uintptr_t)c & 15))
        return fail(TW_ERR_ALIGNMENT, "A and c must be 16-byte aligned");
    int dev = -1;
    TW_HIP(hipGetDevice(&dev));
    if (dev != plan->device)
        return fail(TW_ERR_DEVICE, "the plan was built on device %d, the current device is %d", plan->device, dev);
    uint16_t *const A16 = static_cast<uint16_t *>(A);
    // The persistent kernel: a plan the fused step takes, tiles of at most 512 kept rows, a grid
    // that is resident at once (one workgroup per compute unit), A_t below 4 GiB.  (32 rows of A a
    // workgroup: with 16, which fills the chip on the NMT cell, a workgroup fetches the same
    // number of row pieces of half the size, and a step takes 8.5 us instead of 5.9.)
    const int rb = 32;
    const int64_t row_blocks = ((int64_t)M + rb - 1) / rb;
    const bool persistent = lstm_fused_plan(plan, H) && plan->max_k_pad <= 2 * kSeqSteps * kBlockK &&
                            (int64_t)(H / 32) * row_blocks <= plan->cu_count &&
                            (uint64_t)K * (uint64_t)lda * 2u < (1ull << 32) && T > 1 && plan->d_tickets;
    if (!persistent) {
        // step by step: one launch (or two, through the gate matrix) per time step
        for (int t = 0; t < T; ++t) {
            const int rc = tw_lstm_step(plan, A16 + (int64_t)t * a_step, lda, M, bias, forget_bias, c, ldc, c, ldc,
                                        A16 + (int64_t)(t + 1) * a_step + (int64_t)(K - H) * lda, lda, gates_ws, ldg, stream);
            if (rc != TW_OK)
                return rc;
        }
        return TW_OK;
    }
    LstmSeqArgs a;
    std::memset(&a, 0, sizeof a);
    a.A = A;
    a.kept_k = plan->d_kept_k_pad;
    a.Bp = plan->d_Bp;
    a.bias = bias;
    a.c = c;
    a.status = plan->d_tickets + kTicketInts * kTicketSlots; // the word behind the plan's ticket slots
    a.lda = lda;
    a.a_step = a_step;
    a.ldc = ldc;
    a.M = M;
    a.H = H;
    a.K = K;
    a.T = T;
    a.forget_bias = forget_bias;
    const int limit = get_option(TW_OPT_SPIN_LIMIT);
    a.spin_limit = limit >= 0 ? limit : (1 << 20);
    a.a_bytes = (uint32_t)((uint64_t)K * (uint64_t)lda * 2u);
    lstm_fill_blocks(plan, H, a.blk);
    // the rows of h the steps will hand to each other start out as "not written yet"
    if (T > 1) {
        const int64_t n = (int64_t)(T - 1) * H * ((M + 7) / 8);
        hipLaunchKernelGGL(lstm_mark_unwritten_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                           A16, lda, a_step, M, H, K, T);
    }
    const dim3 grid((unsigned)(H / 32), (unsigned)row_blocks), block(64 * kLstmWaves);
    const bool first_look = get_option(TW_OPT_LSTM_LOOK) != 0;
    if (plan->dtype == TW_F16) {
        if (first_look)
            hipLaunchKernelGGL((tw_lstm_steps_kernel<TW_F16, 32, true>), grid, block, 0, (hipStream_t)stream, a);
        else
            hipLaunchKernelGGL((tw_lstm_steps_kernel<TW_F16, 32, false>), grid, block, 0, (hipStream_t)stream, a);
    } else {
        if (first_look)
            hipLaunchKernelGGL((tw_lstm_steps_kernel<TW_BF16, 32, true>), grid, block, 0, (hipStream_t)stream, a);
        else
            hipLaunchKernelGGL((tw_lstm_steps_kernel<TW_BF16, 32, false>), grid, block, 0, (hipStream_t)stream, a);
    }
    TW_HIP(hipGetLastError());
    return TW_OK;
}

extern "C" int tw_lstm_steps_status(const tw_plan *plan, void *stream)
{
    if (!plan)
        return fail(TW_ERR_NULL, "plan is NULL");
    if (!plan->d_tickets)
        return TW_OK;
    int32_t *const word = plan->d_tickets + kTicketInts * kTicketSlots;
    int32_t v = 0;
    TW_HIP(hipStreamSynchronize((hipStream_t)stream));
    TW_HIP(hipMemcpy(&v, word, sizeof v, hipMemcpyDeviceToHost));
    if (v == 0)
        return TW_OK;
    TW_HIP(hipMemset(word, 0, sizeof v));
    return fail(TW_ERR_DEVICE, "a multi-step LSTM launch of this plan gave up waiting for a step's h (its workgroups were not "
                               "all resident at once); h and c of that call are undefined");
}

extern "C" int tw_lstm_gates(int M, int H, int dtype, const void *gates, int64_t ldg,
                             float forget_bias, const float *c_prev, int64_t ldc_prev, float *c_new,
                             int64_t ldc_new, void *h_new, int64_t ldh, void *stream)
{
    if (dtype != TW_F16 && dtype != TW_BF16)
        return fail(TW_ERR_DTYPE, "dtype %d is neither TW_F16 nor TW_BF16", dtype);
    if (M < 0 || H <= 0)
        return fail(TW_ERR_SHAPE, "M=%d H=%d", M, H);
    if (M == 0)
        return TW_OK;
    if (!gates || !c_prev || !c_new || !h_new)
        return fail(TW_ERR_NULL, "gates, c_prev, c_new or h_new is NULL");
    if (ldg < M || ldc_prev < M || ldc_new < M || ldh < M)
        return fail(TW_ERR_SHAPE, "leading dimensions %lld %lld %lld %lld must be >= M=%d",
                    (long long)ldg, (long long)ldc_prev, (long long)ldc_new, (long long)ldh, M);
    if ((ldg & 7) || (ldh & 7) || (ldc_prev & 3) || (ldc_new & 3))
        return fail(TW_ERR_ALIGNMENT,
                    "ldg and ldh must be multiples of 8 elements, ldc_prev and ldc_new of 4");
    if (((uintptr_t)gates & 15) || ((uintptr_t)h_new & 15) || ((uintptr_t)c_prev & 15) ||
        ((uintptr_t)c_new & 15))
        return fail(TW_ERR_ALIGNMENT, "all buffers must be 16-byte aligned");
    const int64_t n = (int64_t)H * ((M + EPT - 1) / EPT);
    hipLaunchKernelGGL(lstm_gates_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, M, H, dtype, (const uint16_t *)gates, ldg, forget_bias,
                       c_prev, ldc_prev, c_new, ldc_new, (uint16_t *)h_new, ldh);
    TW_HIP(hipGetLastError());
    return TW_OK;
}
