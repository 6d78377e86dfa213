// LSTM gate arithmetic behind the TW GEMM of the NMT configuration: the gate pre-activations
// come out of tw_gemm(_ex) as a K-major [4H][M] matrix, the new hidden state goes straight into
// the K-major A of the next time step.  Elementwise, 18 bytes per (unit, row): at the sizes of a time step (M = 128, H = 1024: 2.4 MB)
// the launch itself is most of its time.
#include "tw_internal.h"

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

} // namespace
} // namespace tw

using namespace tw;

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
