// LSTM gate arithmetic behind the TW GEMM of the NMT configuration: the gate pre-activations
// come out of tw_gemm(_ex) as a K-major [4H][M] matrix, the new hidden state goes straight into
// the K-major A of the next time step.  Elementwise, HBM-bound: 18 bytes per (unit, row).
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

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }

// One thread per 8 consecutive rows m of one hidden unit n.
__global__ void __launch_bounds__(256)
    lstm_gates_kernel(int M, int H, int dtype, const uint16_t *gates, int64_t ldg, float forget_bias,
                      const float *c_prev, int64_t ldcp, float *c_new, int64_t ldcn, uint16_t *h_new,
                      int64_t ldh)
{
    const int cpr = (M + 7) >> 3;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)H * cpr)
        return;
    const int n = (int)(idx / cpr);
    const int m0 = (int)(idx - (int64_t)n * cpr) << 3;
    const int cnt = min(8, M - m0);
    uint16_t g[4][8];
    float c[8];
    if (cnt == 8) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            *reinterpret_cast<uint4 *>(g[q]) =
                *reinterpret_cast<const uint4 *>(gates + ((int64_t)q * H + n) * ldg + m0);
#pragma unroll
        for (int e = 0; e < 8; e += 4)
            *reinterpret_cast<float4 *>(c + e) =
                *reinterpret_cast<const float4 *>(c_prev + (int64_t)n * ldcp + m0 + e);
    } else {
        for (int e = 0; e < cnt; ++e) {
            for (int q = 0; q < 4; ++q)
                g[q][e] = gates[((int64_t)q * H + n) * ldg + m0 + e];
            c[e] = c_prev[(int64_t)n * ldcp + m0 + e];
        }
    }
    uint16_t h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        if (e < cnt) {
            const float i = from16(g[0][e], dtype), j = from16(g[1][e], dtype);
            const float f = from16(g[2][e], dtype), o = from16(g[3][e], dtype);
            const float cn = c[e] * sigmoidf(f + forget_bias) + sigmoidf(i) * tanhf(j);
            c[e] = cn;
            h[e] = to16(tanhf(cn) * sigmoidf(o), dtype);
        }
    }
    if (cnt == 8) {
#pragma unroll
        for (int e = 0; e < 8; e += 4)
            *reinterpret_cast<float4 *>(c_new + (int64_t)n * ldcn + m0 + e) =
                *reinterpret_cast<const float4 *>(c + e);
        *reinterpret_cast<uint4 *>(h_new + (int64_t)n * ldh + m0) = *reinterpret_cast<const uint4 *>(h);
    } else {
        for (int e = 0; e < cnt; ++e) {
            c_new[(int64_t)n * ldcn + m0 + e] = c[e];
            h_new[(int64_t)n * ldh + m0 + e] = h[e];
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
    const int64_t n = (int64_t)H * ((M + 7) / 8);
    hipLaunchKernelGGL(lstm_gates_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, M, H, dtype, (const uint16_t *)gates, ldg, forget_bias,
                       c_prev, ldc_prev, c_new, ldc_new, (uint16_t *)h_new, ldh);
    TW_HIP(hipGetLastError());
    return TW_OK;
}
