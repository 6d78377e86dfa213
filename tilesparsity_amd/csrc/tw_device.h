// Device-side helpers shared by the GEMM kernels of libtwgemm: element types and MFMA wrappers,
// the output store, the fused epilogue's arithmetic, the unit descriptor fetch.
#pragma once

#include "tw_internal.h"

#include <cstddef>

namespace tw {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define TW_LDS(T) __attribute__((address_space(3))) T *
#define TW_GLOBAL(T) __attribute__((address_space(1))) T *

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
// the same for a handful of values with the test of `act` outside the loop over them
template <int N> __device__ __forceinline__ void tw_activate_all(float (&v)[N], int act)
{
    if (act == TW_ACT_RELU) {
#pragma unroll
        for (int e = 0; e < N; ++e)
            v[e] = tw_activate(v[e], TW_ACT_RELU);
    } else if (act == TW_ACT_GELU) {
#pragma unroll
        for (int e = 0; e < N; ++e)
            v[e] = tw_activate(v[e], TW_ACT_GELU);
    } else if (act == TW_ACT_TANH) {
#pragma unroll
        for (int e = 0; e < N; ++e)
            v[e] = tw_activate(v[e], TW_ACT_TANH);
    }
}
// The value of an output element is rounded to fp32 before it is rounded to 16 bits, in every
// kernel: left to itself the compiler turns "multiply, add, convert" into one fused instruction
// with a single rounding in some epilogues and not in others, and the kernels then differ in the
// last bit of about one element in twenty thousand.
__device__ __forceinline__ float tw_fp32_value(float v)
{
    asm volatile("" : "+v"(v));
    return v;
}
// alpha*acc + beta*C is already in `v`: adds the bias of column c and applies the activation
__device__ __forceinline__ float tw_finish(float v, const float *bias, int c, int act)
{
    if (bias)
        v += bias[c];
    return tw_activate(v, act);
}

// Piece `uv` of the unit table: unit uv / n_split, its columns [j * w, (j + 1) * w) with
// w = 32 * piece_nb and j = uv % n_split.  A piece beyond the unit's columns keeps valid
// offsets and has n_cnt == 0: it runs like any other and stores nothing.  The descriptor is
// workgroup-uniform and ends up in scalar registers.
__device__ __forceinline__ UnitDev load_unit(const GemmArgs &p, int uv)
{
    static_assert(sizeof(UnitDev) == 48, "UnitDev is read as 12 words");
    const int ui = uv / p.n_split;
    int32_t w[12];
    if (p.n_arg_units) {
        // from the kernel-argument segment: scalar loads, no global round trip
        const auto *ka = (const __attribute__((address_space(4))) int32_t *)
            __builtin_amdgcn_kernarg_segment_ptr();
#pragma unroll
        for (int i = 0; i < 12; ++i)
            w[i] = ka[offsetof(GemmArgs, arg_units) / 4 + ui * 12 + i];
    } else {
        // the address is workgroup-uniform and the table is constant: scalar loads
        const auto *gu = (const __attribute__((address_space(4))) int32_t *)(uintptr_t)(p.units + ui);
#pragma unroll
        for (int i = 0; i < 12; ++i)
            w[i] = gu[i];
    }
#pragma unroll
    for (int i = 0; i < 12; ++i)
        w[i] = __builtin_amdgcn_readfirstlane(w[i]);
    UnitDev u;
    __builtin_memcpy(&u, w, sizeof(UnitDev));
    if (p.n_split > 1) {
        const int j = uv - ui * p.n_split;
        const int bps = p.piece_nb; // 32-column blocks per piece
        const int nb = min(max(u.nb_cnt - j * bps, 0), bps);
        const int nc = min(max(u.n_cnt - j * bps * kMfmaN, 0), bps * kMfmaN);
        if (nb > 0) {
            u.nb0 += j * bps;
            u.kn_off += j * bps * kMfmaN;
        }
        u.nb_cnt = nb;
        u.n_cnt = nc;
    }
    return u;
}

// Workgroup barrier for hand-overs through LDS only: waits for this wave's LDS operations, not
// for its global loads, stores or atomics in flight (which __syncthreads() would do for stores
// and atomics), so prefetched loads, the item's output stores and the ticket atomic keep flying.
#define TW_LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

} // namespace tw
