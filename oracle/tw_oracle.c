/*
 * CPU oracle for the tile-wise-sparse (TW) GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the host-side algorithm of the reference's
 * perf driver so that the HIP engine can be checked against it.  It is linked
 * or loaded only by the test-suite, by the smoke check and by the benchmark's
 * CPU-baseline leg; the product library never calls into it.
 *
 * Every function names the reference lines it follows
 * (paths relative to the reference tree).
 *
 * How each function is pinned (the reference ships no golden vectors for this
 * path, so the pins are closed forms, known answers and independent forms):
 *   ora_mask_to_offsets      closed form r[i]=kept[i]-i, hand known answer
 *                            [0,1,0,0,1,1,0,1] -> [1,3,3,4], round trip.
 *   ora_random_shuffle/      checked against the real std::random_shuffle of
 *   ora_mask_gen             libstdc++ on the same rand() stream
 *                            (oracle/shuffle_check.cpp).
 *   ora_tile_partition       README known answers (768,384)->3 tiles of
 *                            256/128 and (3072,1536)->12 tiles.
 *   ora_gen_cutlass_weight,  brute force against the element-wise definition
 *   ora_gen_stream_weight    B*mask and (B*mask)[kept_k][:,kept_n].
 *   ora_f32_to_f16/bf16      numpy.float16 cast; bf16 = RNE on the top 16 bits
 *                            (exhaustive against a second formulation).
 *   ora_stream_gemm_nn       two independent forms (gather->GEMM->scatter vs
 *                            dense matmul on B*mask) and numpy.matmul.
 *   ora_mask_dense           numpy.matmul of x and kernel*mask.
 *   ora_checkout             hand cases incl. 0/0 (NaN compares false).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* 0/1 keep vector -> relative offsets  kept[i] - i.
 * Follows Pruning/BERT/utils/MyHook.py:66-74 (convert_mask_to_offset) and the
 * last loop of StreamMaskedGEMM/perf/basic_nn.cu:713-716 (mask_gen).
 * Returns the number of kept entries. */
int ora_mask_to_offsets(const uint8_t *mask, int n, int32_t *offsets)
{
    int kept = 0;
    for (int idx = 0; idx < n; ++idx) {
        if (mask[idx] == 1) {
            offsets[kept] = idx - kept;
            ++kept;
        }
    }
    return kept;
}

/* relative offsets -> absolute kept indices (inverse of the above; the device
 * kernels of the reference evaluate i + mask[i] on the fly,
 * basic_nn.cu:154,191 and cutlass/tile_iterator.h:724-734). */
void ora_offsets_to_kept(const int32_t *offsets, int n_kept, int32_t *kept)
{
    for (int i = 0; i < n_kept; ++i)
        kept[i] = offsets[i] + i;
}

/* ------------------------------------------------------------------------- */
/* std::random_shuffle as libstdc++ implements it when no generator is given:
 *   for (i = first + 1; i != last; ++i) iter_swap(i, first + rand() % ((i - first) + 1));
 * The reference calls it at basic_nn.cu:706 (mask_gen) with glibc rand(),
 * which is never seeded (default seed 1). */
void ora_random_shuffle(int32_t *v, int n)
{
    for (int i = 1; i < n; ++i) {
        int j = rand() % (i + 1);
        int32_t t = v[i];
        v[i] = v[j];
        v[j] = t;
    }
}

static int cmp_i32(const void *a, const void *b)
{
    int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
    return (x > y) - (x < y);
}

/* mask_gen(N, N_pruned): basic_nn.cu:697-718.  Identity permutation, shuffle,
 * keep the first n_kept, sort ascending, store kept[i]-i.  Consumes n-1 calls
 * of rand().  offsets must hold n_kept ints. */
void ora_mask_gen(int n, int n_kept, int32_t *offsets)
{
    int32_t *perm = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n > 0 ? n : 1));
    for (int i = 0; i < n; ++i)
        perm[i] = i;
    ora_random_shuffle(perm, n);
    qsort(perm, (size_t)n_kept, sizeof(int32_t), cmp_i32);
    for (int i = 0; i < n_kept; ++i)
        offsets[i] = perm[i] - i;
    free(perm);
}

/* init_matrix: basic_nn.cu:612-621.  U(-0.5,0.5) from rand(). */
void ora_init_matrix(float *mat, int rows, int cols)
{
    for (int i = 0; i < rows; ++i)
        for (int j = 0; j < cols; ++j)
            mat[(size_t)i * cols + j] = (float)((double)rand() / (double)(RAND_MAX / 1) - 0.5);
}

void ora_srand(unsigned seed) { srand(seed); }

/* transpose_matrix(dst, src, M, N): basic_nn.cu:641-650.
 * dst is M x N row-major, src is N x M row-major. */
void ora_transpose_matrix(float *dst, const float *src, int M, int N)
{
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j)
            dst[(size_t)i * N + j] = src[(size_t)j * M + i];
}

/* ------------------------------------------------------------------------- */
/* Tile partition of TestCutlassGemm: basic_nn.cu:836-885.
 * n_dim is the reference's N_dim (=128, :73).  Arrays must hold block_num
 * entries; returns block_num = ceil(N_pruned / n_dim). */
int ora_tile_partition(int M, int N, int K, int N_pruned, int K_pruned, int n_dim,
                       int32_t *N_ori, int32_t *N_cal, int32_t *K_cal,
                       int32_t *off_B, int32_t *off_C)
{
    int block_num = (N_pruned + n_dim - 1) / n_dim;
    for (int i = 0; i < block_num; ++i)
        K_cal[i] = K_pruned;
    int n_ori_off = 0, n_cal_off = 0;
    for (int i = 0; i < block_num - 1; ++i) {
        N_ori[i] = N / block_num;
        N_cal[i] = n_dim;
        n_ori_off += N_ori[i];
        n_cal_off += N_cal[i];
    }
    N_ori[block_num - 1] = N - n_ori_off;
    N_cal[block_num - 1] = N_pruned - n_cal_off;
    int offset_B = 0, offset_C = 0;
    for (int i = 0; i < block_num; ++i) {
        off_B[i] = offset_B;
        off_C[i] = offset_C;
        offset_B += K * N_ori[i];
        offset_C += M * N_ori[i];
    }
    return block_num;
}

/* ------------------------------------------------------------------------- */
/* gen_cutlass_weight: basic_nn.cu:743-755.  Masked-dense weight B (.) mask,
 * row-major [K,N]; dst must be zero-initialised by the caller (:827). */
void ora_gen_cutlass_weight(float *dst, const float *src, int K, int N,
                            const int32_t *mask_k, const int32_t *mask_n,
                            int pruned_K, int pruned_N, int offset)
{
    (void)K;
    for (int i = 0; i < pruned_K; ++i)
        for (int j = 0; j < pruned_N; ++j) {
            int idx_col = mask_k[i] + i;
            int idx_row = mask_n[j] + j + offset;
            dst[(size_t)idx_col * N + idx_row] = src[(size_t)idx_col * N + idx_row];
        }
}

/* gen_masked_stream_weight: basic_nn.cu:757-769.  Compaction: tile becomes a
 * dense K_t x N_t block, column-major with leading dimension K, starting at
 * element offset*K. dst must be zero-initialised (:828). */
void ora_gen_stream_weight(float *dst, const float *src, int K, int N,
                           const int32_t *mask_k, const int32_t *mask_n,
                           int pruned_K, int pruned_N, int offset)
{
    for (int i = 0; i < pruned_K; ++i)
        for (int j = 0; j < pruned_N; ++j) {
            int idx_col = mask_k[i] + i;
            int idx_row = mask_n[j] + j + offset;
            dst[(size_t)(j + offset) * K + i] = src[(size_t)idx_col * N + idx_row];
        }
}

/* ------------------------------------------------------------------------- */
/* fp32 -> fp16 / bf16 bit patterns, round to nearest even: the arithmetic of
 * `d_array[idx] = (T)s_array[idx]` in float_to_half, basic_nn.cu:122-137
 * (without its off-by-one bound). */
uint16_t ora_f32_to_f16_bits(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mant = x & 0x007FFFFFu;
    int32_t exp = (int32_t)((x >> 23) & 0xFF);
    if (exp == 0xFF) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (mant ? (0x0200u | (mant >> 13)) : 0));
    int32_t e = exp - 127 + 15;
    if (e >= 0x1F)
        return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10)
            return (uint16_t)sign;
        mant |= 0x00800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half_m = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_m & 1)))
            ++half_m;
        return (uint16_t)(sign | half_m);
    }
    uint32_t half_m = mant >> 13;
    uint32_t rem = mant & 0x1FFFu;
    uint32_t h = (uint32_t)(e << 10) | half_m;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1)))
        ++h; /* carries into the exponent correctly, up to inf */
    return (uint16_t)(sign | h);
}

float ora_f16_bits_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1F;
    uint32_t mant = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (mant == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                ++e;
                mant <<= 1;
            } while (!(mant & 0x400u));
            mant &= 0x3FFu;
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | (mant << 13);
        }
    } else if (exp == 0x1F) {
        x = sign | 0x7F800000u | (mant << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

uint16_t ora_f32_to_bf16_bits(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7F800000u) == 0x7F800000u && (x & 0x007FFFFFu))
        return (uint16_t)((x >> 16) | 0x0040u); /* quiet the nan */
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

float ora_bf16_bits_to_f32(uint16_t h)
{
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void ora_cast_f32(const float *src, uint16_t *dst, int64_t n, int to_bf16)
{
    for (int64_t i = 0; i < n; ++i)
        dst[i] = to_bf16 ? ora_f32_to_bf16_bits(src[i]) : ora_f32_to_f16_bits(src[i]);
}

void ora_uncast_f32(const uint16_t *src, float *dst, int64_t n, int from_bf16)
{
    for (int64_t i = 0; i < n; ++i)
        dst[i] = from_bf16 ? ora_bf16_bits_to_f32(src[i]) : ora_f16_bits_to_f32(src[i]);
}

/* ------------------------------------------------------------------------- */
/* deleteRow / insertRow: basic_nn.cu:141-157 and :178-194.
 * Row gather dst[i][j] = src[i + mask[i]][j] and scatter. */
void ora_delete_row(const float *matrix, float *matrix_2, int rows, int columns,
                    const int32_t *mask)
{
    for (int i = 0; i < rows; ++i)
        memcpy(matrix_2 + (size_t)i * columns,
               matrix + (size_t)(i + mask[i]) * columns, sizeof(float) * (size_t)columns);
}

void ora_insert_row(float *matrix, const float *matrix_2, int rows, int columns,
                    const int32_t *mask)
{
    for (int i = 0; i < rows; ++i)
        memcpy(matrix + (size_t)(i + mask[i]) * columns,
               matrix_2 + (size_t)i * columns, sizeof(float) * (size_t)columns);
}

/* Column-major GEMM  C[M x N] = alpha * A[M x K] * B[K x N] + beta * C, fp32
 * accumulate in double for a stable reference (the reference kernel's own
 * arithmetic is fp16; the engine's is fp32-accumulate, compared with a
 * tolerance). lda/ldb/ldc are column strides. */
static void colmajor_gemm(int M, int N, int K, float alpha, const float *A, int lda,
                          const float *B, int ldb, float beta, float *C, int ldc)
{
    double *acc = (double *)malloc(sizeof(double) * (size_t)(M > 0 ? M : 1));
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m)
            acc[m] = 0.0;
        for (int k = 0; k < K; ++k) {
            double b = (double)B[(size_t)n * ldb + k];
            if (b == 0.0)
                continue;
            const float *a = A + (size_t)k * lda;
            for (int m = 0; m < M; ++m)
                acc[m] += (double)a[m] * b;
        }
        for (int m = 0; m < M; ++m) {
            float *c = C + (size_t)n * ldc + m;
            double v = (double)alpha * acc[m];
            if (beta != 0.0f) /* source is read only when beta != 0: cutlass/gemm/linear_scaling.h:106-110 */
                v += (double)beta * (double)*c;
            *c = (float)v;
        }
    }
    free(acc);
}

/* Stream_Gemm_NN_reference: basic_nn.cu:450-503.  Per tile: gather the kept
 * K rows of A (column-major M x K, so a "row" of the K x M view), gather the
 * kept C columns, dense GEMM with the compacted tile (column-major, ld = K),
 * scatter back.  A: [K][M], B_stream: a5 layout, C: [N][M].  mask_k/mask_n are
 * arrays of per-tile pointers to relative offsets.  Pruned C columns are left
 * untouched, as in the reference. */
void ora_stream_gemm_nn(int M, int N, int K, float alpha, const float *A,
                        const float *B, float beta, float *C, int block_num,
                        const int32_t *N_cal, const int32_t *K_cal,
                        const int32_t *const *mask_n, const int32_t *const *mask_k,
                        const int64_t *off_B, const int64_t *off_C)
{
    (void)N;
    float *A_2 = (float *)malloc(sizeof(float) * (size_t)M * (size_t)(K > 0 ? K : 1));
    float *C_2 = NULL;
    for (int bn = 0; bn < block_num; ++bn) {
        int nc = N_cal[bn], kc = K_cal[bn];
        C_2 = (float *)realloc(C_2, sizeof(float) * (size_t)M * (size_t)(nc > 0 ? nc : 1));
        ora_delete_row(A, A_2, kc, M, mask_k[bn]);
        ora_delete_row(C + off_C[bn], C_2, nc, M, mask_n[bn]);
        colmajor_gemm(M, nc, kc, alpha, A_2, M, B + off_B[bn], K, beta, C_2, M);
        ora_insert_row(C + off_C[bn], C_2, nc, M, mask_n[bn]);
    }
    free(A_2);
    free(C_2);
}

/* mask_dense: Pruning/BERT/utils/modeling.py:992-1007.
 * y[M,N] = x[M,K] @ (kernel[K,N] * mask[K,N]) + bias[N], all row-major fp32.
 * bias may be NULL.  Scalar triple loop, double accumulation. */
void ora_mask_dense(const float *x, const float *kernel, const uint8_t *mask,
                    const float *bias, float *y, int M, int K, int N)
{
    double *acc = (double *)malloc(sizeof(double) * (size_t)(N > 0 ? N : 1));
    for (int m = 0; m < M; ++m) {
        for (int n = 0; n < N; ++n)
            acc[n] = 0.0;
        for (int k = 0; k < K; ++k) {
            double xv = (double)x[(size_t)m * K + k];
            const float *w = kernel + (size_t)k * N;
            const uint8_t *mk = mask + (size_t)k * N;
            for (int n = 0; n < N; ++n)
                if (mk[n])
                    acc[n] += xv * (double)w[n];
        }
        for (int n = 0; n < N; ++n)
            y[(size_t)m * N + n] = (float)(acc[n] + (bias ? (double)bias[n] : 0.0));
    }
    free(acc);
}

/* checkout: basic_nn.cu:771-798.  Counts the elements for which
 *   v1/v2 > 1+err || v2/v1 > 1+err || |v2-v1| > err
 * host_cutlass is M x N row-major; host_reference is read transposed when
 * trans != 0.  0/0 is NaN and compares false, exactly as in the reference. */
int64_t ora_checkout(const float *host_cutlass, const float *host_reference,
                     int M, int N, int trans, double err)
{
    int64_t errors = 0;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float v1 = trans ? host_reference[(size_t)j * M + i]
                             : host_reference[(size_t)i * N + j];
            float v2 = host_cutlass[(size_t)i * N + j];
            if (v1 / v2 > (1 + err) || v2 / v1 > (1 + err) || fabsf(v2 - v1) > err)
                ++errors;
        }
    return errors;
}
