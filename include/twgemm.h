/*
 * twgemm.h - C ABI of libtwgemm.so, a tile-wise-sparse (TW) GEMM engine for AMD
 * MI355X (gfx950).
 *
 *     C = alpha * A * (B (.) mask) + beta * C
 *
 * A[M,K] dense activations, B[K,N] a TW-pruned weight: B is split into column
 * tiles; every tile keeps its own ascending list of K rows (kept_k) and of
 * columns (kept_n, relative to the tile's first column).  A *plan* owns the
 * tile table, the index lists and the compacted weight in device memory; the
 * caller owns A and C (device memory).
 *
 * This boundary replaces the host code of the reference's perf driver,
 * StreamMaskedGEMM/perf/basic_nn.cu; each entry point names the reference
 * lines it stands in for.  "Relative offsets" are the reference's mask
 * arrays: offset[i] = kept[i] - i.
 *
 * Conventions
 *   - every function returns TW_OK (0) or a negative tw_status; nothing throws
 *     across this boundary; tw_last_error() holds a message for the calling
 *     thread's last failure.
 *   - "host" pointers are ordinary memory, "device" pointers are HIP device
 *     memory of the current device.
 *   - tw_gemm is asynchronous with respect to `stream` (a hipStream_t passed as
 *     void*, NULL = the default stream), allocates nothing and never
 *     synchronises the device.
 */
#ifndef TWGEMM_H
#define TWGEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TWGEMM_VERSION 100 /* major*10000 + minor*100 + patch */

typedef struct tw_plan tw_plan;

typedef enum tw_status {
    TW_OK = 0,
    TW_ERR_NULL = -1,       /* a required pointer is NULL */
    TW_ERR_SHAPE = -2,      /* M < 0, K/N/G <= 0, bad leading dimension ... */
    TW_ERR_TILE_TABLE = -3, /* tiles do not cover [0,N) exactly once, in order */
    TW_ERR_INDEX_LIST = -4, /* list not strictly ascending or out of range */
    TW_ERR_DTYPE = -5,      /* unknown element type */
    TW_ERR_LAYOUT = -6,     /* unknown layout / pruned-column mode */
    TW_ERR_ALIGNMENT = -7,  /* pointer or leading dimension not 16-byte aligned */
    TW_ERR_NOT_TW = -8,     /* the 0/1 mask is not a tile-wise pattern for this G */
    TW_ERR_DEVICE = -9,     /* HIP runtime failure (message has the HIP error) */
    TW_ERR_ALLOC = -10,     /* host or device allocation failed */
    TW_ERR_BUFFER = -11     /* caller-provided buffer too small */
} tw_status;

typedef enum tw_dtype {
    TW_F16 = 0, /* IEEE half in, fp32 accumulate, half out */
    TW_BF16 = 1 /* bfloat16 in, fp32 accumulate, bfloat16 out */
} tw_dtype;

typedef enum tw_layout {
    /* The reference's layout (basic_nn.cu:418,423-425): A is column-major M x K,
     * i.e. element (m,k) at A[k*lda + m]; C is column-major M x N, element (m,n)
     * at C[n*ldc + m].  A gathered K row is one contiguous M-vector. */
    TW_LAYOUT_KMAJOR = 0,
    /* Element (m,k) at A[m*lda + k]; element (m,n) at C[m*ldc + n]. */
    TW_LAYOUT_ROWMAJOR = 1
} tw_layout;

typedef enum tw_pruned_cols {
    /* pruned C columns are never written (the reference's scatter epilogue,
     * cutlass/gemm/mma_epilogue.h:286) */
    TW_PRUNED_UNTOUCHED = 0,
    /* pruned C columns receive beta*C (exact zero when beta == 0), which is
     * what the product with the masked weight yields */
    TW_PRUNED_ZERO = 1
} tw_pruned_cols;

/* ---- library ---------------------------------------------------------------- */

int tw_version(void);
/* Message of the calling thread's most recent failure ("" if none). */
const char *tw_last_error(void);
const char *tw_status_string(int status);

/* ---- integer helpers (host) ---------------------------------------------------- */

/* 0/1 keep vector -> relative offsets kept[i]-i; *n_kept receives the count.
 * offsets must hold n ints.  Replaces convert_mask_to_offset,
 * Pruning/BERT/utils/MyHook.py:66-74, and the tail of mask_gen,
 * basic_nn.cu:713-716.  Any mask byte other than 0 or 1 is TW_ERR_INDEX_LIST. */
int tw_mask_to_offsets(const uint8_t *mask, int n, int32_t *offsets, int *n_kept);

/* Relative offsets -> ascending kept indices (i + offset[i], basic_nn.cu:154).
 * Fails with TW_ERR_INDEX_LIST unless the result is strictly ascending in
 * [0, limit). */
int tw_offsets_to_kept(const int32_t *offsets, int n_kept, int limit, int32_t *kept);

/* Tile partition of TestCutlassGemm, basic_nn.cu:836-885: block_num =
 * ceil(N_pruned/n_dim) tiles of n_dim kept columns over N/block_num original
 * columns (the last tile takes the remainders), K_cal = K_pruned everywhere,
 * off_B = K * sum(N_ori), off_C = M * sum(N_ori).  Arrays must hold max_tiles
 * entries (TW_ERR_BUFFER otherwise).  The reference's cap of 32 tiles (:74,:837)
 * does not apply. */
int tw_tile_partition(int M, int N, int K, int N_pruned, int K_pruned, int n_dim,
                      int max_tiles, int *block_num, int32_t *N_ori, int32_t *N_cal,
                      int32_t *K_cal, int64_t *off_B, int64_t *off_C);

/* ---- plans -------------------------------------------------------------------- */

/* Build a plan from an explicit tile table and index lists (all host memory).
 *   tile_col0[t], tile_width[t]   tiles must cover [0,N) in order, without gaps
 *   kept_k_ptr[n_tiles+1], kept_k_idx[]   CSR-style lists of kept K rows
 *   kept_n_ptr[n_tiles+1], kept_n_idx[]   kept columns relative to tile_col0[t]
 *   B   fp32 row-major [K,N]: the unpruned (or already masked) weight
 * The weight is compacted and cast on the device (round to nearest even).
 * Replaces mask_gen + gen_masked_stream_weight + float_to_half,
 * basic_nn.cu:697-718, 757-769, 122-137, 891-914. */
int tw_plan_create(int K, int N, int dtype, int n_tiles,
                   const int32_t *tile_col0, const int32_t *tile_width,
                   const int32_t *kept_k_ptr, const int32_t *kept_k_idx,
                   const int32_t *kept_n_ptr, const int32_t *kept_n_idx,
                   const float *B, tw_plan **out);

/* The 0 %-sparse plan: tiles of G columns, every row and column kept.  Running
 * tw_gemm on it is the dense baseline of the same kernel (the role of
 * Cutlass_Gemm_NN, basic_nn.cu:315-375, 1006-1007). */
int tw_plan_create_dense(int K, int N, int G, int dtype, const float *B, tw_plan **out);

/* Build a plan from a dense 0/1 mask [K,N] (host, row-major, one byte per
 * element) split every G original columns: the mask -> kept lists -> offsets ->
 * compaction pre-pass runs as integer HIP kernels.  A row of a tile is kept iff
 * any of its mask bytes is non-zero, a column likewise; a mask that is not the
 * outer product of the two per tile is TW_ERR_NOT_TW.  This is the hand-off
 * from the pruning side (mask-o of mask_dense, Pruning/BERT/utils/modeling.py:1000;
 * exportPrunedModel, Pruning/BERT/utils/MyHook.py:54-89). */
int tw_plan_from_mask(int K, int N, int G, int dtype, const uint8_t *mask,
                      const float *B, tw_plan **out);

/* The same for an explicit tile table (tiles cover [0,N) in order, without gaps), e.g. the
 * tiles that end after every G kept columns of tiled_wise_2d
 * (Pruning/VGG/prune_algo.py:76-88; tw_tiles_every_g_kept_columns below). */
int tw_plan_from_mask_tiles(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                            const int32_t *tile_width, const uint8_t *mask, const float *B,
                            tw_plan **out);

/* The same for a mask whose tiles need not be rows x columns: a tile keeps every row and every
 * column that holds a kept element, and the elements the mask drops inside that cover are stored
 * as zeros, so the product is exactly A (B (.) mask) for ANY mask.  This runs the reference's
 * mixed masks (tiled_wise_1d_mix / tiled_wise_2d_mix, Pruning/VGG/prune_algo.py:151-193: a TW
 * mask plus a small element-wise remainder) on the same kernel; each remainder element costs
 * the tile one more row (and column) of matrix-core work. */
int tw_plan_from_mask_cover(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                            const int32_t *tile_width, const uint8_t *mask, const float *B,
                            tw_plan **out);

/* The same pre-pass on DEVICE operands: mask (K x N bytes) and B (fp32, row-major) are device
 * memory, e.g. the masks tw_prune_* leave on the device and a weight that already lives there, so
 * nothing but the tile table, the list lengths and the lists' host copies crosses the host
 * boundary.  cover != 0 as tw_plan_from_mask_cover, else as tw_plan_from_mask_tiles.  Every
 * kernel and copy of the build runs on `stream` (a hipStream_t, NULL = the default stream), after
 * whatever produced mask and B on that stream; the call waits for that stream and returns when
 * the plan is complete. */
int tw_plan_from_device_mask(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                             const int32_t *tile_width, const uint8_t *mask, const float *B,
                             int cover, void *stream, tw_plan **out);

/* Build a plan from one layer of the reference's exported pruned model (exportPrunedModel,
 * Pruning/BERT/utils/MyHook.py:54-89): mask_i / mask_o are the relative offsets
 * (convert_mask_to_offset, :66-74) of the n_kept_k kept rows and n_kept_n kept columns, kernel is
 * the compacted weight kernel[mask_i][:, mask_o], fp32 row-major [n_kept_k, n_kept_n] (:80-81);
 * all host memory.  K and N are the layer's unpruned sizes (N is the length of the exported
 * bias; K is not stored in the file: any K above the last kept row gives the same product).
 * The plan has one tile over all columns. */
int tw_plan_from_export(int K, int N, int dtype, int n_kept_k, const int32_t *mask_i,
                        int n_kept_n, const int32_t *mask_o, const float *kernel, tw_plan **out);

/* Build a plan from the operands of the reference's Stream_Gemm_NN
 * (basic_nn.cu:378-393): B_stream is the compacted weight in DEVICE memory in
 * the layout of gen_masked_stream_weight (:757-769; tile t column-major with
 * ld = K at element off_B[t]), already in `dtype`; mask_n[t] / mask_k[t] are
 * DEVICE arrays of N_cal[t] / K_cal[t] relative offsets; off_C[t] = M * first
 * original column of tile t. */
int tw_plan_from_stream_operands(int M, int N, int K, int dtype, const void *B_stream,
                                 int block_num, const int32_t *N_cal, const int32_t *K_cal,
                                 const int32_t *const *mask_n, const int32_t *const *mask_k,
                                 const int64_t *off_B, const int64_t *off_C, tw_plan **out);

/* info[] receives: 0 K, 1 N, 2 dtype, 3 n_tiles, 4 sum K_t, 5 sum N_t,
 * 6 sum K_t*N_t (kept weight elements), 7 packed weight bytes on the device,
 * 8 max K_t, 9 max N_t, 10 number of empty tiles (K_t*N_t == 0),
 * 11 total width of all tiles (== N).  n_info <= 12 entries are written. */
int tw_plan_info(const tw_plan *plan, int64_t *info, int n_info);

/* Read a plan back to host memory for bit-exact checks.  Any pointer may be
 * NULL.  Sizes: tile_col0/tile_width n_tiles; kept_*_ptr n_tiles+1;
 * kept_k_idx/mask_k_rel sum K_t; kept_n_idx/mask_n_rel sum N_t; B_stream K*N
 * 16-bit patterns in the layout of gen_masked_stream_weight (basic_nn.cu:757-769)
 * after the cast of float_to_half (:995), zeros in unused slots. */
int tw_plan_export(const tw_plan *plan, int32_t *tile_col0, int32_t *tile_width,
                   int32_t *kept_k_ptr, int32_t *kept_k_idx, int32_t *mask_k_rel,
                   int32_t *kept_n_ptr, int32_t *kept_n_idx, int32_t *mask_n_rel,
                   uint16_t *B_stream);

int tw_plan_destroy(tw_plan *plan);

/* ---- the GEMM ------------------------------------------------------------------ */

/* C = alpha * A * (B (.) mask) + beta * C through one persistent grouped kernel.
 * Replaces Stream_Gemm_NN (basic_nn.cu:378-445) and the masked kernel it launches
 * per tile (cutlass/gemm/gemm.h:84-100, gemm_mainloop.h:230-338, gathered A load
 * tile_iterator.h:786-816, column-scatter epilogue mma_epilogue.h:174-290).
 *   A, C       device pointers of the plan's dtype, 16-byte aligned
 *   a_layout   TW_LAYOUT_KMAJOR (lda >= M) or TW_LAYOUT_ROWMAJOR (lda >= K)
 *   c_layout   TW_LAYOUT_KMAJOR (ldc >= M) or TW_LAYOUT_ROWMAJOR (ldc >= N)
 *   lda, ldc   in elements, multiples of 8
 *   M          rows of A and C; 0 is a no-op
 *   beta       C is read only when beta != 0, and only on kept columns
 *   pruned_cols  tw_pruned_cols
 * Immutable plan: may be called concurrently from several host threads on distinct streams.  A
 * launch of a kernel that draws work from a queue holds one of the plan's 256 counter slots
 * until it ends: eager launches rotate over 192 of them, launches made while their stream is
 * being captured over the other 64 (a recorded launch keeps its slot for every replay).  So at
 * most 192 eager launches of one plan may be in flight at once, and at most 64 recorded launches
 * of one plan may run at the same time as each other.  Nothing checks this: launch number 193
 * (recorded: 65) shares the counters of a launch that has not ended, and both skip or repeat work
 * items - wrong results, no error.  Synchronise or build a second plan before going beyond. */
int tw_gemm(const tw_plan *plan, const void *A, int a_layout, int64_t lda,
            void *C, int c_layout, int64_t ldc, int M, float alpha, float beta,
            int pruned_cols, void *stream);

/* The same with a fused epilogue: C = act(alpha * A (B (.) mask) + beta * C + bias) on the written
 * columns, i.e. the reference's masked dense layer in one pass (mask_dense,
 * Pruning/BERT/utils/modeling.py:992-1007: matmul(input, kernel * mask) + bias, then the
 * activation).  bias is a device fp32 vector of N entries indexed by the original column (or
 * NULL); the arithmetic is fp32 with one rounding to the 16-bit output.  With TW_PRUNED_ZERO a
 * pruned column receives act(beta * C + bias), as it does in the reference, where a fully masked
 * column still gets its bias.  ep == NULL is tw_gemm. */
#define TW_ACT_NONE 0
#define TW_ACT_RELU 1
#define TW_ACT_GELU 2 /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))), modeling.py:264-277 */
#define TW_ACT_TANH 3
typedef struct tw_epilogue {
    const float *bias;
    int activation;
} tw_epilogue;
int tw_gemm_ex(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C,
               int c_layout, int64_t ldc, int M, float alpha, float beta, int pruned_cols,
               const tw_epilogue *ep, void *stream);

/* Re-arms the work-queue counters of a plan (all 256 slots to zero) with a small kernel on
 * `stream`.  A launch leaves its slot at zero when it ends; one that was aborted mid-flight (a
 * device fault elsewhere in the process, a reset) does not, and the next launch to draw that slot
 * would skip work.  Call it with no launch of the plan in flight.  No counterpart in the
 * reference, whose per-tile launches share no state (basic_nn.cu:408-430). */
int tw_plan_reset(tw_plan *plan, void *stream);

/* tw_gemm_ex for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference (Stream_Gemm_NN creates and destroys 32 streams per call,
 * basic_nn.cu:396-406,440-443).  Same arguments and results as tw_gemm_ex, bit for bit; the only
 * scratch memory the kernels use besides the inputs and outputs - the work-queue counters of the
 * launch - lives in a 256-byte array inside the library's device image, one copy per GPU, held
 * until the process ends.  The call allocates and frees nothing: it clears the counters with a
 * small kernel on `stream`, then launches the GEMM on `stream`.
 *   Limit: a launch of more than 2^31 - 1 work items (tile pieces x row blocks of 128 .. 512 rows)
 *   is refused with TW_ERR_SHAPE, as it is by tw_gemm_ex; devices 0..63.
 *   Every call on one GPU shares that GPU's counters: calls that overlap on one GPU (two streams,
 *   two host threads, a graph replay next to an eager call) race and give wrong results.
 *   Serialise them, or use tw_gemm_ex, whose plans carry 256 counter slots of their own (192 for
 *   eager launches, 64 for recorded ones; see tw_gemm).
 *   The once-per-device set-up (the array's device address, kernel attributes) runs when a plan is
 *   built, so a call made while `stream` is being captured does nothing capture forbids. */
int tw_gemm_static(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C,
                   int c_layout, int64_t ldc, int M, float alpha, float beta, int pruned_cols,
                   const tw_epilogue *ep, void *stream);

/* tw_gemm_ex for row-major operands at the speed of the K-major kernels.  The reference's Python
 * operator multiplies a row-major x[M,K] into a row-major result (mask_dense,
 * Pruning/BERT/utils/modeling.py:992-1007).  tw_gemm_ex takes such operands as they are when both
 * are row-major, K <= 2128 and beta == 0 (a kernel that keeps a panel of A in LDS), and else
 * through a layout-generic kernel that gathers 2-byte elements.  Here, in those other cases, a row-major A is first turned into
 * its K-major copy and a row-major C is produced K-major and turned back, both in `workspace`
 * (device memory, 16-byte aligned, at least tw_gemm_staged_workspace(plan, M, a_layout, c_layout)
 * bytes: 2 * round_up(M, 64) * (K for a row-major A + N for a row-major C)); one more pass over
 * each staged operand at the memory rate.  C's old values go through the workspace as well
 * whenever the K-major kernel would leave some of them in place (beta != 0, untouched pruned
 * columns, columns no tile covers).  Same arguments, results and errors as tw_gemm_ex; TW_ERR_BUFFER
 * for a workspace that is missing or too small.  Allocates nothing; with both layouts K-major it is
 * tw_gemm_ex.  Calls that share a workspace must not overlap. */
int64_t tw_gemm_staged_workspace(const tw_plan *plan, int M, int a_layout, int c_layout);
int tw_gemm_staged(const tw_plan *plan, const void *A, int a_layout, int64_t lda, void *C,
                   int c_layout, int64_t ldc, int M, float alpha, float beta, int pruned_cols,
                   const tw_epilogue *ep, void *workspace, int64_t workspace_bytes, void *stream);

/* Process-wide tuning switches of tw_gemm / tw_gemm_ex; value -1 restores the automatic choice.
 * The launch configuration is otherwise picked from the plan and M.  The reference fixes its one
 * configuration at compile time (Volta884GemmTraits<..., Shape<32,128,128>, ...>,
 * basic_nn.cu:250-259, and MAX_BLOCK_NUM streams, :73); tests and tuning runs use these switches
 * to cover every kernel shape (bench.py --shape-grid times the automatic choice against each).  A forced shape or piece width that cannot take the plan (a shape
 * narrower than the plan's unit pieces, TW_SHAPE_WIDE aside operands beyond 4 GiB) is ignored.
 *   TW_OPT_SHAPE        one of the TW_SHAPE_* kernels below
 *   TW_OPT_WGS_PER_CU   workgroups launched per compute unit, 1..8
 *   TW_OPT_PIECE        columns of a tile handed out as one work item: 128, 64 or 32
 *   TW_OPT_XCD_QUEUES   1: one work queue per accelerator die, each owning whole row blocks of A
 *                       (the workgroups of a die then share those rows in their L2);
 *                       0: the work items are dealt out over the dies in turn; automatic: 0
 *                       unless nearly every tile keeps nearly every row (a 0 %-sparse plan);
 *                       2: dealt out over the dies in turn, row block after row block (all tiles
 *                       of a row block before the next) instead of tile after tile
 *   TW_OPT_SPIN_LIMIT   loads a wave of tw_lstm_steps spends looking for a step's h before it gives up
 *   TW_OPT_BALANCE      1: row blocks sized per tile where the items would not fill the chip once
 *   TW_OPT_LDS_DMA      0: the 256-row streaming kernels stage their loads through registers
 *                       instead of writing LDS directly (same results, bit for bit)
 *   TW_OPT_LSTM_LOOK    0: a wave of tw_lstm_steps fetches a step's rows of h at once, past the
 *                       caches, and again until they are all there, instead of first looking at
 *                       one word of every workgroup that writes them (same results, slower)
 * Initial values come from the environment variables TWGEMM_SHAPE, TWGEMM_WGS_PER_CU,
 * TWGEMM_PIECE, TWGEMM_XCD_QUEUES, TWGEMM_SPIN_LIMIT, TWGEMM_BALANCE, TWGEMM_LDS_DMA and
 * TWGEMM_LSTM_LOOK, read once. */
#define TW_OPT_SHAPE 0
#define TW_OPT_WGS_PER_CU 1
#define TW_OPT_PIECE 2
#define TW_OPT_XCD_QUEUES 3
#define TW_OPT_SPIN_LIMIT 4 /* loads a wave of tw_lstm_steps spends looking for a step's h before it gives up (default 2^20) */
#define TW_OPT_BALANCE 5 /* 1: a launch whose items would not fill the chip once gives the tiles with more kept rows lower row blocks (multiples of 64 rows); 0 and automatic: every tile in row blocks of the kernel's full height (the benchmark shapes run no faster with 1) */
#define TW_OPT_LDS_DMA 6 /* the 256-row streaming kernels (256 x 128, 256 x 64) with loads that write LDS directly: 0 never; 1 and automatic: wherever those shapes run */
#define TW_OPT_LSTM_LOOK 7 /* tw_lstm_steps: 1 and automatic: a wave looks at one word per writing workgroup before it fetches a step's rows of h; 0: it fetches the rows themselves until none shows the fill pattern */
#define TW_N_OPTIONS 8
#define TW_SHAPE_WIDE 0    /* 256 x 128 items, 64-bit row addressing (operands beyond 4 GiB) */
#define TW_SHAPE_128x128 1 /* wave-specialised, 128 rows x 128 columns, two workgroups per CU */
#define TW_SHAPE_512x64 2  /* wave-specialised, 512 x 64: tiles of at most 64 kept columns (forced only: 256 x 64 is ahead) */
#define TW_SHAPE_128x64 3  /* wave-specialised, 128 x 64 */
#define TW_SHAPE_256x128 4 /* wave-specialised, 256 x 128, one workgroup per CU, loads straight into LDS */
#define TW_SHAPE_128x32 5  /* wave-specialised, 128 x 32: skinny M */
#define TW_SHAPE_256x64 6  /* wave-specialised, 256 x 64, loads straight into LDS */
#define TW_SHAPE_AS64 7    /* A-stationary, 64 rows of all K in LDS: K up to 1064, beta == 0 */
#define TW_SHAPE_AS32 8    /* A-stationary, 32 rows: K up to 2128, beta == 0 */
#define TW_SHAPE_SKINNY 9  /* 64 rows x 32 columns per workgroup, the kept rows split over its waves: few rows of A */
#define TW_SHAPE_BS 10     /* weight-stationary: a unit's packed weight in registers, A streamed: tiles of at most 192 kept rows, beta == 0 */
#define TW_N_SHAPES 11
/* What a K-major launch of `plan` on M rows would run with, under the options in force:
 * choice[0] the TW_SHAPE_* kernel, [1] the columns of a unit piece, [2] workgroups per compute
 * unit, [3] 1 for one work queue per die.  (No counterpart in the reference, whose kernel is
 * fixed at compile time, basic_nn.cu:250-259; benchmarks name the kernel they timed with it.) */
int tw_gemm_choice(const tw_plan *plan, int M, int64_t lda, int64_t ldc, float beta, int32_t *choice);
int tw_set_option(int option, int value);

/* One-shot drop-in for Stream_Gemm_NN (basic_nn.cu:378-393), same argument
 * meaning: A column-major M x K (lda = M), B the compacted stream weight, C
 * column-major M x N (ldc = M), all DEVICE memory of `dtype`; mask_n/mask_k host
 * arrays of device pointers to relative offsets.  Builds a transient plan,
 * runs tw_gemm on `stream`, synchronises that stream and frees the plan. */
int tw_stream_gemm_nn(int M, int N, int K, int dtype, float alpha, const void *A,
                      const void *B, float beta, void *C, int block_num,
                      const int32_t *N_cal, const int32_t *K_cal,
                      const int32_t *const *mask_n, const int32_t *const *mask_k,
                      const int64_t *off_B, const int64_t *off_C, void *stream);

/* Elementwise fp32 -> dtype cast on the device, round to nearest even
 * (float_to_half, basic_nn.cu:122-137, without its off-by-one bound). */
int tw_cast_f32(const float *src, void *dst, int64_t n, int dtype, void *stream);

/* Row gather / scatter of the reference's in-binary oracle, on the device, for
 * 16-bit elements: dst[i][j] = src[i + mask[i]][j] (deleteRow,
 * basic_nn.cu:141-157, 196-208) and dst[i + mask[i]][j] = src[i][j] (insertRow,
 * :178-194, 224-236).  mask is a device array of `rows` relative offsets. */
int tw_delete_row(const void *matrix, void *matrix_2, int rows, int columns,
                  const int32_t *mask, void *stream);
int tw_insert_row(void *matrix, const void *matrix_2, int rows, int columns,
                  const int32_t *mask, void *stream);

/* The element-wise remainder of a mixed mask.  The reference's mixed producers
 * (tiled_wise_1d_mix / tiled_wise_2d_mix, tw_mix_fn, Pruning/VGG/prune_algo.py:151-193) keep a
 * tile-wise mask mask0 plus the g1percent largest of the elements mask0 drops; the masked layer
 * is then x @ (kernel * mask) with mask = mask0 | remainder (mask_dense,
 * Pruning/BERT/utils/modeling.py:992-1007).  mask0 runs as a plan (tw_plan_from_mask_tiles);
 * tw_side_create takes the remainder - a K x N byte mask, row-major, non-zero = kept, normally
 * mask & ~mask0 - and the fp32 row-major weight B (both host memory) and keeps its elements
 * column by column on the device, their values rounded to `dtype`.  tw_side_gemm adds
 *   C += alpha * A * (B (.) remainder)
 * to a K-major C (column n at C + n * ldc) from a K-major A, as tw_gemm takes them, with vector
 * multiply-adds in fp32 and one rounding of every touched element of C; columns without a
 * remainder element are not touched.  Run it after the plan's tw_gemm on the same stream.  Any
 * mask at all is a valid remainder (tw_plan_from_mask_cover is the alternative for masks whose
 * remainder clusters in few rows). */
typedef struct tw_side tw_side;
int tw_side_create(int K, int N, int dtype, const uint8_t *mask, const float *B, tw_side **out);
void tw_side_destroy(tw_side *side);
int64_t tw_side_nnz(const tw_side *side); /* elements of the remainder */
int tw_side_gemm(const tw_side *side, const void *A, int64_t lda, void *C, int64_t ldc, int M,
                 float alpha, void *stream);

/* LSTM gate arithmetic of the reference's NMT model, whose cells are TensorFlow 1.x
 * tf.contrib.rnn.BasicLSTMCell (Pruning/NMT/nmt/model_helper.py:400-402; BasicLSTMCell.call in
 * tensorflow/python/ops/rnn_cell_impl.py): with i, j, f, o the four H-wide blocks of the gate
 * pre-activations (inputs and h concatenated, times the masked kernel, plus bias: one
 * tw_gemm_ex with N = 4H),
 *   c_new = c_prev * sigmoid(f + forget_bias) + sigmoid(i) * tanh(j)
 *   h_new = tanh(c_new) * sigmoid(o)
 * All matrices are K-major device buffers: gates [4H][ldg] of `dtype` (the GEMM's C), c_prev and
 * c_new fp32 [H][ld] (may be the same buffer), h_new [H][ldh] of `dtype`, which may point into
 * the rows of the next time step's A that hold h (the cell input is concat([x, h])), so that
 * the recurrence needs no transpose or copy.  fp32 arithmetic, one rounding of h. */
int tw_lstm_gates(int M, int H, int dtype, const void *gates, int64_t ldg, float forget_bias,
                  const float *c_prev, int64_t ldc_prev, float *c_new, int64_t ldc_new,
                  void *h_new, int64_t ldh, void *stream);

/* One LSTM time step in one launch: the masked gate GEMM (N = 4H: the i, j, f, o blocks), the
 * bias and the cell arithmetic of tw_lstm_gates, without the gate matrix going to memory (the
 * pre-activations stay in fp32).  A is the K-major concat([x, h]) of the step, as for tw_gemm;
 * bias fp32 [4H] or NULL; c_prev, c_new, h_new as for tw_lstm_gates.  h_new must not overlap
 * the rows of A this launch reads: keep two A buffers and alternate (the cell is built at
 * Pruning/NMT/nmt/model_helper.py:400-402).
 * The fused kernel takes plans whose tiles keep every column and are multiples of 32 columns
 * wide (at most 128), with H a multiple of 32 up to 1024; for any other plan the call runs
 * tw_gemm_ex (TW_PRUNED_ZERO, bias) into `gates_ws` ([4H][ldg] elements of the plan's dtype)
 * and then tw_lstm_gates, or fails with TW_ERR_LAYOUT when gates_ws is NULL. */
int tw_lstm_step(const tw_plan *plan, const void *A, int64_t lda, int M, const float *bias,
                 float forget_bias, const float *c_prev, int64_t ldc_prev, float *c_new,
                 int64_t ldc_new, void *h_new, int64_t ldh, void *gates_ws, int64_t ldg,
                 void *stream);

/* T time steps of that cell in one launch.  A holds T + 1 K-major matrices [K][lda] at a_step
 * elements from each other: A_t = [x_t ; h_(t-1)], the caller fills the K - H rows of x of A_0 ..
 * A_(T-1) and the H rows of h of A_0; step t reads A_t and writes h_t into the rows of h of
 * A_(t+1), so the call leaves the outputs h_0 .. h_(T-1) in A_1 .. A_T.  c (fp32 [H][ldc]) is
 * the cell state, updated in place.  This is the recurrence the reference's dynamic_rnn runs
 * over the cell of Pruning/NMT/nmt/model_helper.py:400-402, one kernel launch per time step
 * there.
 * Plans the fused step takes, with tiles of at most 512 kept rows and (H / 32) x ceil(M / 32)
 * no larger than the number of compute units, run as ONE persistent launch: weights, row
 * numbers, bias and cell state stay in registers, and the workgroups hand the rows of h to each
 * other through A itself: the call first fills the rows of h of A_1 .. A_(T-1) (rows m < M) with
 * the 16-bit pattern 0xFFFF, a step's stores go through to memory, and a workgroup that needs
 * rows of h_t loads them until none shows the pattern (an h_t whose 16 bits come out as 0xFFFF, a
 * NaN, is stored as 0xFFFE).  That needs every workgroup of the launch resident at once; the
 * number of loads a wave spends looking is bounded (TW_OPT_SPIN_LIMIT), and a launch in which a
 * wave gives up (the GPU was shared with other work) sets a status word and drains:
 * tw_lstm_steps_status then returns TW_ERR_DEVICE.  Every other plan, and T == 1, runs as T
 * calls of tw_lstm_step (gates_ws as there).  Asynchronous on `stream`. */
int tw_lstm_steps(const tw_plan *plan, int T, void *A, int64_t lda, int64_t a_step, int M,
                  const float *bias, float forget_bias, float *c, int64_t ldc, void *gates_ws,
                  int64_t ldg, void *stream);
/* Waits for `stream` and returns TW_ERR_DEVICE if a tw_lstm_steps launch of the plan gave up
 * waiting for a step's h since the last call (and clears that), else TW_OK. */
int tw_lstm_steps_status(const tw_plan *plan, void *stream);

/* ---- TW mask producers ---------------------------------------------------------------
 * The reference derives its masks from importance scores with NumPy: per layer a 2-D score
 * matrix [K,N] (|w|; conv kernels HWIO reshaped to (H*W*I) x O, Pruning/VGG/prune_algo.py:16-24),
 * one threshold over the whole network.  These entry points run that on the GPU and return the
 * same masks bit for bit (every float operation repeats NumPy's, in its order).
 *   scores[l]   device, fp32 row-major [K[l], N[l]]   (sign is irrelevant, only squares are used)
 *   masks[l]    device out, one byte per element, 1 = kept
 * np.percentile computes in the type of its `q`: pass TW_Q_F32 when the reference's caller gives
 * the sparsity as a Python number (float32 arithmetic on float32 norms), TW_Q_F64 when it is a
 * NumPy float64.  All layers are processed on `stream`; the calls return after the masks are
 * complete. */
#define TW_Q_F32 0
#define TW_Q_F64 1

/* tiled_wise_1d (Pruning/VGG/prune_algo.py:114-148; BERT pruning type 7,
 * Pruning/BERT/utils/MyHook.py:226-259): tiles of `granularity` original columns (last one
 * ragged); norm of every tile row / tile width; the `sparsity`-th percentile of all of them is
 * the threshold; a tile row is kept iff its norm is strictly above it.  *threshold (optional)
 * receives the threshold. */
int tw_prune_tiled_wise_1d(int n_layers, const int32_t *K, const int32_t *N,
                           const float *const *scores, double sparsity, int q_type,
                           int granularity, uint8_t *const *masks, double *threshold,
                           void *stream);

/* tiled_wise_2d (Pruning/VGG/prune_algo.py:55-112; BERT type 8, MyHook.py:261-313): columns
 * first (column norm / K against the percentile of all column norms), then tiles that end
 * after every `granularity` kept columns, then tile rows as above on the column-pruned scores
 * (norm / original tile width); mask = rows x columns.  With transform != 0 the percentile
 * used for both steps is 100 - sqrt(10000 - 100*sparsity) (prune_algo.py:61, a float64 whatever
 * q_type says); with 0 it is `sparsity` itself (BERT type 8).  col_masks (optional, device,
 * N[l] bytes each) receive the column masks, from which tw_tiles_every_g_kept_columns gives the
 * tile table; thresholds (optional) receives {columns, rows}. */
int tw_prune_tiled_wise_2d(int n_layers, const int32_t *K, const int32_t *N,
                           const float *const *scores, double sparsity, int q_type, int transform,
                           int granularity, uint8_t *const *masks, uint8_t *const *col_masks,
                           double *thresholds, void *stream);

/* granularity_pruning (Pruning/BERT/utils/MyHook.py:202-214): one layer, tiles of `granularity`
 * columns (N must be a multiple), one threshold per tile: the `sparsity`-th percentile of that
 * tile's K row norms (not divided by the width); a tile row is kept iff its norm is strictly
 * above its tile's threshold. */
int tw_prune_granularity(int K, int N, const float *scores, double sparsity, int q_type,
                         int granularity, uint8_t *mask, void *stream);

/* tw_mix_fn (Pruning/VGG/prune_algo.py:151-179), the second stage of tiled_wise_1d_mix and
 * tiled_wise_2d_mix (:182-193): every element scores sqrt(x*x) minus 1 where layer_masks (the
 * TW masks of the first stage, run at sparsity + g1percent) already keeps it; the elements
 * strictly above the (100 - g1percent)-th percentile of all scores join the mask:
 * masks = layer_masks | extra.  masks[l] may be layer_masks[l].  q_type as above, by the type of
 * g1percent. */
int tw_prune_mix(int n_layers, const int32_t *K, const int32_t *N, const float *const *scores,
                 const uint8_t *const *layer_masks, double g1percent, int q_type,
                 uint8_t *const *masks, double *threshold, void *stream);

/* The building blocks of the two producers, on device buffers:
 *   tw_prune_tile_row_norms   norms[t*K + k] = ||scores[k][tile t]|| / width_t in NumPy's float32
 *                             summation order; col_keep (optional, N bytes) zeroes pruned
 *                             columns (prune_algo.py:92, 130)
 *   tw_prune_col_norms        norms[c] = ||scores[:, c]|| / K (prune_algo.py:64)
 *   tw_percentile_linear      np.percentile(values, q) with linear interpolation, in float32
 *                             (TW_Q_F32; the result is that float32 widened) or float64 */
int tw_prune_tile_row_norms(int K, int N, const float *scores, int n_tiles,
                            const int32_t *tile_col0, const int32_t *tile_width,
                            const uint8_t *col_keep, float *norms, void *stream);
int tw_prune_col_norms(int K, int N, const float *scores, float *norms, void *stream);
int tw_percentile_linear(const float *values, int64_t n, double q, int q_type, double *result,
                         void *stream);

/* Tile tables (host): every G original columns (prune_algo.py:119-128), and ending after every
 * G-th kept column, the last tile taking the rest (prune_algo.py:76-88).  tile_col0 and
 * tile_width need room for N entries. */
int tw_tiles_every_g_columns(int N, int G, int32_t *tile_col0, int32_t *tile_width,
                             int32_t *n_tiles);
int tw_tiles_every_g_kept_columns(int N, int G, const uint8_t *col_mask, int32_t *tile_col0,
                                  int32_t *tile_width, int32_t *n_tiles);

/* A tile table for a mask whose tiling is not known (host; mask is K x N bytes, row-major), e.g.
 * the name -> mask dictionaries the reference's pruning runs store (Pruning/VGG/pruning.py:580-581,
 * 639-640; Pruning/NMT/nmt/train.py:741-742).  Left to right, a tile takes columns while their
 * kept rows equal those of the tile's first non-empty column, up to G of them (G <= 0: no limit);
 * empty columns join the tile they fall into.  Every tile of the result is rows x columns, so
 * tw_plan_from_mask_tiles accepts it for ANY mask; a mask that is not tile-wise merely gets
 * narrow tiles.  tile_col0 and tile_width need room for N entries. */
int tw_tiles_from_mask(int K, int N, int G, const uint8_t *mask, int32_t *tile_col0,
                       int32_t *tile_width, int32_t *n_tiles);

#ifdef __cplusplus
}
#endif
#endif /* TWGEMM_H */
