// Host-only part of libtwgemm: error reporting, the integer helpers of the
// reference's host code (relative offsets, tile partition) and list validation.
// Nothing in this file touches the GPU, so these entry points work without one.
#include "tw_internal.h"

#include <cstring>
#include <vector>

namespace tw {

static thread_local std::string g_last_error;

void set_error(const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

int fail(int status, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return status;
}

static int check_list(const char *what, int tile, const int32_t *idx, int n, int limit)
{
    for (int i = 0; i < n; ++i) {
        if (idx[i] < 0 || idx[i] >= limit)
            return fail(TW_ERR_INDEX_LIST, "%s of tile %d: entry %d = %d is outside [0,%d)", what,
                        tile, i, idx[i], limit);
        if (i > 0 && idx[i] <= idx[i - 1])
            return fail(TW_ERR_INDEX_LIST, "%s of tile %d is not strictly ascending at entry %d",
                        what, tile, i);
    }
    return TW_OK;
}

int validate_lists(int K, int N, int n_tiles, const int32_t *tile_col0, const int32_t *tile_width,
                   const int32_t *kept_k_ptr, const int32_t *kept_k_idx,
                   const int32_t *kept_n_ptr, const int32_t *kept_n_idx)
{
    if (K <= 0 || N <= 0 || n_tiles <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d n_tiles=%d must all be positive", K, N, n_tiles);
    if (!tile_col0 || !tile_width || !kept_k_ptr || !kept_n_ptr)
        return fail(TW_ERR_NULL, "tile table or list pointer array is NULL");
    int next = 0;
    for (int t = 0; t < n_tiles; ++t) {
        if (tile_col0[t] != next || tile_width[t] <= 0)
            return fail(TW_ERR_TILE_TABLE,
                        "tile %d starts at column %d with width %d; expected start %d and a "
                        "positive width",
                        t, tile_col0[t], tile_width[t], next);
        next += tile_width[t];
        if (next > N)
            return fail(TW_ERR_TILE_TABLE, "tile %d ends at column %d beyond N=%d", t, next, N);
    }
    if (next != N)
        return fail(TW_ERR_TILE_TABLE, "tiles cover [0,%d) but N=%d", next, N);
    if (kept_k_ptr[0] != 0 || kept_n_ptr[0] != 0)
        return fail(TW_ERR_INDEX_LIST, "kept_k_ptr[0] and kept_n_ptr[0] must be 0");
    for (int t = 0; t < n_tiles; ++t) {
        int nk = kept_k_ptr[t + 1] - kept_k_ptr[t];
        int nn = kept_n_ptr[t + 1] - kept_n_ptr[t];
        if (nk < 0 || nk > K || nn < 0 || nn > tile_width[t])
            return fail(TW_ERR_INDEX_LIST, "tile %d: list lengths K_t=%d N_t=%d out of range", t,
                        nk, nn);
        if ((nk > 0 && !kept_k_idx) || (nn > 0 && !kept_n_idx))
            return fail(TW_ERR_NULL, "index array is NULL but tile %d has entries", t);
        int st = check_list("kept_k", t, kept_k_idx + kept_k_ptr[t], nk, K);
        if (st)
            return st;
        st = check_list("kept_n", t, kept_n_idx + kept_n_ptr[t], nn, tile_width[t]);
        if (st)
            return st;
    }
    return TW_OK;
}

} // namespace tw

extern "C" {

int tw_version(void) { return TWGEMM_VERSION; }

const char *tw_last_error(void) { return tw::g_last_error.c_str(); }

const char *tw_status_string(int status)
{
    switch (status) {
    case TW_OK: return "ok";
    case TW_ERR_NULL: return "null pointer";
    case TW_ERR_SHAPE: return "bad shape";
    case TW_ERR_TILE_TABLE: return "bad tile table";
    case TW_ERR_INDEX_LIST: return "bad index list";
    case TW_ERR_DTYPE: return "unknown dtype";
    case TW_ERR_LAYOUT: return "unknown layout or mode";
    case TW_ERR_ALIGNMENT: return "misaligned pointer or leading dimension";
    case TW_ERR_NOT_TW: return "mask is not tile-wise";
    case TW_ERR_DEVICE: return "HIP runtime failure";
    case TW_ERR_ALLOC: return "allocation failed";
    case TW_ERR_BUFFER: return "buffer too small";
    default: return "unknown status";
    }
}

int tw_mask_to_offsets(const uint8_t *mask, int n, int32_t *offsets, int *n_kept)
{
    if (n < 0)
        return tw::fail(TW_ERR_SHAPE, "n=%d is negative", n);
    if ((n > 0 && (!mask || !offsets)) || !n_kept)
        return tw::fail(TW_ERR_NULL, "mask, offsets or n_kept is NULL");
    int kept = 0;
    for (int idx = 0; idx < n; ++idx) {
        if (mask[idx] > 1)
            return tw::fail(TW_ERR_INDEX_LIST, "mask[%d] = %d is neither 0 nor 1", idx, mask[idx]);
        if (mask[idx]) {
            offsets[kept] = idx - kept;
            ++kept;
        }
    }
    *n_kept = kept;
    return TW_OK;
}

int tw_offsets_to_kept(const int32_t *offsets, int n_kept, int limit, int32_t *kept)
{
    if (n_kept < 0 || limit < 0)
        return tw::fail(TW_ERR_SHAPE, "n_kept=%d limit=%d", n_kept, limit);
    if (n_kept > 0 && (!offsets || !kept))
        return tw::fail(TW_ERR_NULL, "offsets or kept is NULL");
    for (int i = 0; i < n_kept; ++i) {
        int64_t v = (int64_t)offsets[i] + i;
        if (v < 0 || v >= limit)
            return tw::fail(TW_ERR_INDEX_LIST, "offset %d gives index %lld outside [0,%d)", i,
                            (long long)v, limit);
        if (i > 0 && v <= kept[i - 1])
            return tw::fail(TW_ERR_INDEX_LIST, "offsets do not give ascending indices at %d", i);
        kept[i] = (int32_t)v;
    }
    return TW_OK;
}

int tw_tile_partition(int M, int N, int K, int N_pruned, int K_pruned, int n_dim, int max_tiles,
                      int *block_num, int32_t *N_ori, int32_t *N_cal, int32_t *K_cal,
                      int64_t *off_B, int64_t *off_C)
try {
    if (!block_num || !N_ori || !N_cal || !K_cal || !off_B || !off_C)
        return tw::fail(TW_ERR_NULL, "an output array is NULL");
    if (M < 0 || N <= 0 || K <= 0 || n_dim <= 0 || N_pruned <= 0 || N_pruned > N || K_pruned < 0 ||
        K_pruned > K)
        return tw::fail(TW_ERR_SHAPE,
                        "M=%d N=%d K=%d N_pruned=%d K_pruned=%d n_dim=%d: need 0<N_pruned<=N, "
                        "0<=K_pruned<=K",
                        M, N, K, N_pruned, K_pruned, n_dim);
    int bn = (N_pruned + n_dim - 1) / n_dim;
    if (bn > max_tiles)
        return tw::fail(TW_ERR_BUFFER, "%d tiles needed, arrays hold %d", bn, max_tiles);
    int each = N / bn;
    int last_ori = N - each * (bn - 1);
    int last_cal = N_pruned - n_dim * (bn - 1);
    if ((bn > 1 && each < n_dim) || last_ori < last_cal)
        return tw::fail(TW_ERR_SHAPE,
                        "partition keeps more columns than a tile holds (N=%d N_pruned=%d n_dim=%d)",
                        N, N_pruned, n_dim);
    int64_t ob = 0, oc = 0;
    for (int i = 0; i < bn; ++i) {
        N_ori[i] = i + 1 < bn ? each : last_ori;
        N_cal[i] = i + 1 < bn ? n_dim : last_cal;
        K_cal[i] = K_pruned;
        off_B[i] = ob;
        off_C[i] = oc;
        ob += (int64_t)K * N_ori[i];
        oc += (int64_t)M * N_ori[i];
    }
    *block_num = bn;
    return TW_OK;
}
TW_CATCH_TO_STATUS

int tw_tiles_from_mask(int K, int N, int G, const uint8_t *mask, int32_t *tile_col0,
                       int32_t *tile_width, int32_t *n_tiles)
try {
    if (K <= 0 || N <= 0)
        return tw::fail(TW_ERR_SHAPE, "K=%d N=%d must be positive", K, N);
    if (!mask || !tile_col0 || !tile_width || !n_tiles)
        return tw::fail(TW_ERR_NULL, "a pointer is NULL");
    // One pass over the rows: a position-dependent 64-bit fingerprint of every column's kept
    // rows (two columns with different rows collide with probability 2^-64; the plan builders
    // check every element of every tile afterwards, so a collision surfaces as TW_ERR_NOT_TW).
    std::vector<uint64_t> sig((size_t)N, 0);
    std::vector<uint8_t> any((size_t)N, 0);
    for (int k = 0; k < K; ++k) {
        const uint8_t *row = mask + (size_t)k * N;
        for (int c = 0; c < N; ++c) {
            const uint64_t bit = row[c] != 0;
            sig[c] = sig[c] * 0x9E3779B97F4A7C15ull + bit * 0xD6E8FEB86659FD93ull;
            any[c] |= (uint8_t)bit;
        }
    }
    int t = 0, start = 0, kept = 0;
    uint64_t cur = 0;
    for (int c = 0; c < N; ++c) {
        if (!any[c])
            continue; // an empty column rides along with the tile it falls into
        if (kept > 0 && (sig[c] != cur || (G > 0 && kept == G))) {
            tile_col0[t] = start;
            tile_width[t] = c - start;
            ++t;
            start = c;
            kept = 0;
        }
        cur = sig[c];
        ++kept;
    }
    tile_col0[t] = start;
    tile_width[t] = N - start;
    *n_tiles = t + 1;
    return TW_OK;
}
TW_CATCH_TO_STATUS

} // extern "C"
