// Plan construction for libtwgemm: the integer mask -> kept lists -> relative
// offsets -> compaction pre-pass (HIP kernels), the MFMA-ordered weight packing,
// and the read-back used for bit-exact checks.
//
// Packed weight of tile t (K_t x N_t compact, padded to k_pad x n_pad, nblk = n_pad/32):
//   for 64-row step s, 32-column block nb, k16 step ks (0..3), lane l (0..63), e (0..7):
//     Bp[b_off + (((s * nblk + nb) * 4 + ks) * 64 + l) * 8 + e]
//        = compact[s*64 + ks*16 + (l/32)*8 + e][nb*32 + l%32]      (0 outside K_t x N_t)
// i.e. one MFMA B operand is 16 bytes per lane, 1 KiB contiguous per wave, and the whole
// block a 64-row main-loop step needs is one contiguous run of nblk * 4 KiB.
#include "tw_internal.h"

#include <algorithm>
#include <cstring>
#include <mutex>

namespace tw {

constexpr int kPackKS = kBlockK / kMfmaK; // MFMA k steps per packed step

struct PackTile {
    int32_t col0, k_kept, n_kept, k_pad, n_pad, kk_off, kn_off, pad_;
    int64_t b_off;
    int64_t src_off; // stream layout only: element offset of the tile in B_stream
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f)
{
    uint32_t x = __float_as_uint(f);
    if ((x & 0x7F800000u) == 0x7F800000u && (x & 0x007FFFFFu))
        return (uint16_t)((x >> 16) | 0x0040u);
    x += 0x7FFFu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

__device__ __forceinline__ uint16_t f32_to_f16_rne(float f)
{
    _Float16 h = (_Float16)f; // v_cvt_f16_f32, round to nearest even
    return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ uint16_t cast16(float f, int dtype)
{
    return dtype == TW_BF16 ? f32_to_bf16_rne(f) : f32_to_f16_rne(f);
}

// ---------------------------------------------------------------------------------
// packing

// `mask` (optional, K x N bytes): elements whose mask byte is zero are stored as zeros (covering
// plans of masks that are not rows x columns per tile)
__global__ void pack_dense_kernel(const PackTile *tiles, const int32_t *kept_k,
                                  const int32_t *kept_n, const float *B, int N, int dtype,
                                  uint16_t *Bp, const uint8_t *mask)
{
    const PackTile t = tiles[blockIdx.y];
    const int64_t groups = (int64_t)t.k_pad * t.n_pad / 8;
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= groups)
        return;
    const int lane = (int)(g & 63);
    const int64_t blk = g >> 6; // ((step * nblk + nb) * kPackKS + ks)
    const int nblk = t.n_pad / kMfmaN;
    const int ks = (int)(blk % kPackKS);
    const int nb = (int)((blk / kPackKS) % nblk);
    const int k16 = (int)((blk / kPackKS) / nblk) * kPackKS + ks;
    const int n = nb * kMfmaN + (lane & 31);
    const int kk0 = k16 * kMfmaK + (lane >> 5) * 8;
    uint16_t v[8];
    int col = -1;
    if (n < t.n_kept)
        col = t.col0 + kept_n[t.kn_off + n];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int kk = kk0 + e;
        float f = 0.0f;
        if (col >= 0 && kk < t.k_kept) {
            const int64_t src = (int64_t)kept_k[t.kk_off + kk] * N + col;
            if (!mask || mask[src])
                f = B[src];
        }
        v[e] = cast16(f, dtype);
    }
    uint4 out;
    out.x = v[0] | ((uint32_t)v[1] << 16);
    out.y = v[2] | ((uint32_t)v[3] << 16);
    out.z = v[4] | ((uint32_t)v[5] << 16);
    out.w = v[6] | ((uint32_t)v[7] << 16);
    *reinterpret_cast<uint4 *>(Bp + t.b_off + g * 8) = out;
}

// Source is the reference's compacted layout: tile column j, row i at
// Bs[src_off + j*K + i] (gen_masked_stream_weight, basic_nn.cu:765).
__global__ void pack_stream_kernel(const PackTile *tiles, const uint16_t *Bs, int K, uint16_t *Bp)
{
    const PackTile t = tiles[blockIdx.y];
    const int64_t groups = (int64_t)t.k_pad * t.n_pad / 8;
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= groups)
        return;
    const int lane = (int)(g & 63);
    const int64_t blk = g >> 6; // ((step * nblk + nb) * kPackKS + ks)
    const int nblk = t.n_pad / kMfmaN;
    const int ks = (int)(blk % kPackKS);
    const int nb = (int)((blk / kPackKS) % nblk);
    const int k16 = (int)((blk / kPackKS) / nblk) * kPackKS + ks;
    const int n = nb * kMfmaN + (lane & 31);
    const int kk0 = k16 * kMfmaK + (lane >> 5) * 8;
    uint16_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int kk = kk0 + e;
        v[e] = (n < t.n_kept && kk < t.k_kept) ? Bs[t.src_off + (int64_t)n * K + kk] : (uint16_t)0;
    }
    uint4 out;
    out.x = v[0] | ((uint32_t)v[1] << 16);
    out.y = v[2] | ((uint32_t)v[3] << 16);
    out.z = v[4] | ((uint32_t)v[5] << 16);
    out.w = v[6] | ((uint32_t)v[7] << 16);
    *reinterpret_cast<uint4 *>(Bp + t.b_off + g * 8) = out;
}

// Inverse of the packing into the reference's compacted layout at K*col0.
__global__ void unpack_stream_kernel(const PackTile *tiles, const uint16_t *Bp, int K, uint16_t *Bs)
{
    const PackTile t = tiles[blockIdx.y];
    const int64_t groups = (int64_t)t.k_pad * t.n_pad / 8;
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= groups)
        return;
    const int lane = (int)(g & 63);
    const int64_t blk = g >> 6; // ((step * nblk + nb) * kPackKS + ks)
    const int nblk = t.n_pad / kMfmaN;
    const int ks = (int)(blk % kPackKS);
    const int nb = (int)((blk / kPackKS) % nblk);
    const int k16 = (int)((blk / kPackKS) / nblk) * kPackKS + ks;
    const int n = nb * kMfmaN + (lane & 31);
    const int kk0 = k16 * kMfmaK + (lane >> 5) * 8;
    if (n >= t.n_kept)
        return;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int kk = kk0 + e;
        if (kk < t.k_kept)
            Bs[(int64_t)(t.col0 + n) * K + kk] = Bp[t.b_off + g * 8 + e];
    }
}

// ---------------------------------------------------------------------------------
// mask -> flags -> lists  (integer pre-pass)

// The tile table on the device: tcol0[t] is the first column of tile t, tcol0[n_tiles] == N.

// Both flag kernels walk the mask in 16-byte column chunks: thread (slice, chunk) of a block
// handles chunk `chunk` of the rows slice, slice + 256/cw, ... of a 64-row slab, so that the cw
// lanes next to each other read cw * 16 contiguous bytes of one row.  A chunk usually lies inside
// one tile; chunks that straddle a tile boundary, ragged ends and unaligned masks take the
// byte-wise path.

struct ChunkPos {
    int c0, w;       // first column and width (1..16) of the chunk
    int t0;          // tile of the chunk's first column
    bool one_tile;   // the whole chunk lies in tile t0
    bool vec;        // 16-byte loads are possible
    int k_begin, k_end, k_step;
};

__device__ __forceinline__ bool chunk_pos(const uint8_t *mask, int K, int N, const int32_t *tcol0,
                                          int n_tiles, int cw, ChunkPos &q)
{
    const int nchunk = (N + 15) >> 4;
    const int chunk = blockIdx.x * cw + (int)(threadIdx.x % cw);
    if (chunk >= nchunk)
        return false;
    q.c0 = chunk << 4;
    q.w = min(16, N - q.c0);
    int lo = 0, hi = n_tiles; // the tile with tcol0[t] <= c0 < tcol0[t+1]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tcol0[mid] <= q.c0)
            lo = mid;
        else
            hi = mid;
    }
    q.t0 = lo;
    q.one_tile = tcol0[lo + 1] >= q.c0 + q.w;
    q.vec = q.w == 16 && (N & 15) == 0 && ((uintptr_t)mask & 15) == 0;
    q.k_step = 256 / cw;
    q.k_begin = blockIdx.y * 64 + (int)(threadIdx.x / cw);
    q.k_end = min(K, (int)blockIdx.y * 64 + 64);
    return true;
}

// the chunk's bytes as four words, byte j of the chunk in bits 8*(j%4) of word j/4; 0 beyond w
__device__ __forceinline__ void load_chunk(const uint8_t *src, const ChunkPos &q, uint32_t (&v)[4])
{
    if (q.vec) {
        const uint4 x = *reinterpret_cast<const uint4 *>(src);
        v[0] = x.x;
        v[1] = x.y;
        v[2] = x.z;
        v[3] = x.w;
    } else {
        v[0] = v[1] = v[2] = v[3] = 0u;
        for (int j = 0; j < q.w; ++j)
            v[j >> 2] |= (uint32_t)src[j] << ((j & 3) * 8);
    }
}

__device__ __forceinline__ uint32_t chunk_byte(const uint32_t (&v)[4], int j)
{
    return (v[j >> 2] >> ((j & 3) * 8)) & 0xFFu;
}

// Rows a thread loads before it looks at any of them, so that this many 16-byte loads are in
// flight per lane.
constexpr int kFlagBatch = 8;

// rowflag[t*K + k] = 1 where any byte of mask[k][tcol0[t] .. tcol0[t+1]) is non-zero,
// colflag[c] = 1 where any byte of column c is; both arrays start zeroed and only receive ones.
__global__ void __launch_bounds__(256)
    mask_flags_kernel(const uint8_t *__restrict__ mask, int K, int N,
                      const int32_t *__restrict__ tcol0, int n_tiles, int cw,
                      uint8_t *__restrict__ rowflag, uint8_t *__restrict__ colflag)
{
    ChunkPos q;
    if (!chunk_pos(mask, K, N, tcol0, n_tiles, cw, q))
        return;
    // Of the lanes that hold chunks of one row inside one tile, only the lowest one with a
    // non-zero chunk stores the row flag.  seg_mask: the lanes below this one from the tile's
    // first whole chunk in this row on (they all lie in tile t0 when this chunk does).
    const int lane = (int)(threadIdx.x & 63u);
    unsigned long long seg_mask = 0ull;
    if (q.one_tile) {
        const int in_row = (int)(threadIdx.x % cw);
        const int first_chunk = (tcol0[q.t0] + 15) >> 4;
        const int seg_lane = lane - in_row + max(0, first_chunk - (int)blockIdx.x * cw);
        seg_mask = ((1ull << lane) - 1ull) & ~((1ull << seg_lane) - 1ull);
    }
    uint32_t acc[4] = {0u, 0u, 0u, 0u};
    for (int k0 = q.k_begin; k0 < q.k_end; k0 += kFlagBatch * q.k_step) {
        uint32_t v[kFlagBatch][4];
#pragma unroll
        for (int i = 0; i < kFlagBatch; ++i) {
            const int k = k0 + i * q.k_step;
            if (k < q.k_end)
                load_chunk(mask + (int64_t)k * N + q.c0, q, v[i]);
            else
                v[i][0] = v[i][1] = v[i][2] = v[i][3] = 0u;
        }
#pragma unroll
        for (int i = 0; i < kFlagBatch; ++i) {
            const int k = k0 + i * q.k_step;
            const bool nz = (v[i][0] | v[i][1] | v[i][2] | v[i][3]) != 0u;
            // lanes of one row run the same iterations, so a row's lanes all vote here
            const unsigned long long votes = __ballot(nz && q.one_tile);
            if (!nz)
                continue; // also every row past k_end
            if (q.one_tile) {
                if ((votes & seg_mask) == 0ull)
                    rowflag[(int64_t)q.t0 * K + k] = 1;
            } else {
                int t = q.t0, t_end = tcol0[t + 1];
                uint32_t any = 0;
                for (int j = 0; j < q.w; ++j) {
                    if (q.c0 + j >= t_end) {
                        if (any)
                            rowflag[(int64_t)t * K + k] = 1;
                        any = 0;
                        ++t;
                        t_end = tcol0[t + 1];
                    }
                    any |= chunk_byte(v[i], j);
                }
                if (any)
                    rowflag[(int64_t)t * K + k] = 1;
            }
            acc[0] |= v[i][0];
            acc[1] |= v[i][1];
            acc[2] |= v[i][2];
            acc[3] |= v[i][3];
        }
    }
    for (int j = 0; j < q.w; ++j)
        if (chunk_byte(acc, j))
            colflag[q.c0 + j] = 1;
}

// counts the elements where mask != rowflag & colflag (a TW mask has none)
__global__ void __launch_bounds__(256)
    validate_tw_kernel(const uint8_t *__restrict__ mask, int K, int N,
                       const int32_t *__restrict__ tcol0, int n_tiles, int cw,
                       const uint8_t *__restrict__ rowflag, const uint8_t *__restrict__ colflag,
                       unsigned long long *__restrict__ mismatch)
{
    ChunkPos q;
    unsigned bad = 0;
    if (chunk_pos(mask, K, N, tcol0, n_tiles, cw, q)) {
        // 0x01 in every byte of the chunk whose column is kept
        uint32_t cf[4] = {0u, 0u, 0u, 0u};
        for (int j = 0; j < q.w; ++j)
            cf[j >> 2] |= (colflag[q.c0 + j] ? 1u : 0u) << ((j & 3) * 8);
        for (int k0 = q.k_begin; k0 < q.k_end; k0 += kFlagBatch * q.k_step) {
            uint32_t v[kFlagBatch][4];
            uint32_t rf[kFlagBatch]; // all ones where the row of tile t0 is kept
#pragma unroll
            for (int i = 0; i < kFlagBatch; ++i) {
                const int k = k0 + i * q.k_step;
                if (k < q.k_end) {
                    load_chunk(mask + (int64_t)k * N + q.c0, q, v[i]);
                    rf[i] = rowflag[(int64_t)q.t0 * K + k] ? 0xFFFFFFFFu : 0u;
                } else {
                    v[i][0] = v[i][1] = v[i][2] = v[i][3] = 0u;
                    rf[i] = 0u;
                }
            }
#pragma unroll
            for (int i = 0; i < kFlagBatch; ++i) {
                const int k = k0 + i * q.k_step;
                if (q.one_tile) {
                    // byte-parallel: 0x01 where the mask byte is non-zero, against (row kept) & cf;
                    // a row past k_end has v == 0 and rf == 0 and adds nothing
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const uint32_t x = v[i][w];
                        const uint32_t nz =
                            ((x | ((x & 0x7F7F7F7Fu) + 0x7F7F7F7Fu)) >> 7) & 0x01010101u;
                        bad += __popc(nz ^ (cf[w] & rf[i]));
                    }
                } else if (k < q.k_end) {
                    int t = q.t0, t_end = tcol0[t + 1];
                    bool r = rf[i] != 0u;
                    for (int j = 0; j < q.w; ++j) {
                        if (q.c0 + j >= t_end) {
                            ++t;
                            t_end = tcol0[t + 1];
                            r = rowflag[(int64_t)t * K + k] != 0;
                        }
                        const bool m = chunk_byte(v[i], j) != 0;
                        const bool e = r && chunk_byte(cf, j);
                        bad += m != e;
                    }
                }
            }
        }
    }
    // one atomic per wave that saw a mismatch
    for (int off = 32; off > 0; off >>= 1)
        bad += __shfl_down(bad, off);
    if ((threadIdx.x & 63) == 0 && bad)
        atomicAdd(mismatch, (unsigned long long)bad);
}

// Counting and compaction work on segments of kSegFlags flags (rows of one tile, or columns of
// one tile), one workgroup per segment: grid (n_tiles, n_seg_k + n_seg_n), y < n_seg_k rows.
// seg_counts holds the kept flags per segment, tile-major: first the n_tiles * n_seg_k row
// entries, then the n_tiles * n_seg_n column entries.
constexpr int kSegFlags = 1024;
constexpr int kSegRounds = kSegFlags / 256;

struct FlagSegment {
    const uint8_t *flag; // the tile's flag vector
    int n;               // its length
    int first;           // first flag of this segment
    int entry;           // index of this segment among the row (or column) entries
    bool rows;
};

__device__ __forceinline__ FlagSegment flag_segment(const uint8_t *rowflag, const uint8_t *colflag,
                                                    int K, const int32_t *tcol0, int n_seg_k,
                                                    int n_seg_n)
{
    FlagSegment g;
    const int t = blockIdx.x;
    g.rows = (int)blockIdx.y < n_seg_k;
    const int seg = g.rows ? (int)blockIdx.y : (int)blockIdx.y - n_seg_k;
    g.flag = g.rows ? rowflag + (int64_t)t * K : colflag + tcol0[t];
    g.n = g.rows ? K : tcol0[t + 1] - tcol0[t];
    g.first = seg * kSegFlags;
    g.entry = t * (g.rows ? n_seg_k : n_seg_n) + seg;
    return g;
}

__global__ void __launch_bounds__(256)
    count_flags_kernel(const uint8_t *__restrict__ rowflag, const uint8_t *__restrict__ colflag,
                       int K, const int32_t *__restrict__ tcol0, int n_tiles, int n_seg_k,
                       int n_seg_n, int32_t *__restrict__ seg_counts)
{
    __shared__ int s_wave[4];
    const FlagSegment g = flag_segment(rowflag, colflag, K, tcol0, n_seg_k, n_seg_n);
    int c = 0;
#pragma unroll
    for (int j = 0; j < kSegRounds; ++j) {
        const int i = g.first + j * 256 + (int)threadIdx.x;
        if (i < g.n)
            c += g.flag[i] != 0;
    }
    for (int off = 32; off > 0; off >>= 1)
        c += __shfl_down(c, off);
    if ((threadIdx.x & 63) == 0)
        s_wave[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0)
        seg_counts[(g.rows ? 0 : n_tiles * n_seg_k) + g.entry] =
            s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
}

// Ordered compaction of one segment: the ascending kept indices and the relative offsets
// kept[i] - i land where the segments before it (seg_counts, tile-major) leave off.
__global__ void __launch_bounds__(256)
    compact_lists_kernel(const uint8_t *__restrict__ rowflag, const uint8_t *__restrict__ colflag,
                         int K, const int32_t *__restrict__ tcol0, int n_tiles, int n_seg_k,
                         int n_seg_n, const int32_t *__restrict__ seg_counts,
                         int32_t *__restrict__ kept_k, int32_t *__restrict__ rel_k,
                         int32_t *__restrict__ kept_n, int32_t *__restrict__ rel_n)
{
    __shared__ int s_sum[2][4];
    __shared__ int s_round[kSegRounds][4];
    const FlagSegment g = flag_segment(rowflag, colflag, K, tcol0, n_seg_k, n_seg_n);
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    bool f[kSegRounds];
#pragma unroll
    for (int j = 0; j < kSegRounds; ++j) {
        const int i = g.first + j * 256 + (int)threadIdx.x;
        f[j] = i < g.n && g.flag[i] != 0;
    }
    // kept flags before this segment: in the tiles before (a) and earlier in this tile (b)
    const int32_t *cnt = seg_counts + (g.rows ? 0 : n_tiles * n_seg_k);
    const int tile_first = (int)blockIdx.x * (g.rows ? n_seg_k : n_seg_n);
    int a = 0, b = 0;
    for (int i = (int)threadIdx.x; i < g.entry; i += 256) {
        const int v = cnt[i];
        if (i < tile_first)
            a += v;
        else
            b += v;
    }
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_down(a, off);
        b += __shfl_down(b, off);
    }
    int before[kSegRounds];
#pragma unroll
    for (int j = 0; j < kSegRounds; ++j) {
        const unsigned long long votes = __ballot(f[j]);
        before[j] = __popcll(votes & ((1ull << lane) - 1ull));
        if (lane == 0)
            s_round[j][wave] = __popcll(votes);
    }
    if (lane == 0) {
        s_sum[0][wave] = a;
        s_sum[1][wave] = b;
    }
    __syncthreads();
    const int in_tile = s_sum[1][0] + s_sum[1][1] + s_sum[1][2] + s_sum[1][3];
    const int tile_base = s_sum[0][0] + s_sum[0][1] + s_sum[0][2] + s_sum[0][3];
    int32_t *kept = (g.rows ? kept_k : kept_n) + tile_base;
    int32_t *rel = (g.rows ? rel_k : rel_n) + tile_base;
    int rank = in_tile; // position in the tile's list of this round's first kept flag
#pragma unroll
    for (int j = 0; j < kSegRounds; ++j) {
        int mine = rank + before[j];
        for (int w = 0; w < wave; ++w)
            mine += s_round[j][w];
        if (f[j]) {
            const int i = g.first + j * 256 + (int)threadIdx.x;
            kept[mine] = i;
            rel[mine] = i - mine;
        }
        rank += s_round[j][0] + s_round[j][1] + s_round[j][2] + s_round[j][3];
    }
}

// ---------------------------------------------------------------------------------

static int round_up(int v, int m) { return (v + m - 1) / m * m; }

static std::vector<PackTile> pack_tiles(const tw_plan *p, const int64_t *src_off)
{
    std::vector<PackTile> v(p->n_tiles);
    for (int t = 0; t < p->n_tiles; ++t) {
        PackTile &q = v[t];
        q.col0 = p->tile_col0[t];
        q.k_kept = p->kept_k_ptr[t + 1] - p->kept_k_ptr[t];
        q.n_kept = p->kept_n_ptr[t + 1] - p->kept_n_ptr[t];
        q.k_pad = p->k_pad[t];
        q.n_pad = p->n_pad[t];
        q.kk_off = p->kept_k_ptr[t];
        q.kn_off = p->kept_n_ptr[t];
        q.pad_ = 0;
        q.b_off = p->b_off[t];
        q.src_off = src_off ? src_off[t] : 0;
    }
    return v;
}

static int64_t max_groups(const tw_plan *p)
{
    int64_t g = 0;
    for (int t = 0; t < p->n_tiles; ++t)
        g = std::max<int64_t>(g, (int64_t)p->k_pad[t] * p->n_pad[t] / 8);
    return g;
}

template <typename T> static int upload(T **dst, const std::vector<T> &src)
{
    *dst = nullptr;
    size_t bytes = std::max<size_t>(src.size(), 1) * sizeof(T);
    if (hipMalloc((void **)dst, bytes) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of %zu bytes failed", bytes);
    if (!src.empty()) {
        hipError_t e = hipMemcpy(*dst, src.data(), src.size() * sizeof(T), hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            hipFree(*dst);
            *dst = nullptr;
            return fail(TW_ERR_DEVICE, "upload of %zu bytes failed: %s", bytes, hipGetErrorString(e));
        }
    }
    return TW_OK;
}

static void free_plan(tw_plan *p);

// Owners of what a builder holds until it succeeds: whatever path leaves the builder (an error
// return, an exception on its way to the status conversion), the device buffer and the
// half-built plan are released.
struct DeviceBuffer {
    void *ptr = nullptr;
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    ~DeviceBuffer()
    {
        if (ptr)
            (void)hipFree(ptr);
    }
};
struct PlanOwner {
    tw_plan *p = nullptr;
    PlanOwner() = default;
    PlanOwner(const PlanOwner &) = delete;
    PlanOwner &operator=(const PlanOwner &) = delete;
    ~PlanOwner()
    {
        if (p)
            free_plan(p);
    }
    tw_plan *release()
    {
        tw_plan *r = p;
        p = nullptr;
        return r;
    }
};

int finalize_plan_geometry(tw_plan *p, hipStream_t s)
{
    const int dst = prepare_device();
    if (dst != TW_OK)
        return dst;
    const int nt = p->n_tiles;
    p->k_pad.assign(nt, 0);
    p->n_pad.assign(nt, 0);
    p->b_off.assign(nt, 0);
    int64_t off = 0;
    std::vector<UnitDev> units;
    std::vector<TileDev> ztiles;
    std::vector<int32_t> pruned_n;
    std::vector<int32_t> kept_k_pad; // the GEMM kernel's copy: k_pad entries per tile
    p->max_unit_n = 0;
    p->n_halves = 0;
    for (int t = 0; t < nt; ++t) {
        const int kt = p->kept_k_ptr[t + 1] - p->kept_k_ptr[t];
        const int ntk = p->kept_n_ptr[t + 1] - p->kept_n_ptr[t];
        p->k_pad[t] = ntk > 0 ? round_up(kt, kBlockK) : 0;
        p->n_pad[t] = kt > 0 ? round_up(ntk, kMfmaN) : 0;
        if (p->k_pad[t] == 0 || p->n_pad[t] == 0) {
            // nothing to multiply; kept columns (if any) still receive alpha*0 + beta*C
            p->k_pad[t] = 0;
            p->n_pad[t] = ntk > 0 ? round_up(ntk, kMfmaN) : 0;
        }
        const int32_t kkp_off = (int32_t)kept_k_pad.size();
        kept_k_pad.insert(kept_k_pad.end(), p->kept_k_idx.begin() + p->kept_k_ptr[t],
                          p->kept_k_idx.begin() + p->kept_k_ptr[t + 1]);
        // padding past k_pad: the kernel prefetches the index list up to eight 64-row steps ahead
        kept_k_pad.resize(kkp_off + p->k_pad[t] + 8 * kBlockK, 0);
        p->b_off[t] = off;
        off += (int64_t)p->k_pad[t] * p->n_pad[t];
        off = (off + 511) / 512 * 512; // keep every tile 1 KiB aligned
        for (int nc0 = 0; nc0 < ntk; nc0 += kMaxUnitN) {
            UnitDev u;
            u.col0 = p->tile_col0[t];
            u.k_kept = kt;
            u.k_pad = p->k_pad[t];
            u.n_cnt = std::min(kMaxUnitN, ntk - nc0);
            u.nb0 = nc0 / kMfmaN;
            u.nb_cnt = (u.n_cnt + kMfmaN - 1) / kMfmaN;
            u.kk_off = kkp_off;
            u.kn_off = p->kept_n_ptr[t] + nc0;
            u.b_off = p->b_off[t];
            u.tile = t;
            u.nblk = p->n_pad[t] / kMfmaN;
            units.push_back(u);
            p->max_unit_n = std::max(p->max_unit_n, u.n_cnt);
            p->n_halves += (u.n_cnt + 63) / 64;
        }
        if (ntk < p->tile_width[t]) {
            TileDev z;
            z.col0 = p->tile_col0[t];
            z.n_pruned = p->tile_width[t] - ntk;
            z.pn_off = (int32_t)pruned_n.size();
            z.pad_ = 0;
            const int32_t *kn = p->kept_n_idx.data() + p->kept_n_ptr[t];
            int j = 0;
            for (int c = 0; c < p->tile_width[t]; ++c) {
                if (j < ntk && kn[j] == c)
                    ++j;
                else
                    pruned_n.push_back(c);
            }
            ztiles.push_back(z);
        }
    }
    // work queue order: heaviest kept-K first, ties keep a tile's pieces adjacent
    std::stable_sort(units.begin(), units.end(),
                     [](const UnitDev &a, const UnitDev &b) { return a.k_kept > b.k_kept; });
    p->packed_elems = off;
    p->n_units = (int)units.size();
    p->h_units = units;
    p->n_pipe_units = 0;
    for (const UnitDev &u : units)
        p->n_pipe_units += u.k_pad > 0;
    // nearly dense: kept rows summed over the tiles that keep any, against all K rows for each of
    // those tiles (a tile pruned away whole takes no part on either side)
    int64_t tiles_with_rows = 0;
    for (int t = 0; t < nt; ++t)
        tiles_with_rows += p->kept_k_ptr[t + 1] > p->kept_k_ptr[t];
    p->rows_shared = tiles_with_rows > 1 && p->n_pipe_units > 0 &&
                     (int64_t)p->kept_k_idx.size() * 10 >= (int64_t)p->K * tiles_with_rows * 9;
    p->n_zero_tiles = (int)ztiles.size();
    p->max_k_pad = 0;
    p->pipe_steps = 0;
    for (const UnitDev &u : units) {
        p->max_k_pad = std::max(p->max_k_pad, u.k_pad);
        p->pipe_steps += u.k_pad / kBlockK;
    }

    // One device allocation for everything the plan owns besides lists that were compacted on
    // the device: [staged tables, uploaded with one copy][ticket slots][packed weight], the last
    // two zeroed with one memset.
    std::vector<int32_t> rel_k, rel_n;
    const bool lists_here = p->d_kept_k == nullptr;
    if (lists_here) {
        rel_k.resize(p->kept_k_idx.size());
        rel_n.resize(p->kept_n_idx.size());
        for (int t = 0; t < nt; ++t) {
            for (int i = p->kept_k_ptr[t]; i < p->kept_k_ptr[t + 1]; ++i)
                rel_k[i] = p->kept_k_idx[i] - (i - p->kept_k_ptr[t]);
            for (int i = p->kept_n_ptr[t]; i < p->kept_n_ptr[t + 1]; ++i)
                rel_n[i] = p->kept_n_idx[i] - (i - p->kept_n_ptr[t]);
        }
    }
    const std::vector<PackTile> ptab = pack_tiles(p, nullptr);
    std::vector<char> stage;
    auto put = [&stage](const void *src, size_t bytes) { // returns the 256-aligned offset
        const size_t off = (stage.size() + 255) / 256 * 256;
        stage.resize(off + std::max<size_t>(bytes, 4), 0);
        if (bytes)
            std::memcpy(stage.data() + off, src, bytes);
        return off;
    };
    const size_t o_units = put(units.data(), units.size() * sizeof(UnitDev));
    const size_t o_tiles = put(ztiles.data(), ztiles.size() * sizeof(TileDev));
    const size_t o_pruned = put(pruned_n.data(), pruned_n.size() * sizeof(int32_t));
    const size_t o_kkpad = put(kept_k_pad.data(), kept_k_pad.size() * sizeof(int32_t));
    const size_t o_ptab = put(ptab.data(), ptab.size() * sizeof(PackTile));
    std::vector<int32_t> blocks;
    for (size_t ui = 0; ui < units.size(); ++ui)
        for (int nb = 0; nb < units[ui].nb_cnt; ++nb)
            blocks.push_back((int32_t)ui * 4 + nb);
    p->n_blocks = (int)blocks.size();
    p->blocks_per_unit = units.empty() ? 0 : units[0].nb_cnt;
    for (const UnitDev &u : units)
        if (u.nb_cnt != p->blocks_per_unit)
            p->blocks_per_unit = 0;
    const size_t o_blocks = put(blocks.data(), blocks.size() * sizeof(int32_t));
    std::vector<uint32_t> kpairs; // see GemmArgs::kept_pairs
    if (p->K < 0xFFFF) {
        // the padding names row K here (a row of zeros behind the kernel's panel of A), not row 0
        std::vector<uint16_t> padded(kept_k_pad.size(), (uint16_t)p->K);
        for (const UnitDev &u : units)
            for (int i = 0; i < u.k_kept; ++i)
                padded[u.kk_off + i] = (uint16_t)kept_k_pad[u.kk_off + i];
        kpairs.resize(kept_k_pad.size() / 2);
        for (size_t st = 0; st < kept_k_pad.size() / 64; ++st)
            for (int g16 = 0; g16 < 4; ++g16)
                for (int e = 0; e < 8; ++e) {
                    const size_t lo = st * 64 + g16 * 16 + (e >> 2) * 8 + (e & 3);
                    kpairs[st * 32 + e * 4 + g16] = (uint32_t)padded[lo] | ((uint32_t)padded[lo + 4] << 16);
                }
    }
    const size_t o_kpairs = put(kpairs.data(), kpairs.size() * sizeof(uint32_t));
    size_t o_kk = 0, o_kn = 0, o_rk = 0, o_rn = 0;
    if (lists_here) {
        o_kk = put(p->kept_k_idx.data(), p->kept_k_idx.size() * sizeof(int32_t));
        o_kn = put(p->kept_n_idx.data(), p->kept_n_idx.size() * sizeof(int32_t));
        o_rk = put(rel_k.data(), rel_k.size() * sizeof(int32_t));
        o_rn = put(rel_n.data(), rel_n.size() * sizeof(int32_t));
    }
    const size_t o_tickets = (stage.size() + 255) / 256 * 256;
    const size_t ticket_bytes = sizeof(int32_t) * kTicketInts * (kTicketSlots + 1); // (the last: status words)
    const size_t o_bp = (o_tickets + ticket_bytes + 1023) / 1024 * 1024;
    const size_t bp_bytes = (size_t)std::max<int64_t>(p->packed_elems, 8) * 2;
    char *slab = nullptr;
    if (hipMalloc((void **)&slab, o_bp + bp_bytes) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of %zu bytes for the plan failed", o_bp + bp_bytes);
    p->d_slab = slab;
    TW_HIP(hipMemcpyAsync(slab, stage.data(), stage.size(), hipMemcpyHostToDevice, s));
    // the packing kernel follows on the same stream and the builders wait for it; a plan with
    // nothing to pack waits here (the staged tables are host memory of this call: wait either way
    // before they go out of scope)
    TW_HIP(hipMemsetAsync(slab + o_tickets, 0, o_bp + bp_bytes - o_tickets, s));
    TW_HIP(hipStreamSynchronize(s));
    p->d_units = reinterpret_cast<UnitDev *>(slab + o_units);
    p->d_tiles = reinterpret_cast<TileDev *>(slab + o_tiles);
    p->d_pruned_n = reinterpret_cast<int32_t *>(slab + o_pruned);
    p->d_kept_k_pad = reinterpret_cast<int32_t *>(slab + o_kkpad);
    p->d_pack_tiles = slab + o_ptab;
    p->d_blocks = reinterpret_cast<int32_t *>(slab + o_blocks);
    p->d_kept_pairs = kpairs.empty() ? nullptr : reinterpret_cast<uint32_t *>(slab + o_kpairs);
    if (lists_here) {
        p->d_kept_k = reinterpret_cast<int32_t *>(slab + o_kk);
        p->d_kept_n = reinterpret_cast<int32_t *>(slab + o_kn);
        p->d_rel_k = reinterpret_cast<int32_t *>(slab + o_rk);
        p->d_rel_n = reinterpret_cast<int32_t *>(slab + o_rn);
    }
    p->d_tickets = reinterpret_cast<int32_t *>(slab + o_tickets);
    p->d_Bp = slab + o_bp;
    TW_HIP(hipGetDevice(&p->device));
    {
        // the CU count of a device does not change: ask once per device
        static std::mutex mu;
        static std::vector<int> cu_of;
        std::lock_guard<std::mutex> lock(mu);
        if ((int)cu_of.size() <= p->device)
            cu_of.resize(p->device + 1, 0);
        if (cu_of[p->device] == 0) {
            int n = 0;
            TW_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, p->device));
            cu_of[p->device] = n;
        }
        p->cu_count = cu_of[p->device];
    }
    return TW_OK;
}

int pack_from_dense(tw_plan *p, const float *d_B, hipStream_t s, const uint8_t *d_mask)
{
    const int64_t mg = max_groups(p);
    if (mg == 0)
        return TW_OK;
    dim3 grid((unsigned)((mg + 255) / 256), (unsigned)p->n_tiles);
    hipLaunchKernelGGL(pack_dense_kernel, grid, dim3(256), 0, s,
                       static_cast<const PackTile *>(p->d_pack_tiles), p->d_kept_k, p->d_kept_n, d_B,
                       p->N, p->dtype, (uint16_t *)p->d_Bp, d_mask);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess)
        e = hipStreamSynchronize(s);
    if (e != hipSuccess)
        return fail(TW_ERR_DEVICE, "weight packing kernel failed: %s", hipGetErrorString(e));
    return TW_OK;
}

int pack_from_stream(tw_plan *p, const void *d_Bs, const int64_t *off_B, hipStream_t s)
{
    const int64_t mg = max_groups(p);
    if (mg == 0)
        return TW_OK;
    std::vector<PackTile> pt = pack_tiles(p, off_B);
    PackTile *d_pt = nullptr;
    int st = upload(&d_pt, pt);
    if (st)
        return st;
    DeviceBuffer pt_owner;
    pt_owner.ptr = d_pt;
    dim3 grid((unsigned)((mg + 255) / 256), (unsigned)p->n_tiles);
    hipLaunchKernelGGL(pack_stream_kernel, grid, dim3(256), 0, s, d_pt, (const uint16_t *)d_Bs,
                       p->K, (uint16_t *)p->d_Bp);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess)
        e = hipStreamSynchronize(s);
    if (e != hipSuccess)
        return fail(TW_ERR_DEVICE, "stream-weight packing kernel failed: %s", hipGetErrorString(e));
    return TW_OK;
}

int unpack_to_stream(const tw_plan *p, uint16_t *d_Bs, hipStream_t s)
{
    TW_HIP(hipMemsetAsync(d_Bs, 0, (size_t)p->K * p->N * 2, s));
    const int64_t mg = max_groups(p);
    if (mg > 0) {
        std::vector<PackTile> pt = pack_tiles(p, nullptr);
        PackTile *d_pt = nullptr;
        int st = upload(&d_pt, pt);
        if (st)
            return st;
        DeviceBuffer pt_owner;
        pt_owner.ptr = d_pt;
        dim3 grid((unsigned)((mg + 255) / 256), (unsigned)p->n_tiles);
        hipLaunchKernelGGL(unpack_stream_kernel, grid, dim3(256), 0, s, d_pt,
                           (const uint16_t *)p->d_Bp, p->K, d_Bs);
        hipError_t e = hipGetLastError();
        if (e == hipSuccess)
            e = hipStreamSynchronize(s);
        if (e != hipSuccess)
            return fail(TW_ERR_DEVICE, "unpack kernel failed: %s", hipGetErrorString(e));
    }
    TW_HIP(hipStreamSynchronize(s));
    return TW_OK;
}

static void free_plan(tw_plan *p)
{
    if (!p)
        return;
    hipFree(p->d_lists);
    hipFree(p->d_slab);
    delete p;
}

static int check_dtype(int dtype)
{
    if (dtype != TW_F16 && dtype != TW_BF16)
        return fail(TW_ERR_DTYPE, "dtype %d is neither TW_F16 nor TW_BF16", dtype);
    return TW_OK;
}

// uploads a host fp32 [K,N] weight and packs it
static int pack_host_weight(tw_plan *p, const float *B)
{
    if (p->packed_elems == 0)
        return TW_OK;
    DeviceBuffer d_B;
    size_t bytes = (size_t)p->K * p->N * sizeof(float);
    if (hipMalloc(&d_B.ptr, bytes) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of %zu bytes for the weight upload failed", bytes);
    hipError_t e = hipMemcpy(d_B.ptr, B, bytes, hipMemcpyHostToDevice);
    return e == hipSuccess ? pack_from_dense(p, static_cast<const float *>(d_B.ptr), nullptr)
                           : fail(TW_ERR_DEVICE, "weight upload failed: %s", hipGetErrorString(e));
}

} // namespace tw

using namespace tw;

extern "C" {

int tw_plan_create(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                   const int32_t *tile_width, const int32_t *kept_k_ptr, const int32_t *kept_k_idx,
                   const int32_t *kept_n_ptr, const int32_t *kept_n_idx, const float *B,
                   tw_plan **out)
try {
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    int st = check_dtype(dtype);
    if (st)
        return st;
    st = validate_lists(K, N, n_tiles, tile_col0, tile_width, kept_k_ptr, kept_k_idx, kept_n_ptr,
                        kept_n_idx);
    if (st)
        return st;
    if (!B)
        return fail(TW_ERR_NULL, "B is NULL");
    PlanOwner owner;
    tw_plan *p = owner.p = new (std::nothrow) tw_plan;
    if (!p)
        return fail(TW_ERR_ALLOC, "out of host memory");
    p->K = K;
    p->N = N;
    p->dtype = dtype;
    p->n_tiles = n_tiles;
    p->tile_col0.assign(tile_col0, tile_col0 + n_tiles);
    p->tile_width.assign(tile_width, tile_width + n_tiles);
    p->kept_k_ptr.assign(kept_k_ptr, kept_k_ptr + n_tiles + 1);
    p->kept_n_ptr.assign(kept_n_ptr, kept_n_ptr + n_tiles + 1);
    p->kept_k_idx.assign(kept_k_idx, kept_k_idx + kept_k_ptr[n_tiles]);
    p->kept_n_idx.assign(kept_n_idx, kept_n_idx + kept_n_ptr[n_tiles]);
    if ((st = finalize_plan_geometry(p, nullptr)) || (st = pack_host_weight(p, B)))
        return st;
    *out = owner.release();
    return TW_OK;
}
TW_CATCH_TO_STATUS

int tw_plan_create_dense(int K, int N, int G, int dtype, const float *B, tw_plan **out)
try {
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (K <= 0 || N <= 0 || G <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d G=%d must all be positive", K, N, G);
    const int nt = (N + G - 1) / G;
    std::vector<int32_t> col0(nt), width(nt), kp(nt + 1), np(nt + 1), ki, ni;
    ki.reserve((size_t)nt * K);
    ni.reserve(N);
    kp[0] = np[0] = 0;
    for (int t = 0; t < nt; ++t) {
        col0[t] = t * G;
        width[t] = std::min(G, N - t * G);
        for (int k = 0; k < K; ++k)
            ki.push_back(k);
        for (int c = 0; c < width[t]; ++c)
            ni.push_back(c);
        kp[t + 1] = (int32_t)ki.size();
        np[t + 1] = (int32_t)ni.size();
    }
    return tw_plan_create(K, N, dtype, nt, col0.data(), width.data(), kp.data(), ki.data(),
                          np.data(), ni.data(), B, out);
}
TW_CATCH_TO_STATUS

int tw_plan_from_mask(int K, int N, int G, int dtype, const uint8_t *mask, const float *B,
                      tw_plan **out)
try {
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (K <= 0 || N <= 0 || G <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d G=%d must all be positive", K, N, G);
    const int nt = (N + G - 1) / G;
    std::vector<int32_t> col0(nt), width(nt);
    for (int t = 0; t < nt; ++t) {
        col0[t] = t * G;
        width[t] = std::min(G, N - t * G);
    }
    return tw_plan_from_mask_tiles(K, N, dtype, nt, col0.data(), width.data(), mask, B, out);
}
TW_CATCH_TO_STATUS

// The pre-pass on device operands: d_mask is K x N bytes, d_B the fp32 weight, both row-major in
// device memory.  Temporaries (flags, counters, the tile table) share one allocation.
static int plan_from_device_mask(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                                 const int32_t *tile_width, const uint8_t *d_mask, const float *d_B,
                                 bool cover, hipStream_t s, tw_plan **out)
{
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    int st = check_dtype(dtype);
    if (st)
        return st;
    if (K <= 0 || N <= 0 || n_tiles <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d n_tiles=%d must all be positive", K, N, n_tiles);
    if (!d_mask || !d_B || !tile_col0 || !tile_width)
        return fail(TW_ERR_NULL, "mask, B or the tile table is NULL");
    const int nt = n_tiles;
    std::vector<int32_t> tcol0(nt + 1);
    {
        int c = 0;
        for (int t = 0; t < nt; ++t) {
            if (tile_col0[t] != c || tile_width[t] <= 0)
                return fail(TW_ERR_TILE_TABLE,
                            "tile %d: col0=%d width=%d, tiles must cover [0,N) in order without gaps",
                            t, tile_col0[t], tile_width[t]);
            tcol0[t] = c;
            c += tile_width[t];
        }
        if (c != N)
            return fail(TW_ERR_TILE_TABLE, "tiles cover %d columns, N=%d", c, N);
        tcol0[nt] = N;
    }

    // one allocation for all temporaries, carved at 256-byte boundaries
    auto up = [](size_t b) { return (b + 255) / 256 * 256; };
    int max_width = 0;
    for (int t = 0; t < nt; ++t)
        max_width = std::max(max_width, tile_width[t]);
    const int n_seg_k = (K + kSegFlags - 1) / kSegFlags, n_seg_n = (max_width + kSegFlags - 1) / kSegFlags;
    if ((int64_t)nt * (n_seg_k + n_seg_n) > INT32_MAX || n_seg_k + n_seg_n > 65535)
        return fail(TW_ERR_SHAPE, "K=%d rows in %d tiles are more than the pre-pass indexes", K, nt);
    const size_t n_seg = (size_t)nt * (n_seg_k + n_seg_n);
    const size_t o_rowflag = 0;
    const size_t o_colflag = o_rowflag + up((size_t)nt * K);
    const size_t o_mismatch = o_colflag + up((size_t)N);
    const size_t o_counts = o_mismatch + up(sizeof(unsigned long long));
    const size_t o_tcol0 = o_counts + up(sizeof(int32_t) * n_seg);
    const size_t ws_bytes = o_tcol0 + up(sizeof(int32_t) * (nt + 1));
    // the workspace and the half-built plan are released on every way out of this function;
    // every kernel and copy runs on the caller's stream, which this function waits for
    DeviceBuffer ws_owner;
    PlanOwner owner;
#define TW_TRY(call) TW_HIP(call)
    TW_TRY(hipMalloc(&ws_owner.ptr, ws_bytes));
    char *const ws = static_cast<char *>(ws_owner.ptr);
    uint8_t *d_rowflag = reinterpret_cast<uint8_t *>(ws + o_rowflag);
    uint8_t *d_colflag = reinterpret_cast<uint8_t *>(ws + o_colflag);
    unsigned long long *d_mismatch = reinterpret_cast<unsigned long long *>(ws + o_mismatch);
    int32_t *d_seg_counts = reinterpret_cast<int32_t *>(ws + o_counts);
    int32_t *d_tcol0 = reinterpret_cast<int32_t *>(ws + o_tcol0);
    TW_TRY(hipMemcpyAsync(d_tcol0, tcol0.data(), sizeof(int32_t) * (nt + 1), hipMemcpyHostToDevice, s));
    // row flags, column flags and the mismatch counter start at zero (adjacent in the workspace)
    TW_TRY(hipMemsetAsync(ws, 0, o_counts, s));

    const dim3 seg_grid((unsigned)nt, (unsigned)(n_seg_k + n_seg_n));
    {
        // lanes next to each other take the chunks of one row: 64 of them where a row has that
        // many, else 32 or 16 (two or four rows per wave)
        const int nchunk = (N + 15) / 16;
        const int cw = nchunk > 32 ? 64 : (nchunk > 16 ? 32 : 16);
        const dim3 grid((unsigned)((nchunk + cw - 1) / cw), (unsigned)((K + 63) / 64));
        hipLaunchKernelGGL(mask_flags_kernel, grid, dim3(256), 0, s, d_mask, K, N, d_tcol0, nt,
                           cw, d_rowflag, d_colflag);
        hipLaunchKernelGGL(validate_tw_kernel, grid, dim3(256), 0, s, d_mask, K, N, d_tcol0, nt,
                           cw, d_rowflag, d_colflag, d_mismatch);
        hipLaunchKernelGGL(count_flags_kernel, seg_grid, dim3(256), 0, s, d_rowflag, d_colflag,
                           K, d_tcol0, nt, n_seg_k, n_seg_n, d_seg_counts);
        TW_TRY(hipGetLastError());
    }
    // the mismatch counter and the segment counts come back with one copy (they are adjacent)
    std::vector<char> back(o_tcol0 - o_mismatch);
    TW_TRY(hipMemcpyAsync(back.data(), ws + o_mismatch, back.size(), hipMemcpyDeviceToHost, s));
    TW_TRY(hipStreamSynchronize(s));
    unsigned long long mismatch = 0;
    std::memcpy(&mismatch, back.data(), sizeof(mismatch));
    const int32_t *seg_counts = reinterpret_cast<const int32_t *>(back.data() + (o_counts - o_mismatch));
    if (mismatch != 0 && !cover) {
        return fail(TW_ERR_NOT_TW,
                    "%llu mask elements differ from (row kept) & (column kept) of their tile",
                    mismatch);
    }

    tw_plan *const p = owner.p = new (std::nothrow) tw_plan;
    if (!p)
        return fail(TW_ERR_ALLOC, "out of host memory");
    p->K = K;
    p->N = N;
    p->dtype = dtype;
    p->n_tiles = nt;
    p->tile_col0.resize(nt);
    p->tile_width.resize(nt);
    p->kept_k_ptr.assign(nt + 1, 0);
    p->kept_n_ptr.assign(nt + 1, 0);
    for (int t = 0; t < nt; ++t) {
        p->tile_col0[t] = tile_col0[t];
        p->tile_width[t] = tile_width[t];
        int rows = 0, cols = 0;
        for (int g = 0; g < n_seg_k; ++g)
            rows += seg_counts[(size_t)t * n_seg_k + g];
        for (int g = 0; g < n_seg_n; ++g)
            cols += seg_counts[(size_t)nt * n_seg_k + (size_t)t * n_seg_n + g];
        p->kept_k_ptr[t + 1] = p->kept_k_ptr[t] + rows;
        p->kept_n_ptr[t + 1] = p->kept_n_ptr[t] + cols;
    }
    const size_t sk = std::max(p->kept_k_ptr[nt], 1), sn = std::max(p->kept_n_ptr[nt], 1);
    // [kept_k | kept_n | rel_k | rel_n], each at a 256-byte boundary: the first two come back
    // to the host with one copy
    const size_t l_kn = up(sizeof(int32_t) * sk), l_rk = l_kn + up(sizeof(int32_t) * sn);
    const size_t l_rn = l_rk + up(sizeof(int32_t) * sk);
    char *lists = nullptr;
    TW_TRY(hipMalloc((void **)&lists, l_rn + up(sizeof(int32_t) * sn)));
    p->d_lists = lists;
    p->d_kept_k = reinterpret_cast<int32_t *>(lists);
    p->d_kept_n = reinterpret_cast<int32_t *>(lists + l_kn);
    p->d_rel_k = reinterpret_cast<int32_t *>(lists + l_rk);
    p->d_rel_n = reinterpret_cast<int32_t *>(lists + l_rn);
    hipLaunchKernelGGL(compact_lists_kernel, seg_grid, dim3(256), 0, s, d_rowflag, d_colflag, K,
                       d_tcol0, nt, n_seg_k, n_seg_n, d_seg_counts, p->d_kept_k, p->d_rel_k,
                       p->d_kept_n, p->d_rel_n);
    TW_TRY(hipGetLastError());
    p->kept_k_idx.resize(p->kept_k_ptr[nt]);
    p->kept_n_idx.resize(p->kept_n_ptr[nt]);
    {
        std::vector<char> both(l_kn + sizeof(int32_t) * sn);
        TW_TRY(hipMemcpyAsync(both.data(), lists, both.size(), hipMemcpyDeviceToHost, s));
        TW_TRY(hipStreamSynchronize(s));
        if (!p->kept_k_idx.empty())
            std::memcpy(p->kept_k_idx.data(), both.data(), sizeof(int32_t) * p->kept_k_idx.size());
        if (!p->kept_n_idx.empty())
            std::memcpy(p->kept_n_idx.data(), both.data() + l_kn, sizeof(int32_t) * p->kept_n_idx.size());
    }
#undef TW_TRY
    st = validate_lists(K, N, nt, p->tile_col0.data(), p->tile_width.data(), p->kept_k_ptr.data(),
                        p->kept_k_idx.data(), p->kept_n_ptr.data(), p->kept_n_idx.data());
    if (!st)
        st = finalize_plan_geometry(p, s);
    // rows and columns of a covering tile are the union of its elements: the elements the mask
    // drops inside that cover are stored as zeros
    if (!st && p->packed_elems > 0)
        st = pack_from_dense(p, d_B, s, cover && mismatch != 0 ? d_mask : nullptr);
    if (st)
        return st;
    *out = owner.release();
    return TW_OK;
}

// host operands: one upload buffer for the mask and the weight, then the device pre-pass
static int plan_from_mask_impl(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                               const int32_t *tile_width, const uint8_t *mask, const float *B,
                               bool cover, tw_plan **out)
{
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (int st = check_dtype(dtype))
        return st;
    if (K <= 0 || N <= 0 || n_tiles <= 0)
        return fail(TW_ERR_SHAPE, "K=%d N=%d n_tiles=%d must all be positive", K, N, n_tiles);
    if (!mask || !B || !tile_col0 || !tile_width)
        return fail(TW_ERR_NULL, "mask, B or the tile table is NULL");
    const size_t b_bytes = (size_t)K * N * sizeof(float), m_bytes = (size_t)K * N;
    DeviceBuffer upload_buf;
    if (hipMalloc(&upload_buf.ptr, b_bytes + m_bytes) != hipSuccess)
        return fail(TW_ERR_ALLOC, "hipMalloc of %zu bytes for the mask and weight upload failed",
                    b_bytes + m_bytes);
    char *const buf = static_cast<char *>(upload_buf.ptr);
    hipError_t e = hipMemcpy(buf, B, b_bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess)
        e = hipMemcpy(buf + b_bytes, mask, m_bytes, hipMemcpyHostToDevice);
    return e == hipSuccess
               ? plan_from_device_mask(K, N, dtype, n_tiles, tile_col0, tile_width,
                                       reinterpret_cast<const uint8_t *>(buf + b_bytes),
                                       reinterpret_cast<const float *>(buf), cover, nullptr, out)
               : fail(TW_ERR_DEVICE, "mask / weight upload failed: %s", hipGetErrorString(e));
}

int tw_plan_from_device_mask(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                             const int32_t *tile_width, const uint8_t *mask, const float *B,
                             int cover, void *stream, tw_plan **out)
try {
    return plan_from_device_mask(K, N, dtype, n_tiles, tile_col0, tile_width, mask, B, cover != 0,
                                 (hipStream_t)stream, out);
}
TW_CATCH_TO_STATUS

int tw_plan_from_mask_tiles(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                            const int32_t *tile_width, const uint8_t *mask, const float *B,
                            tw_plan **out)
try {
    return plan_from_mask_impl(K, N, dtype, n_tiles, tile_col0, tile_width, mask, B, false, out);
}
TW_CATCH_TO_STATUS

int tw_plan_from_mask_cover(int K, int N, int dtype, int n_tiles, const int32_t *tile_col0,
                            const int32_t *tile_width, const uint8_t *mask, const float *B,
                            tw_plan **out)
try {
    return plan_from_mask_impl(K, N, dtype, n_tiles, tile_col0, tile_width, mask, B, true, out);
}
TW_CATCH_TO_STATUS

int tw_plan_from_export(int K, int N, int dtype, int n_kept_k, const int32_t *mask_i,
                        int n_kept_n, const int32_t *mask_o, const float *kernel, tw_plan **out)
try {
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (K <= 0 || N <= 0 || n_kept_k < 0 || n_kept_k > K || n_kept_n < 0 || n_kept_n > N)
        return fail(TW_ERR_SHAPE, "K=%d N=%d with %d kept rows and %d kept columns", K, N,
                    n_kept_k, n_kept_n);
    if ((n_kept_k > 0 && !mask_i) || (n_kept_n > 0 && !mask_o) ||
        (n_kept_k > 0 && n_kept_n > 0 && !kernel))
        return fail(TW_ERR_NULL, "mask_i, mask_o or kernel is NULL");
    std::vector<int32_t> kk((size_t)std::max(n_kept_k, 1)), kn((size_t)std::max(n_kept_n, 1));
    int st = tw_offsets_to_kept(mask_i, n_kept_k, K, kk.data());
    if (!st)
        st = tw_offsets_to_kept(mask_o, n_kept_n, N, kn.data());
    if (st)
        return st;
    // one tile over all columns: every unit of 128 compact columns shares the kept rows
    std::vector<float> B((size_t)K * N, 0.0f);
    for (int i = 0; i < n_kept_k; ++i) {
        float *dst = B.data() + (size_t)kk[i] * N;
        const float *src = kernel + (size_t)i * n_kept_n;
        for (int j = 0; j < n_kept_n; ++j)
            dst[kn[j]] = src[j];
    }
    const int32_t col0 = 0, width = N;
    const int32_t kp[2] = {0, n_kept_k}, np[2] = {0, n_kept_n};
    return tw_plan_create(K, N, dtype, 1, &col0, &width, kp, kk.data(), np, kn.data(), B.data(),
                          out);
}
TW_CATCH_TO_STATUS

int tw_plan_from_stream_operands(int M, int N, int K, int dtype, const void *B_stream,
                                 int block_num, const int32_t *N_cal, const int32_t *K_cal,
                                 const int32_t *const *mask_n, const int32_t *const *mask_k,
                                 const int64_t *off_B, const int64_t *off_C, tw_plan **out)
try {
    if (!out)
        return fail(TW_ERR_NULL, "out is NULL");
    *out = nullptr;
    int st = check_dtype(dtype);
    if (st)
        return st;
    if (M <= 0 || N <= 0 || K <= 0 || block_num <= 0)
        return fail(TW_ERR_SHAPE, "M=%d N=%d K=%d block_num=%d must all be positive", M, N, K,
                    block_num);
    if (!B_stream || !N_cal || !K_cal || !mask_n || !mask_k || !off_B || !off_C)
        return fail(TW_ERR_NULL, "an operand pointer is NULL");
    std::vector<int32_t> col0(block_num), width(block_num), kp(block_num + 1, 0),
        np(block_num + 1, 0), ki, ni;
    for (int t = 0; t < block_num; ++t) {
        if (off_C[t] % M != 0)
            return fail(TW_ERR_TILE_TABLE, "off_C[%d] = %lld is not a multiple of M", t,
                        (long long)off_C[t]);
        col0[t] = (int32_t)(off_C[t] / M);
        if (N_cal[t] < 0 || K_cal[t] < 0 || K_cal[t] > K)
            return fail(TW_ERR_SHAPE, "tile %d: N_cal=%d K_cal=%d", t, N_cal[t], K_cal[t]);
        if ((N_cal[t] > 0 && !mask_n[t]) || (K_cal[t] > 0 && !mask_k[t]))
            return fail(TW_ERR_NULL, "mask pointer of tile %d is NULL", t);
    }
    for (int t = 0; t < block_num; ++t) {
        const int next = t + 1 < block_num ? col0[t + 1] : N;
        width[t] = next - col0[t];
        if (width[t] <= 0 || N_cal[t] > width[t])
            return fail(TW_ERR_TILE_TABLE, "tile %d: width %d, N_cal %d", t, width[t], N_cal[t]);
        if (off_B[t] < 0 || off_B[t] + (int64_t)std::max(N_cal[t] - 1, 0) * K + K_cal[t] >
                                (int64_t)K * N)
            return fail(TW_ERR_SHAPE, "off_B[%d] = %lld leaves the K*N weight buffer", t,
                        (long long)off_B[t]);
        std::vector<int32_t> rel_k(K_cal[t]), rel_n(N_cal[t]);
        if (K_cal[t])
            TW_HIP(hipMemcpy(rel_k.data(), mask_k[t], sizeof(int32_t) * K_cal[t],
                             hipMemcpyDeviceToHost));
        if (N_cal[t])
            TW_HIP(hipMemcpy(rel_n.data(), mask_n[t], sizeof(int32_t) * N_cal[t],
                             hipMemcpyDeviceToHost));
        size_t k0 = ki.size(), n0 = ni.size();
        ki.resize(k0 + K_cal[t]);
        ni.resize(n0 + N_cal[t]);
        if ((st = tw_offsets_to_kept(rel_k.data(), K_cal[t], K, ki.data() + k0)) ||
            (st = tw_offsets_to_kept(rel_n.data(), N_cal[t], width[t], ni.data() + n0)))
            return st;
        kp[t + 1] = (int32_t)ki.size();
        np[t + 1] = (int32_t)ni.size();
    }
    st = validate_lists(K, N, block_num, col0.data(), width.data(), kp.data(), ki.data(), np.data(),
                        ni.data());
    if (st)
        return st;
    PlanOwner owner;
    tw_plan *p = owner.p = new (std::nothrow) tw_plan;
    if (!p)
        return fail(TW_ERR_ALLOC, "out of host memory");
    p->K = K;
    p->N = N;
    p->dtype = dtype;
    p->n_tiles = block_num;
    p->tile_col0 = col0;
    p->tile_width = width;
    p->kept_k_ptr = kp;
    p->kept_n_ptr = np;
    p->kept_k_idx = ki;
    p->kept_n_idx = ni;
    if ((st = finalize_plan_geometry(p, nullptr)) ||
        (st = pack_from_stream(p, B_stream, off_B, nullptr)))
        return st;
    *out = owner.release();
    return TW_OK;
}
TW_CATCH_TO_STATUS

int tw_plan_info(const tw_plan *p, int64_t *info, int n_info)
{
    if (!p || !info)
        return fail(TW_ERR_NULL, "plan or info is NULL");
    int64_t v[12] = {0};
    v[0] = p->K;
    v[1] = p->N;
    v[2] = p->dtype;
    v[3] = p->n_tiles;
    for (int t = 0; t < p->n_tiles; ++t) {
        const int64_t kt = p->kept_k_ptr[t + 1] - p->kept_k_ptr[t];
        const int64_t nt = p->kept_n_ptr[t + 1] - p->kept_n_ptr[t];
        v[4] += kt;
        v[5] += nt;
        v[6] += kt * nt;
        v[8] = std::max(v[8], kt);
        v[9] = std::max(v[9], nt);
        v[10] += (kt * nt == 0);
        v[11] += p->tile_width[t];
    }
    v[7] = p->packed_elems * 2;
    for (int i = 0; i < n_info && i < 12; ++i)
        info[i] = v[i];
    return TW_OK;
}

int tw_plan_export(const tw_plan *p, int32_t *tile_col0, int32_t *tile_width, int32_t *kept_k_ptr,
                   int32_t *kept_k_idx, int32_t *mask_k_rel, int32_t *kept_n_ptr,
                   int32_t *kept_n_idx, int32_t *mask_n_rel, uint16_t *B_stream)
try {
    if (!p)
        return fail(TW_ERR_NULL, "plan is NULL");
    const int nt = p->n_tiles;
    if (tile_col0)
        memcpy(tile_col0, p->tile_col0.data(), sizeof(int32_t) * nt);
    if (tile_width)
        memcpy(tile_width, p->tile_width.data(), sizeof(int32_t) * nt);
    if (kept_k_ptr)
        memcpy(kept_k_ptr, p->kept_k_ptr.data(), sizeof(int32_t) * (nt + 1));
    if (kept_n_ptr)
        memcpy(kept_n_ptr, p->kept_n_ptr.data(), sizeof(int32_t) * (nt + 1));
    const size_t sk = p->kept_k_idx.size(), sn = p->kept_n_idx.size();
    // the index lists come back from the device copies the kernels read
    if (kept_k_idx && sk)
        TW_HIP(hipMemcpy(kept_k_idx, p->d_kept_k, sizeof(int32_t) * sk, hipMemcpyDeviceToHost));
    if (mask_k_rel && sk)
        TW_HIP(hipMemcpy(mask_k_rel, p->d_rel_k, sizeof(int32_t) * sk, hipMemcpyDeviceToHost));
    if (kept_n_idx && sn)
        TW_HIP(hipMemcpy(kept_n_idx, p->d_kept_n, sizeof(int32_t) * sn, hipMemcpyDeviceToHost));
    if (mask_n_rel && sn)
        TW_HIP(hipMemcpy(mask_n_rel, p->d_rel_n, sizeof(int32_t) * sn, hipMemcpyDeviceToHost));
    if (B_stream) {
        DeviceBuffer d_Bs;
        const size_t bytes = (size_t)p->K * p->N * 2;
        if (hipMalloc(&d_Bs.ptr, bytes) != hipSuccess)
            return fail(TW_ERR_ALLOC, "hipMalloc of %zu bytes failed", bytes);
        if (int st = unpack_to_stream(p, static_cast<uint16_t *>(d_Bs.ptr), nullptr))
            return st;
        const hipError_t e = hipMemcpy(B_stream, d_Bs.ptr, bytes, hipMemcpyDeviceToHost);
        if (e != hipSuccess)
            return fail(TW_ERR_DEVICE, "read-back failed: %s", hipGetErrorString(e));
    }
    return TW_OK;
}
TW_CATCH_TO_STATUS

int tw_plan_destroy(tw_plan *plan)
{
    free_plan(plan);
    return TW_OK;
}

} // extern "C"
