// Internal declarations shared by the host code and the HIP kernels of libtwgemm.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <new>
#include <string>
#include <vector>

#include "twgemm.h"

namespace tw {

// Geometry shared by the pack kernel and the GEMM kernels.
constexpr int kMfmaN = 32;    // columns of one MFMA block (packing granularity in n)
constexpr int kMfmaK = 16;    // k extent of one v_mfma_f32_32x32x16
constexpr int kBlockK = 64;   // k rows per packed weight step; K_t is padded to this
constexpr int kMaxUnitN = 128; // compact columns handled by one work item
constexpr int kTicketSlots = 256;
constexpr int kEagerSlots = 192;  // slots of eager launches; the rest serve launches recorded in graphs
constexpr int kMaxArgUnits = 32;
constexpr int kBalColumns = 8; // columns of the item matrix that may have row blocks of their own height

// One schedulable piece of a tile: at most kMaxUnitN compact columns.
// 48 bytes; read with scalar loads.
struct UnitDev {
    int32_t col0;     // first original column of the tile in C
    int32_t k_kept;   // K_t
    int32_t k_pad;    // K_t rounded up to kBlockK
    int32_t n_cnt;    // compact columns in this unit
    int32_t nb0;      // first 32-column block of the tile's packed weight used here
    int32_t nb_cnt;   // 32-column blocks in this unit
    int32_t kk_off;   // offset of the tile's kept_k list in the padded array (k_pad entries)
    int32_t kn_off;   // offset of this unit's first compact column in kept_n
    int64_t b_off;    // element offset of the tile's packed weight
    int32_t tile;     // owning tile
    int32_t nblk;     // 32-column blocks of the whole tile (n_pad / 32)
};

// Zero-fill work for TW_PRUNED_ZERO: the pruned columns of one tile.
struct TileDev {
    int32_t col0;
    int32_t n_pruned; // pruned original columns in the tile
    int32_t pn_off;   // offset into pruned_n
    int32_t pad_;
};

// The work of one launch is a matrix of items: `n_all_u` columns (pieces of units that have kept
// K rows first, heaviest first; then pieces of units without; then, with TW_PRUNED_ZERO, the tiles
// whose pruned columns are filled) by `n_mblk` blocks of BM rows.  It is handed out through
// kXcd queues, one per accelerator die: workgroup b runs on die b % kXcd and draws from that
// die's queue only, so the workgroups that share an L2 work on the same rows of A.  Queue x owns
// the row blocks [x * n_own, (x + 1) * n_own) (all their items, row block after row block) and
// every kXcd-th item of the remaining `n_tail_mblk` row blocks (unit after unit).
constexpr int kXcd = 8;
constexpr int kTicketInts = 16; // per slot: [0, kXcd) next index of each queue, [kXcd] workgroups done

struct GemmArgs {
    const UnitDev *units;   // sorted by k_kept descending
    const TileDev *tiles;
    const int32_t *kept_k;
    // The kept-K lists once more for the A-stationary kernel: one word per lane and group of 16
    // k rows, the two rows a lane addresses in the group as 16-bit halves.  Entry
    // kk_off / 2 + step * 32 + e * 4 + group holds rows (e / 4) * 8 + e % 4 and that + 4 of the
    // group, so that the four words of a step a lane needs are one 16-byte load (null when K
    // does not fit 16 bits).  The padding of a list up to whole steps names row K: the kernel keeps
    // a row of zeros there, behind its panel of A.
    const uint32_t *kept_pairs;
    const int32_t *kept_n;
    const int32_t *pruned_n;
    const void *Bp;
    const void *A;
    void *C;
    int64_t lda, ldc;
    int32_t M;
    int32_t n_mblk;       // ceil(M / BM)
    int32_t n_split;      // a unit is handed out as n_split pieces of 32 * piece_nb compact columns
    int32_t piece_nb;
    int32_t n_pipe_u;     // pieces of units with at least one kept K row
    int32_t n_gemm_u;     // + pieces of units without (their columns receive beta * C)
    int32_t n_all_u;      // + tiles with pruned columns to fill
    int32_t n_own;        // row blocks owned by each queue
    int32_t n_own_items;  // n_own * n_all_u
    int32_t n_tail_mblk;  // n_mblk - kXcd * n_own
    int32_t n_tail_items; // n_tail_mblk * n_all_u
    float alpha, beta;
    const float *bias;    // fp32 [N] added to every written column before the activation, or null
    int32_t act;          // TW_ACT_*
    int32_t store_through; // output stores write through to memory (large outputs) or stay in L2
    int32_t *ticket;      // kTicketInts counters, zero between launches
    // Row blocks sized per column of the item matrix (n_bal > 0: one list of items for all
    // queues, n_own == 0, n_tail_items items): column u has items of bal_rows[u] rows, the items
    // bal_first[u] .. bal_first[u + 1] - 1 of the list.  See balance_items.
    int32_t n_bal;
    // The 256 x 128 kernel in its direct-to-LDS form: bytes of A (K * lda elements) and
    // of the packed weight, the sizes of the two buffers its loads are checked against.
    int32_t lds_dma;
    uint32_t a_bytes, b_bytes;
    int32_t rb_major;     // the items no queue owns are dealt out row block after row block instead of column after column
    int32_t bal_first[kBalColumns + 1];
    int32_t bal_rows[kBalColumns];
    // Copy of `units` inside the kernel arguments for plans of at most kMaxArgUnits units
    // (n_arg_units == 0 otherwise): a workgroup then reads its first unit through the scalar
    // cache instead of waiting for a global load before it can fetch anything else.
    int32_t n_arg_units;
    UnitDev arg_units[kMaxArgUnits];
};

} // namespace tw

struct tw_plan {
    int K = 0, N = 0, dtype = 0, n_tiles = 0;
    int device = 0;
    // host copies
    std::vector<int32_t> tile_col0, tile_width, kept_k_ptr, kept_k_idx, kept_n_ptr, kept_n_idx;
    std::vector<int32_t> k_pad, n_pad;
    std::vector<int64_t> b_off; // element offset of each tile's packed weight
    int64_t packed_elems = 0;
    int n_units = 0, n_pipe_units = 0, n_zero_tiles = 0, max_unit_n = 0;
    std::vector<tw::UnitDev> h_units; // host copy of d_units (queue order)
    // device
    int32_t *d_kept_k = nullptr, *d_kept_n = nullptr, *d_rel_k = nullptr, *d_rel_n = nullptr;
    int32_t *d_pruned_n = nullptr;
    int32_t *d_kept_k_pad = nullptr; // per tile k_pad entries at 4-aligned offsets (kernel's copy)
    tw::UnitDev *d_units = nullptr;
    tw::TileDev *d_tiles = nullptr;
    void *d_Bp = nullptr;
    int32_t *d_tickets = nullptr; // kTicketSlots slots of kTicketInts counters
    // every (unit, 32-column block) pair of the plan, in unit order: unit * 4 + block (the work
    // list of the A-stationary kernel)
    int32_t *d_blocks = nullptr;
    int n_blocks = 0;
    uint32_t *d_kept_pairs = nullptr; // GemmArgs::kept_pairs
    // Ownership: every pointer above points into one of these two allocations.  d_lists holds the
    // four index arrays when the pre-pass compacted them on the device (else they sit in d_slab);
    // d_slab holds the unit / tile tables, the pruned-column and padded kept-K lists, the packing
    // table, the ticket slots and the packed weight.
    void *d_lists = nullptr;
    void *d_slab = nullptr;
    void *d_pack_tiles = nullptr; // tw::PackTile[n_tiles] for packing from a dense weight
    mutable unsigned next_slot = 0, next_capture_slot = 0;
    int blocks_per_unit = 0; // 32-column blocks of every unit where all units have the same number, else 0
    int n_halves = 0;   // pieces of 64 compact columns over all units (the skinny kernel's work per row block)
    bool rows_shared = false; // the tiles that keep rows keep nearly all of them (a dense or almost dense plan)
    int max_k_pad = 0;        // most kept rows of a tile, rounded up to whole steps
    int64_t pipe_steps = 0;   // steps of 64 kept rows over all units that have any
    int cu_count = 0;
};

namespace tw {

void set_error(const char *fmt, ...);
int get_option(int option_id);
// once per device: symbol look-ups and function attributes, which HIP refuses while a stream is
// being captured; run by every plan when it is built and again (one flag load) by the launches
int prepare_device(); // a tw_set_option value, or -1
int fail(int status, const char *fmt, ...);

#define TW_HIP(call)                                                                     \
    do {                                                                                 \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess)                                                            \
            return ::tw::fail(TW_ERR_DEVICE, "%s failed: %s", #call, hipGetErrorString(e_)); \
    } while (0)

// Closes a function-try-block of a C-ABI entry point: no C++ exception crosses the boundary.
#define TW_CATCH_TO_STATUS                                                               \
    catch (const std::bad_alloc &)                                                       \
    {                                                                                    \
        return ::tw::fail(TW_ERR_ALLOC, "out of host memory");                           \
    }                                                                                    \
    catch (const std::exception &e)                                                      \
    {                                                                                    \
        return ::tw::fail(TW_ERR_ALLOC, "host-side failure: %s", e.what());              \
    }

// validation shared by the plan builders (host only)
int validate_lists(int K, int N, int n_tiles, const int32_t *tile_col0, const int32_t *tile_width,
                   const int32_t *kept_k_ptr, const int32_t *kept_k_idx,
                   const int32_t *kept_n_ptr, const int32_t *kept_n_idx);

// fills the host-side geometry (k_pad, n_pad, b_off, packed_elems) of a plan whose
// lists are set, uploads lists/units/tiles and allocates the packed weight (zeroed); the copies
// run on `s`, which is waited for.
int finalize_plan_geometry(tw_plan *p, hipStream_t s);

// device pack: packed weight from a row-major fp32 [K,N] device buffer
int pack_from_dense(tw_plan *p, const float *d_B, hipStream_t s, const uint8_t *d_mask = nullptr);
// device pack: packed weight from the reference's compacted stream layout (16-bit, device)
int pack_from_stream(tw_plan *p, const void *d_Bs, const int64_t *off_B, hipStream_t s);
// true when tw_gemm_ex takes a row-major A and a row-major C of this plan with a kernel of its own
// (no layout-generic kernel, no staging): K short enough for a panel of A in LDS and C not read
bool takes_row_major_directly(const tw_plan *p, float beta);
// the weight-stationary kernel (tw_gemm_bs.hip): whether it takes the plan, and its launch with
// `per_cu` workgroups meant to share a compute unit
bool bs_takes(const tw_plan *p, int64_t lda, int64_t ldc, bool reads_c);
int launch_bs(const tw_plan *p, const GemmArgs &a, int per_cu, hipStream_t s);
double bs_fill(const tw_plan *p, int M); // share of the chip's workgroup slots its launch fills
// device unpack: compacted stream layout (K*N 16-bit, zero elsewhere) from the packed weight
int unpack_to_stream(const tw_plan *p, uint16_t *d_Bs, hipStream_t s);

} // namespace tw
