/*
 * torchex_scatter.h -- C ABI of the MI355X (gfx950) voxel scatter-reduction
 * library, libtorchex_scatter.so.
 *
 * Plain C: device pointers, 64-bit sizes, an opaque stream handle
 * (a hipStream_t passed as void*; NULL = the null stream) and an int status.
 * No torch type crosses this line.  The library allocates no device memory:
 * every buffer, workspaces included, is owned by the caller.  Calls are
 * asynchronous on `stream` and re-entrant, with one exception that says so:
 * txs_scatter_forward_resident, which uses a table inside the library.
 * State the library keeps, all of it per GPU, filled on first use and never changed
 * afterwards (so it does not make two calls depend on each other): the number of
 * compute units (sizes the table-mode launch), a flag per kernel that its dynamic-LDS
 * limit has been raised, and the device address of the resident table.
 *
 * Each entry point names the reference interface it stands in for
 * (paths relative to the TorchEx tree).
 *
 * Data layout
 *   feats      [N, C]   row-major contiguous, dtype fp32 / fp16 / bf16
 *   unq_inv    [N]      int32 voxel id of every row, any order, ids in [0, U)
 *   preSum     [U+1]    int32 CSR offsets: rows of voxel u occupy sorted
 *                       positions preSum[u] .. preSum[u+1]-1
 *   perm       [N]      int32 row id at each sorted position (stable: ascending
 *                       row inside a voxel); NULL when unq_inv is already
 *                       non-decreasing (position == row)
 *   seg        [N]      int32 voxel id at each sorted position, bit 31 set when
 *                       the voxel is "special" (see below)
 *   slot_of    [U]      int32 >= 0 for a special voxel (for a heavy one: its slot
 *                       in heavy_ids and its row in scratch), else -1
 *   heavy_ids  [n_special] int32 ids of the special voxels, the n_heavy heavy
 *                       ones first (slot order), the empty ones after them
 *   scratch    8-byte cells: first [n_heavy * C], one row per heavy voxel, which
 *                       MUST BE ZERO ON ENTRY to txs_scatter_forward and are zero again
 *                       when the call's kernels have finished; behind them, room for
 *                       the partial tables of table mode (never read before written,
 *                       left dirty).  txs_scatter_scratch_cells() gives the total.
 *   out        [U, C]   dtype of feats;  arg [U, C] int32 (row index into feats)
 *
 * Table mode: when there are few voxels with many rows each (at least 512 rows per
 * voxel on average) and a whole [U, C] table fits in the LDS of a compute unit, forward
 * and backward run in ROW order instead of voxel order: the forward reduces contiguous
 * spans of rows into per-workgroup LDS tables (LDS atomics), stores them as partial
 * tables in `scratch` and combines them in a second kernel; the backward stages the
 * upstream rows in LDS and writes the input gradient sequentially.  Rows narrower than
 * a cache line are then read and written as a stream instead of one by one.  Table mode
 * needs the row-order ids (unq_inv, or grouped rows) and, forward, the extra scratch.
 *
 * Special voxels: a voxel with more than `heavy_threshold` rows is reduced by
 * many wavefronts whose partials meet in `scratch` through atomics (fp32
 * atomic add for sum/mean, 64-bit atomic max on a packed value|row word for
 * max); a voxel with zero rows is special too so that it still gets an output
 * row.  All other voxels are reduced in registers by one group of lanes and
 * written once.
 */
#ifndef TORCHEX_SCATTER_H
#define TORCHEX_SCATTER_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    TXS_OK = 0,
    TXS_ERR_INVALID_ARG = 1,
    TXS_ERR_LAUNCH = 2,
    TXS_ERR_UNSUPPORTED = 3,
    TXS_ERR_TOO_LARGE = 4 /* txs_scatter_forward_resident: num_heavy * channel exceeds the resident table */
};
enum { TXS_F32 = 0, TXS_F16 = 1, TXS_BF16 = 2 };
enum { TXS_SUM = 0, TXS_MEAN = 1, TXS_MAX = 2, TXS_MAX_REFTIE = 3 };
/* Which kernels a forward / backward call may use: the library's choice, the voxel-order
 * kernels only, or the row-order table kernels only (TXS_ERR_UNSUPPORTED if they do not
 * apply to the call). */
enum { TXS_PATH_AUTO = 0, TXS_PATH_VOXEL_ORDER = 1, TXS_PATH_TABLE = 2 };

/* Slots of the int32[TXS_STATS_LEN] device array the plan functions fill. */
enum {
    TXS_STAT_UNSORTED = 0,     /* 1 if unq_inv[i] > unq_inv[i+1] for some i */
    TXS_STAT_OUT_OF_RANGE = 1, /* 1 if some id is outside [0, U) */
    TXS_STAT_MAX_CNT = 2,      /* largest voxel population */
    TXS_STAT_NUM_SPECIAL = 3,  /* number of special voxels (heavy or empty) */
    TXS_STAT_NUM_EMPTY = 4,    /* number of voxels with zero rows */
    TXS_STAT_COUNT_MISMATCH = 5, /* 1 if the caller's unq_cnts is not the histogram of unq_inv */
    TXS_STAT_NUM_UNQ = 6,      /* number of distinct keys found by txs_unique_runs */
    TXS_STAT_NUM_HEAVY = 7,    /* number of voxels above the heavy threshold (NUM_SPECIAL - NUM_EMPTY) */
    TXS_STAT_NEED_GENERAL = 8, /* txs_plan_build only: 1 if it left the outputs unwritten (see there) */
    TXS_STATS_LEN = 16
};

/* Library ABI version (8); bumped when a signature or the meaning of an argument changes. */
int txs_abi_version(void);

/* Human-readable text for a status code. */
const char *txs_status_string(int status);

/* Name of the kernel instantiation that txs_scatter_forward (backward == 0) or
 * txs_scatter_backward (backward != 0) launches for these extents, as a profiler lists
 * it without namespaces ("scatter_fwd_kernel<F32,4,MAX>": dtype, elements per lane,
 * operator; "scatter_bwd_kernel<F32,4,MAX,8>": the same and the chunk length).  pointer_alignment is
 * the alignment in bytes of the least aligned tensor (16 for ordinary allocations);
 * table_allowed != 0 means the call would be made with TXS_PATH_AUTO, row-order ids and
 * enough scratch ("table_fwd_kernel<F32,4,MAX>" is then reported where table mode applies).
 * For logs and benchmarks; buf needs at least 48 bytes. */
int txs_kernel_name(int backward, int op, int dtype, int64_t num_total, int64_t channel,
                    int64_t num_unq, int64_t pointer_alignment, int table_allowed, char *buf,
                    int64_t buf_len);

/* Default population above which a voxel is reduced through atomics (64), and the
 * smallest heavy_threshold the plan functions accept (16: a smaller one is refused with
 * TXS_ERR_INVALID_ARG). */
int txs_default_heavy_threshold(void);
int txs_chunk_rows(void);

/* ---- index preparation (what ScatterData.__init__ computes) --------------- */

/* Replaces getPreSum_launcher (torchex/src/scatter/scatter.cpp:18, kernel
 * scatter_kernel.cu:85-100): CSR offsets from the run boundaries of a SORTED
 * unq_inv.  preSum has `num_presum` entries and must be zero-filled by the
 * caller (torchex/operator_py/scatter_op.py:126); writes outside it are
 * dropped. */
int txs_get_presum(const int32_t *unq_inv, int32_t *preSum, int64_t num_total,
                   int64_t num_presum, void *stream);

/* Order and range flags of unq_inv: sets stats[UNSORTED] / stats[OUT_OF_RANGE].
 * First step of what ScatterData.__init__ (scatter_op.py:13-21) does, extended
 * to unsorted input.  stats [TXS_STATS_LEN] must be zero-filled by the caller;
 * the plan calls below accumulate into it and nothing is read back by the
 * library, so the whole plan needs one host synchronisation (to read stats). */
int txs_plan_check(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, int32_t *stats,
                   void *stream);

/* Sorted keys and the stable permutation: keys[j] = voxel id at sorted position
 * j, perm[j] = its row (ascending rows inside a voxel).  LSD radix sort, three
 * kernels per pass, no inter-block spinning.  When stats[UNSORTED] is 0 (read
 * on the device) the passes return at once, keys becomes a copy of unq_inv and
 * perm is left unwritten (position == row).  sort_ws: int32 workspace of
 * txs_sort_workspace_len(num_total, num_unq) entries. */
int txs_plan_sort(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, const int32_t *stats,
                  int32_t *perm, int32_t *keys, int32_t *sort_ws, void *stream);
int64_t txs_sort_workspace_len(int64_t num_total, int64_t num_unq);

/* CSR offsets from sorted keys: preSum[u] = first sorted position with key >= u,
 * preSum[num_unq] = num_total (no atomics, no scan).  On sorted input this is
 * what txs_get_presum / the reference's getPreSum produce, with empty voxels
 * handled too. */
int txs_plan_presum(const int32_t *sorted_keys, int64_t num_total, int64_t num_unq,
                    int32_t *preSum, void *stream);

/* Table of special voxels (heavy or empty) from CSR offsets, stats[MAX_CNT],
 * stats[NUM_SPECIAL], stats[NUM_HEAVY], stats[NUM_EMPTY]; when unq_cnts (int64 [num_unq], as
 * torch.unique returns it) is given, stats[COUNT_MISMATCH] is set if it is not
 * the histogram of unq_inv (the consistency check of scatter_op.py:19).
 * heavy_ids must hold num_unq entries: on return its first NUM_HEAVY entries
 * are the heavy voxels and its LAST NUM_EMPTY entries the empty ones; the list
 * txs_scatter_forward takes is those two pieces put together, heavy first.
 * num_unq_dev (may be NULL): device int holding the true voxel count when the
 * host only knows the upper bound passed as num_unq (after txs_unique_runs).
 * cnts_out (may be NULL): int64 [num_unq] voxel populations, the unq_cnts of
 * torch.unique. */
int txs_plan_special(const int32_t *preSum, int64_t num_unq, int32_t heavy_threshold,
                     const int64_t *unq_cnts, int32_t *slot_of, int32_t *heavy_ids, int32_t *stats,
                     const int32_t *num_unq_dev, int64_t *cnts_out, void *stream);

/* Everything ScatterData.__init__ needs, in one call: order/range flags, the stable
 * permutation, CSR offsets, special-voxel table, statistics and the flagged per-position
 * ids (what txs_plan_check, txs_plan_sort, txs_plan_presum, txs_plan_special and
 * txs_plan_seg_flag produce one after the other).  Up to 2^22 voxels this runs as a
 * bucket sort -- tile histograms of the high digit of the ids; scan; stable scatter by
 * bucket; then workgroups that sort a bucket's low digit in LDS and write the bucket's
 * slice of all outputs -- beyond that it runs the calls named above.
 * stats [TXS_STATS_LEN] needs no initialisation for up to 2^22 voxels (also with no rows or
 * no voxels at all: the call clears it) and must be zero-filled by the caller beyond
 * (zero-filling always is fine); perm is left unwritten when
 * stats[UNSORTED] stays 0.  unq_cnts may be NULL.  slot_of and heavy_ids may both be NULL
 * for a caller that wants the order and the offsets only (the ranks of ingroup_inds): no
 * special-voxel table is made then, seg carries plain ids, and of the statistics only
 * UNSORTED, OUT_OF_RANGE and NEED_GENERAL are set.  plan_ws: int32 workspace of
 * txs_plan_workspace_len(num_total, num_unq) entries, 8-byte aligned.
 * One bucket holding more than 262,144 rows (a few voxels that own most of the rows)
 * makes the bucket kernels step aside: stats[NEED_GENERAL] is then 1, only
 * stats[UNSORTED] and stats[OUT_OF_RANGE] are valid, and the caller zero-fills stats
 * again and calls txs_plan_build_general with the same arguments. */
int txs_plan_build(const int32_t *unq_inv, int64_t num_total, int64_t num_unq,
                   int32_t heavy_threshold, const int64_t *unq_cnts, int32_t *plan_ws,
                   int32_t *perm, int32_t *seg, int32_t *preSum, int32_t *slot_of,
                   int32_t *heavy_ids, int32_t *stats, void *stream);
int64_t txs_plan_workspace_len(int64_t num_total, int64_t num_unq);
/* The same outputs through the general sequence (any number of voxels, any occupancy). */
int txs_plan_build_general(const int32_t *unq_inv, int64_t num_total, int64_t num_unq,
                           int32_t heavy_threshold, const int64_t *unq_cnts, int32_t *plan_ws,
                           int32_t *perm, int32_t *seg, int32_t *preSum, int32_t *slot_of,
                           int32_t *heavy_ids, int32_t *stats, void *stream);

/* In place: sorted keys -> seg (sets bit 31 on positions of special voxels). */
int txs_plan_seg_flag(int32_t *keys_to_seg, int64_t num_total, int64_t num_unq,
                      const int32_t *slot_of, void *stream);

/* Turns the num_heavy heavy voxels at the front of heavy_ids back into ordinary ones: bit 31
 * comes off their positions in seg, slot_of becomes -1, stats[NUM_HEAVY] = 0 and
 * stats[NUM_SPECIAL] = stats[NUM_EMPTY]; the caller then passes only the empty voxels as
 * the special list.  For a plan with a handful of voxels just above the heavy threshold
 * (a LiDAR sweep in 0.2 m voxels: 8 of 326,859, the fullest with 69 rows): the forward
 * reduces such runs in registers and LDS like any other, a run may only not reach much
 * further than the 64 positions a tile stages behind its end (the rest is then read row by
 * row), and without heavy voxels the forward call needs no second kernel.  (Part of the
 * index preparation that extends scatter_op.py:13-21; the reference has no heavy voxels.) */
int txs_plan_demote_heavy(const int32_t *preSum, int32_t *seg, int32_t *slot_of,
                          const int32_t *heavy_ids, int64_t num_heavy, int64_t num_total,
                          int64_t num_unq, int32_t *stats, void *stream);

/* seg by binary search of each position in preSum, for callers that hold only
 * CSR offsets of already grouped rows (the reference's scatter_ext.sum /
 * scatter_ext.max argument lists, scatter.cpp:20-53). */
int txs_plan_seg_from_presum(const int32_t *preSum, int64_t num_total, int64_t num_unq,
                             const int32_t *slot_of, int32_t *seg, void *stream);

/* ---- callers on either side of the path ------------------------------------ */

/* Dynamic voxelization front-end: per point, coors = floor((p - range_lo) /
 * voxel_size) with the arithmetic of torch.div(..., rounding_mode='floor') on
 * fp32 (the reference's voxelize_single, test/test_incremental_mask.py:20-26)
 * and key = (x * dims[1] + y) * dims[2] + z (operator_py/incremental_points.py:
 * 18-19, operator_py/grid_hash.py:14).  points: [num_total, point_stride] fp32,
 * xyz first.  range_lo / voxel_size / dims are HOST arrays of 3.  coors (may be
 * NULL): int32 [num_total, 3].  A point outside the grid sets
 * stats[OUT_OF_RANGE] and gets key 0. */
int txs_voxel_keys(const float *points, int64_t num_total, int64_t point_stride,
                   const float *range_lo, const float *voxel_size, const int32_t *dims,
                   int32_t *coors, int32_t *keys, int32_t *stats, void *stream);

/* What torch.unique(keys, return_inverse=True, return_counts=True) computes,
 * fused with the plan: from keys sorted by txs_plan_sort (called with the key
 * bound in place of num_unq) it writes unq_keys [<= num_total] (ascending),
 * unq_inv [num_total] (int32), preSum, seg (dense voxel id per sorted
 * position) and stats[NUM_UNQ]; follow with txs_plan_special (num_unq_dev =
 * &stats[NUM_UNQ], cnts_out for the counts) and txs_plan_seg_flag.  One sort
 * serves both the unique and the scatter plan.  unique_ws: int32 workspace of
 * txs_unique_workspace_len(num_total) entries. */
int txs_unique_runs(const int32_t *sorted_keys, const int32_t *perm, int64_t num_total,
                    int32_t *unique_ws, int32_t *seg, int32_t *unq_inv, int32_t *unq_keys,
                    int32_t *preSum, int32_t *stats, void *stream);
int64_t txs_unique_workspace_len(int64_t num_total);

/* The same triple without a sort, for keys from a bounded grid (a voxelised point cloud: what
 * test/test_incremental_mask.py:20-26 followed by a torch.unique computes).  An occupancy
 * map of the key space -- one byte per key set by plain stores, then packed to one bit per
 * key -- gives every key its dense id: the number of occupied keys below it, i.e. the
 * unq_inv of torch.unique(keys, return_inverse=True), whose ids ascend with the keys.
 *   txs_unique_bitmap_count   builds the map and writes the number of distinct keys to
 *                             stats[NUM_UNQ]; stats[OUT_OF_RANGE] is set if a key is outside
 *                             [0, key_bound) (the array is not cleared first).
 *   txs_unique_bitmap_assign  writes unq_inv [num_total] and the ascending unq_keys
 *                             [up to min(num_total, key_bound)] from the same workspace.
 * A caller reads NUM_UNQ back while the second call runs, then builds the plan of unq_inv
 * (txs_plan_build) and takes the counts from its offsets (txs_counts_from_presum).
 * keys: int32, or int64 when key_is_int64 is non-zero (torch.unique's input as it comes).
 * The cost grows with key_bound (the map is cleared and read once), so this pays when the
 * grid is not much larger than the input.  bitmap_ws: int32 workspace of
 * txs_unique_bitmap_workspace_len(key_bound) entries, 16-byte aligned. */
int txs_unique_bitmap_count(const void *keys, int key_is_int64, int64_t num_total,
                            int64_t key_bound, int32_t *bitmap_ws, int32_t *stats, void *stream);
int txs_unique_bitmap_assign(const void *keys, int key_is_int64, int64_t num_total,
                             int64_t key_bound, const int32_t *bitmap_ws, int32_t *unq_inv,
                             int32_t *unq_keys, void *stream);
int64_t txs_unique_bitmap_workspace_len(int64_t key_bound);

/* unq_cnts[u] = preSum[u + 1] - preSum[u] as int64: the counts torch.unique(...,
 * return_counts=True) returns, which ScatterData keeps (scatter_op.py:14-17). */
int txs_counts_from_presum(const int32_t *preSum, int64_t num_unq, int64_t *unq_cnts, void *stream);


/* Rank of every element inside its group, from the plan of its group ids:
 * out[row] = sorted position - preSum[group].  Replaces ingroup_inds_launcher
 * (torchex/src/ingroup_inds/ingroup_inds.cpp:14-19, kernel
 * ingroup_inds_kernel.cu:17-30); ranks ascend with the element index inside a
 * group (the reference's atomic counter gives them in arbitrary order). */
int txs_ingroup_inds(const int32_t *seg, const int32_t *perm, const int32_t *preSum,
                     int64_t num_total, int64_t num_unq, int64_t *out, void *stream);

/* The whole of ingroup_inds (operator_py/ingroup_inds_op.py:10-27) in one call: the index
 * preparation of the group ids (order and offsets only) and the ranks, queued together; for
 * up to 2^22 groups the kernels that place the rows write the ranks themselves and leave
 * perm / seg unwritten.  num_groups: an upper bound of the ids (num_total serves for the
 * inverse of a unique).  plan_ws, perm, seg, preSum, stats as for txs_plan_build (stats
 * zero-filled).  On return stats[OUT_OF_RANGE] tells of an id outside [0, num_groups) and
 * stats[NEED_GENERAL] of a bucket too crowded for the bucket kernels: in both cases `out` is
 * not valid and the caller ranks again (with the true bound, or through
 * txs_plan_build_general followed by txs_ingroup_inds). */
int txs_group_ranks(const int32_t *group_ids, int64_t num_total, int64_t num_groups,
                    int32_t *plan_ws, int32_t *perm, int32_t *seg, int32_t *preSum, int64_t *out,
                    int32_t *stats, void *stream);

/* Points inside (enlarged) rotated boxes.  Replaces dynamic_point_pool_launcher
 * (torchex/src/dynamic_point_pool/dynamic_point_pool.cpp:20-32, kernels
 * dynamic_point_pool_kernel.cu:73-170,280-310): for every (box, point) pair with
 * the point inside the box enlarged by extra_wlh (HOST array of 3), one output
 * entry: point index, box index and 13 floats (x, y, z, local x/y/z, the six
 * face offsets, in-margin flag).  At most max_pts_per_box entries per box and
 * max_all_pts in total.  Entries are written compactly at [0, *num_out) in
 * (box, point) order -- deterministic, where the reference's atomic counters
 * give an arbitrary order and an arbitrary surviving subset under the caps.
 * rois [num_boxes, 7] (x, y, z of the bottom centre, w, l, h, rz), pts
 * [num_pts, 3]; outputs are caller-allocated with max_all_pts entries and
 * need no initialisation; num_out is a device int.  workspace: int32 array of
 * txs_dpp_workspace_len(num_pts, num_boxes) entries, 8-byte aligned. */
int txs_dynamic_point_pool(const float *rois, const float *pts, int64_t num_boxes, int64_t num_pts,
                           const float *extra_wlh, int32_t max_pts_per_box, int64_t max_all_pts,
                           int32_t *workspace, int64_t *out_pts_idx, int64_t *out_roi_idx,
                           float *out_pts_feats, int32_t *num_out, void *stream);
int64_t txs_dpp_workspace_len(int64_t num_pts, int64_t num_boxes);

/* The same for a batch of samples held in one pair of tensors.  Replaces
 * dynamic_point_pool_mixed_launcher (torchex/src/dynamic_point_pool/dynamic_point_pool.cpp:108-164,
 * kernel generate_pts_mask_for_box3d_mixed, dynamic_point_pool_kernel.cu:173-212): rois_batch
 * [num_boxes] and pts_batch [num_pts] give the sample of every box and point, and a point is
 * tested only against the boxes of its own sample.  Both NULL: txs_dynamic_point_pool. */
int txs_dynamic_point_pool_mixed(const float *rois, const int32_t *rois_batch, const float *pts,
                                 const int32_t *pts_batch, int64_t num_boxes, int64_t num_pts,
                                 const float *extra_wlh, int32_t max_pts_per_box, int64_t max_all_pts,
                                 int32_t *workspace, int64_t *out_pts_idx, int64_t *out_roi_idx,
                                 float *out_pts_feats, int32_t *num_out, void *stream);

/* Hash table of int32 (key, value) pairs.  Replace build_hash_table_launcher /
 * probe_hash_table_launcher (torchex/src/grid_hash/grid_hash.cpp:14-27, kernels
 * grid_hash_kernel.cu:19-49, probing of src/utils/functions.cuh:30-64).
 * table: int32 [table_size, 2], table_size a power of two >= num_keys, 8-byte
 * aligned; build fills it with -1 first.  Keys must be unique and >= 0.
 * fail_flag (may be NULL): device int set to 1 if a key could not be placed.
 * probe writes the value of each key, or -1 for a key that is not in the table
 * (the reference asserts instead). */
int txs_grid_hash_build(const int32_t *keys, const int32_t *values, int64_t num_keys, int32_t *table,
                        int64_t table_size, int32_t *fail_flag, void *stream);
int txs_grid_hash_probe(const int32_t *keys, int64_t num_keys, const int32_t *table,
                        int64_t table_size, int32_t *out_values, void *stream);

/* ---- the hot path --------------------------------------------------------- */

/* Forward reduction.  Replaces scatter_sum_launcher / scatter_max_launcher
 * (scatter.cpp:12-16, kernels scatter_kernel.cu:102-171) and fuses the divide
 * of ScatterMeanFunction.forward (scatter_op.py:69) for op == TXS_MEAN.
 *   op TXS_SUM / TXS_MEAN: arg is ignored (may be NULL); fp32 accumulation.
 *   op TXS_MAX: out = max, arg = smallest row index attaining it; NaN never
 *     wins; a voxel with no non-NaN entry (or no rows) gets the lowest finite
 *     value of the dtype and arg = -1 (the reference's (-FLT_MAX, -1) init,
 *     scatter_kernel.cu:139-140).
 *   op TXS_MAX_REFTIE: same values; among equal maxima the winner is the row
 *     the reference kernel itself would report for the voxel's rows taken in
 *     ascending order with block width clamp(up_2n(max_cnt), 32, 1024)
 *     (scatter_kernel.cu:41-83,146-152,187: last row of a thread's residue
 *     class, then smallest bit-reversed lane, then smallest bit-reversed warp);
 *     -inf never wins, as in the reference.  max_cnt is the largest voxel
 *     population (the reference launcher's argument); other ops ignore it.
 * out (and arg) need no initialisation: every element is written.
 * unq_inv (may be NULL): the row-order voxel ids; without them (and with a perm)
 *   table mode is not available.  num_heavy: TXS_STAT_NUM_HEAVY of the plan.
 * scratch / scratch_cells: see "Data layout"; scratch may be NULL (scratch_cells 0) when
 *   there is no heavy voxel.  With fewer than txs_scatter_scratch_cells() cells (but at
 *   least num_heavy * channel) the call still works, on the voxel-order kernels.
 * path: TXS_PATH_AUTO, or one of the other two to force a choice. */
int txs_scatter_forward(int op, int dtype, const void *feats, const int32_t *unq_inv,
                        const int32_t *perm, const int32_t *seg, const int32_t *preSum,
                        const int32_t *slot_of, const int32_t *heavy_ids, int64_t num_special,
                        int64_t num_heavy, void *scratch, int64_t scratch_cells, void *out,
                        int32_t *arg, int64_t num_total, int64_t channel, int64_t num_unq,
                        int64_t max_cnt, int path, void *stream);

/* Number of 8-byte scratch cells that lets txs_scatter_forward choose freely between its
 * kernels for these extents: num_heavy * channel, plus the partial tables of table mode
 * where it applies.  -1 for invalid extents. */
int64_t txs_scatter_scratch_cells(int64_t num_total, int64_t channel, int64_t num_unq,
                                  int64_t num_heavy);

/* txs_scatter_forward for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and results as txs_scatter_forward,
 * except that no scratch is passed in: the call uses a table that lives in the
 * library's own device image (one copy per GPU, 8 MiB, held until the process ends).
 * The call allocates and frees nothing and only launches kernels: it clears the
 * num_heavy * channel cells the heavy voxels use, then runs the same kernels as
 * txs_scatter_forward (table mode only where its partial tables fit in the rest).
 *   Limit: num_heavy * channel <= txs_resident_table_cells() (1,048,576 cells, e.g.
 *   8192 heavy voxels of 128 channels); beyond it the call returns TXS_ERR_TOO_LARGE
 *   and launches nothing.
 *   Every call on one GPU shares that GPU's table: two calls that overlap in time on
 *   one GPU (different streams, or different host threads) race.  Calls queued on one
 *   stream are ordered and safe.
 *   The device that owns `stream` must be current.  The table's address is looked up
 *   the first time the call runs on a GPU; txs_resident_table_init() does that lookup
 *   ahead of time for the current GPU (call it before a graph capture starts). */
int txs_scatter_forward_resident(int op, int dtype, const void *feats, const int32_t *unq_inv,
                                 const int32_t *perm, const int32_t *seg, const int32_t *preSum,
                                 const int32_t *slot_of, const int32_t *heavy_ids, int64_t num_special,
                                 int64_t num_heavy, void *out, int32_t *arg, int64_t num_total,
                                 int64_t channel, int64_t num_unq, int64_t max_cnt, int path,
                                 void *stream);
int txs_resident_table_init(void);
int64_t txs_resident_table_cells(void);

/* Backward as one gather pass over the sorted positions.  Replaces the ATen
 * ops of ScatterSumFunction.backward (scatter_op.py:47-50: g[unq_inv]),
 * ScatterMeanFunction.backward (:74-78: (g / unq_cnts)[unq_inv]) and the
 * intended ScatterMaxFunction.backward (:106-111: zeros.scatter_(0, arg, g),
 * i.e. g_in[i,c] = g[u,c] if arg[u,c] == i else 0).
 * g_in [N, C] needs no initialisation.  arg is read only for TXS_MAX.
 * unq_inv (may be NULL) and path: as for txs_scatter_forward. */
int txs_scatter_backward(int op, int dtype, const void *grad_out, const int32_t *arg,
                         const int32_t *unq_inv, const int32_t *perm, const int32_t *seg,
                         const int32_t *preSum, void *grad_in, int64_t num_total, int64_t channel,
                         int64_t num_unq, int path, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TORCHEX_SCATTER_H */
