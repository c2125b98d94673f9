// scatter_ext: PyTorch-ROCm host glue for the voxel scatter path.
//
// Takes the place of torchex/src/scatter/scatter.cpp.  The three functions of
// the reference module keep their names and positional signatures
// (scatter.cpp:66-70: sum, max, getPreSum; outputs caller-allocated and written
// in place); the plan/forward/backward functions are what the Python wrappers
// in torchex_amd/scatter_op.py use.  All device work goes through the C ABI of
// libtorchex_scatter.so (include/torchex_scatter.h): this file only validates
// tensors, allocates through the torch caching allocator, picks the current HIP
// stream and device, and turns status codes into exceptions.

#include <torch/extension.h>

// PyTorch-ROCm keeps the device type spelled "cuda"; these are its HIP guard
// and stream accessors for that spelling.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <algorithm>
#include <limits>
#include <optional>
#include <tuple>
#include <utility>
#include <vector>

#include "torchex_scatter.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

void check_dev(const Tensor &x, const char *name) {
    // same two conditions as CHECK_INPUT in scatter.cpp:4-10
    TORCH_CHECK(x.device().is_cuda(), name, " must be a GPU tensor");
    TORCH_CHECK(x.is_contiguous(), name, " must be contiguous");
}

void check_i32(const Tensor &x, const char *name) {
    check_dev(x, name);
    TORCH_CHECK(x.scalar_type() == at::kInt, name, " must be int32, got ", x.scalar_type());
}

int dtype_code(const Tensor &x, const char *name) {
    switch (x.scalar_type()) {
        case at::kFloat: return TXS_F32;
        case at::kHalf: return TXS_F16;
        case at::kBFloat16: return TXS_BF16;
        default: TORCH_CHECK(false, name, " must be float32, float16 or bfloat16, got ", x.scalar_type());
    }
    return -1;
}

void check_status(int st, const char *what) {
    TORCH_CHECK(st == TXS_OK, "torchex scatter: ", what, " failed: ", txs_status_string(st));
}

void *cur_stream(const Tensor &x) {
    return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.device().index()).stream();
}

const int32_t *i32p(const Tensor &x) { return x.numel() ? x.data_ptr<int32_t>() : nullptr; }
int32_t *i32w(Tensor &x) { return x.numel() ? x.data_ptr<int32_t>() : nullptr; }
const int32_t *opt_i32p(const OptTensor &x) { return (x.has_value() && x->defined()) ? i32p(*x) : nullptr; }

Tensor empty_i32(int64_t n, const Tensor &like) {
    return at::empty({n}, like.options().dtype(at::kInt));
}

std::vector<int64_t> read_stats(const Tensor &stats) {
    // the one host synchronisation of index preparation: an asynchronous copy into pinned
    // host memory (from the caching host allocator), then a wait on the stream
    Tensor h = at::empty({TXS_STATS_LEN}, stats.options().device(at::kCPU).pinned_memory(true));
    h.copy_(stats, /*non_blocking=*/true);
    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(stats.device().index()).synchronize();
    std::vector<int64_t> v(TXS_STATS_LEN);
    for (int i = 0; i < TXS_STATS_LEN; ++i) v[i] = h.data_ptr<int32_t>()[i];
    return v;
}

// The special-voxel list the forward call takes: txs_plan_special leaves the heavy
// voxels at the front of its `capacity`-entry array and the empty ones at its back.
Tensor special_list(const Tensor &heavy_all, int64_t capacity, const std::vector<int64_t> &hs) {
    const int64_t n_heavy = hs[TXS_STAT_NUM_HEAVY], n_empty = hs[TXS_STAT_NUM_EMPTY];
    Tensor heavy = heavy_all.narrow(0, 0, n_heavy);
    if (n_empty == 0) return heavy.contiguous();
    return at::cat({heavy, heavy_all.narrow(0, capacity - n_empty, n_empty)});
}

// A handful of voxels just above the default heavy threshold are not worth the heavy path:
// the forward kernel reduces a run a little longer than the 64 positions a tile stages behind
// its end like any other (the last few rows one by one), and a plan without heavy voxels saves
// every forward call its second kernel.  A threshold chosen by the caller is left alone.
constexpr int64_t kDemoteMostVoxels = 64;  // heavy voxels at most ...
constexpr int64_t kDemoteLongest = 96;     // ... none of them longer than this
void demote_few_heavy(std::vector<int64_t> &hs, int64_t heavy_threshold, const Tensor &preSum, Tensor &seg,
                      Tensor &slot_of, const Tensor &heavy_all, Tensor &stats, int64_t N, int64_t U, void *st) {
    const int64_t n_heavy = hs[TXS_STAT_NUM_HEAVY];
    if (heavy_threshold != txs_default_heavy_threshold() || n_heavy == 0 || n_heavy > kDemoteMostVoxels ||
        hs[TXS_STAT_MAX_CNT] > kDemoteLongest || hs[TXS_STAT_OUT_OF_RANGE])
        return;
    check_status(txs_plan_demote_heavy(i32p(preSum), i32w(seg), i32w(slot_of), i32p(heavy_all), n_heavy, N, U,
                                       i32w(stats), st),
                 "plan_demote_heavy");
    hs[TXS_STAT_NUM_HEAVY] = 0;
    hs[TXS_STAT_NUM_SPECIAL] = hs[TXS_STAT_NUM_EMPTY];
}

// ScatterData index preparation for an unq_inv in any order
// (extends torchex/operator_py/scatter_op.py:13-21).  Everything is queued on
// the current stream; the only host synchronisation is the read of `stats`.
// returns (preSum, perm | None, seg, slot_of, heavy_ids, stats)
// assume_sorted: the caller states that unq_inv is non-decreasing (the only order the
// reference accepts); the sort is then not even queued, and the statement is checked
// on the device (an unsorted unq_inv raises).
std::tuple<Tensor, OptTensor, Tensor, Tensor, Tensor, std::vector<int64_t>> build_plan(
    const Tensor &unq_inv, int64_t num_unq, int64_t heavy_threshold, const OptTensor &unq_cnts,
    bool assume_sorted) {
    check_i32(unq_inv, "unq_inv");
    TORCH_CHECK(unq_inv.dim() == 1, "unq_inv must be 1-D");
    TORCH_CHECK(num_unq >= 0, "num_unq must be non-negative");
    const int64_t *cnts = nullptr;
    if (unq_cnts.has_value()) {
        check_dev(*unq_cnts, "unq_cnts");
        TORCH_CHECK(unq_cnts->scalar_type() == at::kLong && unq_cnts->numel() == num_unq,
                    "unq_cnts must be int64 with num_unq entries");
        cnts = num_unq ? unq_cnts->data_ptr<int64_t>() : nullptr;
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(unq_inv.device());
    const int64_t N = unq_inv.numel(), U = num_unq;
    void *st = cur_stream(unq_inv);
    Tensor stats = at::zeros({TXS_STATS_LEN}, unq_inv.options());
    Tensor seg, perm;
    Tensor preSum = empty_i32(U + 1, unq_inv);
    Tensor slot_of = empty_i32(U, unq_inv);
    Tensor heavy_all = empty_i32(U, unq_inv);
    std::vector<int64_t> hs;
    if (assume_sorted) {
        check_status(txs_plan_check(i32p(unq_inv), N, U, i32w(stats), st), "plan_check");
        seg = unq_inv.clone();  // sorted ids are their own sorted keys
        check_status(txs_plan_presum(i32p(seg), U > 0 ? N : 0, U, i32w(preSum), st), "plan_presum");
        check_status(txs_plan_special(i32p(preSum), U, (int32_t)heavy_threshold, cnts, i32w(slot_of),
                                      i32w(heavy_all), i32w(stats), nullptr, nullptr, st),
                     "plan_special");
        check_status(txs_plan_seg_flag(i32w(seg), U > 0 ? N : 0, U, i32p(slot_of), st), "plan_seg_flag");
        hs = read_stats(stats);
    } else {
        seg = empty_i32(N, unq_inv);
        perm = empty_i32(N, unq_inv);
        Tensor ws = empty_i32(txs_plan_workspace_len(N, U), unq_inv);
        check_status(txs_plan_build(i32p(unq_inv), N, U, (int32_t)heavy_threshold, cnts, i32w(ws), i32w(perm),
                                    i32w(seg), i32w(preSum), i32w(slot_of), i32w(heavy_all), i32w(stats), st),
                     "plan_build");
        hs = read_stats(stats);
        if (hs[TXS_STAT_NEED_GENERAL]) {
            // a few voxels own most of the rows: the bucket kernels stepped aside
            stats.zero_();
            check_status(txs_plan_build_general(i32p(unq_inv), N, U, (int32_t)heavy_threshold, cnts, i32w(ws),
                                                i32w(perm), i32w(seg), i32w(preSum), i32w(slot_of),
                                                i32w(heavy_all), i32w(stats), st),
                         "plan_build_general");
            hs = read_stats(stats);
        }
    }
    TORCH_CHECK(hs[TXS_STAT_OUT_OF_RANGE] == 0 && (U > 0 || N == 0),
                "unq_inv holds ids outside [0, num_unq=", U, ")");
    TORCH_CHECK(!(assume_sorted && hs[TXS_STAT_UNSORTED]),
                "unq_inv was declared sorted (assume_sorted=True) but is not non-decreasing");
    demote_few_heavy(hs, heavy_threshold, preSum, seg, slot_of, heavy_all, stats, N, U, st);
    OptTensor perm_out;
    if (hs[TXS_STAT_UNSORTED]) perm_out = perm;
    Tensor heavy_ids = special_list(heavy_all, U, hs);
    return {preSum, perm_out, seg, slot_of, heavy_ids, hs};
}

// Plan for callers that hold only CSR offsets of already grouped rows.
// returns (seg, slot_of, heavy_ids, stats)
std::tuple<Tensor, Tensor, Tensor, std::vector<int64_t>> plan_from_presum(
    const Tensor &preSum, int64_t num_total, int64_t heavy_threshold) {
    check_i32(preSum, "preSum");
    TORCH_CHECK(preSum.dim() == 1 && preSum.numel() >= 1, "preSum must be 1-D with num_unq+1 entries");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(preSum.device());
    const int64_t U = preSum.numel() - 1, N = num_total;
    void *st = cur_stream(preSum);
    Tensor stats = at::zeros({TXS_STATS_LEN}, preSum.options());
    Tensor slot_of = empty_i32(U, preSum);
    Tensor heavy_all = empty_i32(U, preSum);
    check_status(txs_plan_special(i32p(preSum), U, (int32_t)heavy_threshold, nullptr, i32w(slot_of),
                                  i32w(heavy_all), i32w(stats), nullptr, nullptr, st),
                 "plan_special");
    Tensor seg = empty_i32(N, preSum);
    if (U > 0)
        check_status(txs_plan_seg_from_presum(i32p(preSum), N, U, i32p(slot_of), i32w(seg), st),
                     "plan_seg_from_presum");
    std::vector<int64_t> hs = read_stats(stats);
    if (U > 0) demote_few_heavy(hs, heavy_threshold, preSum, seg, slot_of, heavy_all, stats, N, U, st);
    Tensor heavy_ids = special_list(heavy_all, U, hs);
    return {seg, slot_of, heavy_ids, hs};
}

// Dynamic voxelization front-end: coors and linear keys of every point; no host
// synchronisation (range violations are flagged in the returned stats tensor).
// returns (coors [N,3] int32, keys [N] int32, stats [TXS_STATS_LEN] int32)
std::tuple<Tensor, Tensor, Tensor> voxel_keys(const Tensor &points, std::vector<double> range_lo,
                                              std::vector<double> voxel_size,
                                              std::vector<int64_t> dims) {
    check_dev(points, "points");
    TORCH_CHECK(points.dim() == 2 && points.size(1) >= 3, "points must be [N, >=3]");
    TORCH_CHECK(points.scalar_type() == at::kFloat, "points must be float32");
    TORCH_CHECK(range_lo.size() == 3 && voxel_size.size() == 3 && dims.size() == 3,
                "range_lo, voxel_size and dims need 3 entries");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(points.device());
    const int64_t N = points.size(0);
    const float lo[3] = {(float)range_lo[0], (float)range_lo[1], (float)range_lo[2]};
    const float vs[3] = {(float)voxel_size[0], (float)voxel_size[1], (float)voxel_size[2]};
    const int32_t dm[3] = {(int32_t)dims[0], (int32_t)dims[1], (int32_t)dims[2]};
    Tensor coors = at::empty({N, 3}, points.options().dtype(at::kInt));
    Tensor keys = at::empty({N}, points.options().dtype(at::kInt));
    Tensor stats = at::zeros({TXS_STATS_LEN}, points.options().dtype(at::kInt));
    check_status(txs_voxel_keys(N ? points.data_ptr<float>() : nullptr, N, points.size(1), lo, vs, dm,
                                i32w(coors), i32w(keys), i32w(stats), cur_stream(points)),
                 "voxel_keys");
    return {coors, keys, stats};
}

// torch.unique(keys, return_inverse=True, return_counts=True) fused with the
// scatter plan: one sort, one host synchronisation.
// returns (unq_keys, unq_inv, unq_cnts, preSum, perm | None, seg, slot_of, heavy_ids, stats)
std::tuple<Tensor, Tensor, Tensor, Tensor, OptTensor, Tensor, Tensor, Tensor, std::vector<int64_t>>
unique_plan(const Tensor &keys_in, int64_t key_bound, int64_t heavy_threshold, const OptTensor &stats_in) {
    check_dev(keys_in, "keys");
    TORCH_CHECK(keys_in.scalar_type() == at::kInt || keys_in.scalar_type() == at::kLong,
                "keys must be int32 or int64, got ", keys_in.scalar_type());
    TORCH_CHECK(keys_in.dim() == 1, "keys must be 1-D");
    TORCH_CHECK(key_bound > 0, "key_bound must be positive");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(keys_in.device());
    const int64_t N = keys_in.numel();
    void *st = cur_stream(keys_in);
    const auto i32 = keys_in.options().dtype(at::kInt);
    Tensor stats = stats_in.has_value() ? *stats_in : at::zeros({TXS_STATS_LEN}, i32);
    check_i32(stats, "stats");
    TORCH_CHECK(stats.numel() == TXS_STATS_LEN, "stats must have TXS_STATS_LEN entries");
    // Keys from a grid that is not much larger than the input: dense ids from an occupancy
    // map (no sort of the keys), then the index preparation of those ids.  `stats` is read
    // twice: the number of distinct keys, which sizes the plan (fetched while the ids are
    // still being written), and the plan's own figures.
    if (N > 0 && key_bound <= (int64_t(1) << 28) && key_bound <= 64 * N) {
        const int is64 = keys_in.scalar_type() == at::kLong;
        Tensor inv = at::empty({N}, i32), unq = at::empty({std::min(N, key_bound)}, i32);
        Tensor bws = at::empty({txs_unique_bitmap_workspace_len(key_bound)}, i32);
        check_status(txs_unique_bitmap_count(keys_in.data_ptr(), is64, N, key_bound, i32w(bws), i32w(stats), st),
                     "unique_bitmap_count");
        Tensor h = at::empty({TXS_STATS_LEN}, stats.options().device(at::kCPU).pinned_memory(true));
        h.copy_(stats, /*non_blocking=*/true);
        at::cuda::CUDAEvent counted;
        counted.record(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(keys_in.device().index()));
        check_status(txs_unique_bitmap_assign(keys_in.data_ptr(), is64, N, key_bound, i32p(bws), i32w(inv), i32w(unq), st),
                     "unique_bitmap_assign");
        counted.synchronize();
        TORCH_CHECK(h.data_ptr<int32_t>()[TXS_STAT_OUT_OF_RANGE] == 0,
                    "keys (or points) outside the grid: keys must be in [0, ", key_bound, ")");
        const int64_t U = h.data_ptr<int32_t>()[TXS_STAT_NUM_UNQ];
        auto [preSum, perm_out, seg, slot_of, heavy_ids, hs] = build_plan(inv, U, heavy_threshold, std::nullopt, false);
        Tensor cnts = at::empty({U}, keys_in.options().dtype(at::kLong));
        check_status(txs_counts_from_presum(i32p(preSum), U, U ? cnts.data_ptr<int64_t>() : nullptr, st),
                     "counts_from_presum");
        hs[TXS_STAT_NUM_UNQ] = U;
        return {unq.narrow(0, 0, U), inv, cnts, preSum, perm_out, seg, slot_of, heavy_ids, hs};
    }
    // int64 keys are narrowed for the sort; one outside int32 is first pinned to a value that
    // stays outside [0, key_bound) (key_bound is below 2^31 - 1), so that the range check on
    // the device flags it instead of seeing its low 32 bits
    const Tensor keys = keys_in.scalar_type() == at::kInt
                            ? keys_in
                            : keys_in.clamp(-1, (int64_t)std::numeric_limits<int32_t>::max()).to(at::kInt);
    Tensor seg = empty_i32(N, keys), perm = empty_i32(N, keys), inv = empty_i32(N, keys);
    Tensor unq = empty_i32(N, keys), preSum = empty_i32(N + 1, keys);
    Tensor slot_of = empty_i32(N, keys), heavy_all = empty_i32(N, keys);
    Tensor cnts = at::empty({N}, keys.options().dtype(at::kLong));
    Tensor ws = empty_i32(txs_sort_workspace_len(N, key_bound), keys);
    Tensor uws = empty_i32(txs_unique_workspace_len(N), keys);
    check_status(txs_plan_check(i32p(keys), N, key_bound, i32w(stats), st), "plan_check");
    Tensor sorted_keys = empty_i32(N, keys);  // unique_runs reads neighbours: not the same array as seg
    check_status(txs_plan_sort(i32p(keys), N, key_bound, i32p(stats), i32w(perm), i32w(sorted_keys),
                               i32w(ws), st),
                 "plan_sort");
    check_status(txs_unique_runs(i32p(sorted_keys), i32p(perm), N, i32w(uws), i32w(seg), i32w(inv),
                                 i32w(unq), i32w(preSum), i32w(stats), st),
                 "unique_runs");
    const int32_t *u_dev = stats.data_ptr<int32_t>() + TXS_STAT_NUM_UNQ;
    check_status(txs_plan_special(i32p(preSum), N, (int32_t)heavy_threshold, nullptr, i32w(slot_of),
                                  i32w(heavy_all), i32w(stats), u_dev,
                                  N ? cnts.data_ptr<int64_t>() : nullptr, st),
                 "plan_special");
    check_status(txs_plan_seg_flag(i32w(seg), N, N, i32p(slot_of), st), "plan_seg_flag");
    std::vector<int64_t> hs = read_stats(stats);
    TORCH_CHECK(hs[TXS_STAT_OUT_OF_RANGE] == 0, "keys (or points) outside the grid: keys must be in [0, ",
                key_bound, ")");
    const int64_t U = hs[TXS_STAT_NUM_UNQ];
    demote_few_heavy(hs, heavy_threshold, preSum, seg, slot_of, heavy_all, stats, N, U, st);
    OptTensor perm_out;
    if (hs[TXS_STAT_UNSORTED]) perm_out = perm;
    return {unq.narrow(0, 0, U), inv, cnts.narrow(0, 0, U), preSum.narrow(0, 0, U + 1), perm_out, seg,
            slot_of.narrow(0, 0, U), special_list(heavy_all, N, hs), hs};
}

// ingroup_inds(seg, perm | None, preSum, num_unq) -> int64 [N]
Tensor ingroup_inds(const Tensor &seg, const OptTensor &perm, const Tensor &preSum, int64_t num_unq) {
    check_i32(seg, "seg");
    check_i32(preSum, "preSum");
    if (perm.has_value()) check_i32(*perm, "perm");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(seg.device());
    const int64_t N = seg.numel();
    Tensor out = at::empty({N}, seg.options().dtype(at::kLong));
    check_status(txs_ingroup_inds(i32p(seg), opt_i32p(perm), i32p(preSum), N, num_unq,
                                  N ? out.data_ptr<int64_t>() : nullptr, cur_stream(seg)),
                 "ingroup_inds");
    return out;
}

// group_ranks(ids) -> int64 ranks, one call for the whole of ingroup_inds: index preparation
// with the number of rows as the bound of the ids (true for the inverse of a unique; the
// largest id is then never read back), the rank kernel, one host synchronisation.  Ids at
// or above the number of rows take a second pass with their true bound.
// `out`: int64, contiguous, one entry per id; written in place.
void group_ranks_into(const Tensor &ids_in, Tensor &out) {
    check_dev(ids_in, "group_inds");
    TORCH_CHECK(ids_in.scalar_type() == at::kInt || ids_in.scalar_type() == at::kLong,
                "group_inds must be int32 or int64");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(ids_in.device());
    Tensor ids = ids_in.reshape({-1}).contiguous();
    if (ids.scalar_type() != at::kInt) ids = ids.to(at::kInt);
    const int64_t N = ids.numel();
    if (N == 0) return;
    void *st = cur_stream(ids);
    // `exact`: U is the true bound of the ids (largest id + 1), not the guess `number of rows`
    auto attempt = [&](int64_t U, bool exact) -> bool {
        Tensor stats = at::zeros({TXS_STATS_LEN}, ids.options());
        Tensor seg = empty_i32(N, ids), perm = empty_i32(N, ids);
        Tensor preSum = empty_i32(U + 1, ids);
        Tensor ws = empty_i32(txs_plan_workspace_len(N, U), ids);
        const int32_t heavy = txs_default_heavy_threshold();
        // order and offsets only (no special-voxel table) and the ranks, queued together
        check_status(txs_group_ranks(i32p(ids), N, U, i32w(ws), i32w(perm), i32w(seg), i32w(preSum),
                                     out.data_ptr<int64_t>(), i32w(stats), st),
                     "group_ranks");
        std::vector<int64_t> hs = read_stats(stats);
        if (hs[TXS_STAT_OUT_OF_RANGE]) return false;
        if (hs[TXS_STAT_NEED_GENERAL]) {
            // one bucket holds most of the rows.  Under the guessed bound that usually means few
            // groups with small ids: the true bound gives narrower buckets, often none to sort by
            if (!exact) return false;
            stats.zero_();
            check_status(txs_plan_build_general(i32p(ids), N, U, heavy, nullptr, i32w(ws), i32w(perm), i32w(seg),
                                                i32w(preSum), nullptr, nullptr, i32w(stats), st),
                         "plan_build_general");
            hs = read_stats(stats);
            // ids already in order leave perm unwritten: position == row
            check_status(txs_ingroup_inds(i32p(seg), hs[TXS_STAT_UNSORTED] ? i32p(perm) : nullptr, i32p(preSum), N, U,
                                          out.data_ptr<int64_t>(), st),
                         "ingroup_inds");
        }
        return true;
    };
    if (!attempt(N, false)) {
        const int64_t lo = ids.min().item<int64_t>(), hi = ids.max().item<int64_t>();
        TORCH_CHECK(lo >= 0, "group_inds must be non-negative");
        TORCH_CHECK(attempt(hi + 1, true), "group_inds could not be ranked");
    }
}

Tensor group_ranks(const Tensor &ids_in) {
    check_dev(ids_in, "group_inds");
    Tensor out = at::empty({ids_in.numel()}, ids_in.options().dtype(at::kLong));
    group_ranks_into(ids_in, out);
    return out;
}

// ---- the reference's ingroup_indices module (ingroup_inds.cpp:28-54) --------

// forward(group_inds, out_inds): both int64 and caller-allocated (the wrapper passes
// zeros_like(group_inds) - 1, ingroup_inds_op.py:15-17); every entry of out_inds is written.
void ingroup_inds_ref(Tensor group_inds, Tensor out_inds) {
    check_dev(group_inds, "group_inds");
    check_dev(out_inds, "out_inds");
    TORCH_CHECK(group_inds.scalar_type() == at::kLong, "group_inds must be int64, got ", group_inds.scalar_type());
    TORCH_CHECK(out_inds.scalar_type() == at::kLong, "out_inds must be int64, got ", out_inds.scalar_type());
    TORCH_CHECK(out_inds.numel() == group_inds.numel(), "out_inds must have one entry per element of group_inds");
    TORCH_CHECK(out_inds.device() == group_inds.device(), "group_inds and out_inds live on different devices");
    group_ranks_into(group_inds, out_inds);
}

// dynamic_point_pool(rois [B,7], pts [P,3], extra_wlh, max_pts_per_box, max_all_pts)
// -> (out_pts_idx int64 [M], out_roi_idx int64 [M], out_pts_feats float [M,13]); one host sync to read M.
// rois_batch [B] / pts_batch [P] (int32, both or neither): the sample of every box and point.
std::tuple<Tensor, Tensor, Tensor> dynamic_point_pool(const Tensor &rois, const Tensor &pts,
                                                      std::vector<double> extra_wlh,
                                                      int64_t max_pts_per_box, int64_t max_all_pts,
                                                      const OptTensor &rois_batch, const OptTensor &pts_batch) {
    check_dev(rois, "rois");
    check_dev(pts, "pts");
    TORCH_CHECK(rois_batch.has_value() == pts_batch.has_value(), "rois_batch and pts_batch go together");
    if (rois_batch.has_value()) {
        check_i32(*rois_batch, "rois_batch");
        check_i32(*pts_batch, "pts_batch");
        TORCH_CHECK(rois_batch->dim() == 1 && rois_batch->numel() == rois.size(0), "rois_batch must be [num_boxes]");
        TORCH_CHECK(pts_batch->dim() == 1 && pts_batch->numel() == pts.size(0), "pts_batch must be [num_pts]");
    }
    TORCH_CHECK(rois.dim() == 2 && rois.size(1) == 7 && rois.scalar_type() == at::kFloat,
                "rois must be float32 [num_boxes, 7]");
    TORCH_CHECK(pts.dim() == 2 && pts.size(1) == 3 && pts.scalar_type() == at::kFloat,
                "pts must be float32 [num_pts, 3]");
    TORCH_CHECK(extra_wlh.size() == 3, "extra_wlh needs 3 entries");
    TORCH_CHECK(max_all_pts >= 0 && max_pts_per_box >= 0, "caps must be non-negative");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(pts.device());
    const int64_t B = rois.size(0), P = pts.size(0);
    const float extra[3] = {(float)extra_wlh[0], (float)extra_wlh[1], (float)extra_wlh[2]};
    auto iopt = pts.options().dtype(at::kInt);
    Tensor ws = at::empty({txs_dpp_workspace_len(P, B) + 2}, iopt);
    Tensor idx = at::empty({max_all_pts}, pts.options().dtype(at::kLong));
    Tensor roi = at::empty({max_all_pts}, pts.options().dtype(at::kLong));
    Tensor feats = at::empty({max_all_pts, 13}, pts.options());
    Tensor num = at::zeros({1}, iopt);
    check_status(txs_dynamic_point_pool_mixed(B ? rois.data_ptr<float>() : nullptr, opt_i32p(rois_batch),
                                        P ? pts.data_ptr<float>() : nullptr, opt_i32p(pts_batch),
                                        B, P, extra, (int32_t)max_pts_per_box, max_all_pts, i32w(ws),
                                        max_all_pts ? idx.data_ptr<int64_t>() : nullptr,
                                        max_all_pts ? roi.data_ptr<int64_t>() : nullptr,
                                        max_all_pts ? feats.data_ptr<float>() : nullptr, i32w(num),
                                        cur_stream(pts)),
                 "dynamic_point_pool");
    const int64_t M = num.cpu().data_ptr<int32_t>()[0];
    return {idx.narrow(0, 0, M), roi.narrow(0, 0, M), feats.narrow(0, 0, M)};
}

// ---- the reference's dynamic_point_pool_ext module (dynamic_point_pool.cpp:58-169) ----

// The outputs come from the caller (the wrapper fills them with -1 / -1 / 0,
// dynamic_point_pool_op.py:33-35), max_all_pts is their length, and the entries are
// written from index 0 on; what lies behind the last entry keeps the caller's fill.  No
// host synchronisation (the reference reads its counter back between its two kernels).
void dpp_into(const Tensor &rois, const OptTensor &rois_batch, const Tensor &pts, const OptTensor &pts_batch,
              const std::vector<double> &extra_wlh, int64_t max_pts_per_box, Tensor &out_pts_idx,
              Tensor &out_roi_idx, Tensor &out_pts_feats) {
    check_dev(rois, "rois");
    check_dev(pts, "pts");
    check_dev(out_pts_idx, "out_pts_idx");
    check_dev(out_roi_idx, "out_roi_idx");
    check_dev(out_pts_feats, "out_pts_feats");
    TORCH_CHECK(rois.dim() == 2 && rois.size(1) == 7 && rois.scalar_type() == at::kFloat,
                "rois must be float32 [num_boxes, 7]");
    TORCH_CHECK(pts.dim() == 2 && pts.size(1) == 3 && pts.scalar_type() == at::kFloat,
                "pts must be float32 [num_pts, 3]");
    TORCH_CHECK(extra_wlh.size() == 3, "extra_wlh needs 3 entries");
    TORCH_CHECK(max_pts_per_box >= 0, "max_num_pts_per_box must be non-negative");
    const int64_t B = rois.size(0), P = pts.size(0), M = out_pts_idx.size(0);
    TORCH_CHECK(out_pts_idx.scalar_type() == at::kLong && out_pts_idx.dim() == 1, "out_pts_idx must be int64 [max_all_pts]");
    TORCH_CHECK(out_roi_idx.scalar_type() == at::kLong && out_roi_idx.dim() == 1 && out_roi_idx.size(0) == M,
                "out_roi_idx must be int64 [max_all_pts]");
    TORCH_CHECK(out_pts_feats.scalar_type() == at::kFloat && out_pts_feats.dim() == 2 && out_pts_feats.size(0) == M &&
                    out_pts_feats.size(1) == 13,
                "out_pts_feats must be float32 [max_all_pts, 13]");  // info_dim == 13, dynamic_point_pool.cpp:80-81
    if (rois_batch.has_value()) {
        check_i32(*rois_batch, "rois_batch");
        check_i32(*pts_batch, "pts_batch");
        TORCH_CHECK(rois_batch->numel() == B, "rois_batch must be [num_boxes]");
        TORCH_CHECK(pts_batch->numel() == P, "pts_batch must be [num_pts]");
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(pts.device());
    const float extra[3] = {(float)extra_wlh[0], (float)extra_wlh[1], (float)extra_wlh[2]};
    auto iopt = pts.options().dtype(at::kInt);
    Tensor ws = at::empty({txs_dpp_workspace_len(P, B) + 2}, iopt);
    Tensor num = at::zeros({1}, iopt);
    check_status(txs_dynamic_point_pool_mixed(B ? rois.data_ptr<float>() : nullptr, opt_i32p(rois_batch),
                                              P ? pts.data_ptr<float>() : nullptr, opt_i32p(pts_batch), B, P, extra,
                                              (int32_t)max_pts_per_box, M, i32w(ws),
                                              M ? out_pts_idx.data_ptr<int64_t>() : nullptr,
                                              M ? out_roi_idx.data_ptr<int64_t>() : nullptr,
                                              M ? out_pts_feats.data_ptr<float>() : nullptr, i32w(num), cur_stream(pts)),
                 "dynamic_point_pool");
}

// forward(rois, pts, extra_wlh, max_num_pts_per_box, out_pts_idx, out_roi_idx, out_pts_feats)
void dpp_forward_ref(Tensor rois, Tensor pts, std::vector<double> extra_wlh, int64_t max_num_pts_per_box,
                     Tensor out_pts_idx, Tensor out_roi_idx, Tensor out_pts_feats) {
    dpp_into(rois, std::nullopt, pts, std::nullopt, extra_wlh, max_num_pts_per_box, out_pts_idx, out_roi_idx,
             out_pts_feats);
}

// dynamic_point_pool_mixed_gpu(rois, rois_batch, pts, pts_batch, extra_wlh, max_num_pts_per_box, out...)
void dpp_mixed_ref(Tensor rois, Tensor rois_batch, Tensor pts, Tensor pts_batch, std::vector<double> extra_wlh,
                   int64_t max_num_pts_per_box, Tensor out_pts_idx, Tensor out_roi_idx, Tensor out_pts_feats) {
    dpp_into(rois, rois_batch, pts, pts_batch, extra_wlh, max_num_pts_per_box, out_pts_idx, out_roi_idx,
             out_pts_feats);
}

int64_t up_2n_host(int64_t n) {  // torchex/src/grid_hash/grid_hash.cpp:28-37
    int64_t p = 1;
    while (p < n) p <<= 1;
    return p;
}

// build_table(coors int32 [N], values int32 [N]) -> table int32 [up_2n(N), 2]
// (torchex/src/grid_hash/grid_hash.cpp:49-78)
Tensor grid_hash_build(const Tensor &coors, const Tensor &values) {
    check_i32(coors, "coors");
    check_i32(values, "values");
    TORCH_CHECK(coors.dim() == 1 && values.dim() == 1 && coors.numel() == values.numel(),
                "coors and values must be 1-D of equal length");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(coors.device());
    const int64_t N = coors.numel(), size = up_2n_host(N > 0 ? N : 1);
    Tensor table = at::empty({size, 2}, coors.options());
    check_status(txs_grid_hash_build(i32p(coors), i32p(values), N, table.data_ptr<int32_t>(), size, nullptr,
                                     cur_stream(coors)),
                 "grid_hash_build");
    return table;
}

// probe_table(coors int32 [N], table) -> values int32 [N] (-1 where the key is absent)
// (torchex/src/grid_hash/grid_hash.cpp:85-112)
Tensor grid_hash_probe(const Tensor &coors, const Tensor &table) {
    check_i32(coors, "coors");
    check_i32(table, "table");
    TORCH_CHECK(coors.dim() == 1, "coors must be 1-D");
    TORCH_CHECK(table.dim() == 2 && table.size(1) == 2, "table must be [size, 2]");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(coors.device());
    Tensor out = at::empty_like(coors);
    check_status(txs_grid_hash_probe(i32p(coors), coors.numel(), table.data_ptr<int32_t>(), table.size(0),
                                     i32w(out), cur_stream(coors)),
                 "grid_hash_probe");
    return out;
}

// Zeroed scratch for forward calls on a [num_total, channel] feature matrix: the heavy
// voxels' rows first (which the kernels leave zeroed), behind them room for the partial
// tables of table mode where it applies.
Tensor make_scratch(int64_t num_total, int64_t channel, int64_t num_unq, int64_t num_heavy, const Tensor &like) {
    const int64_t cells = txs_scatter_scratch_cells(num_total, channel, num_unq, num_heavy);
    TORCH_CHECK(cells >= 0, "make_scratch: invalid extents");
    return at::zeros({cells}, like.options().dtype(at::kLong));
}

int check_path(int64_t path) {
    TORCH_CHECK(path == TXS_PATH_AUTO || path == TXS_PATH_VOXEL_ORDER || path == TXS_PATH_TABLE,
                "path must be 0 (auto), 1 (voxel-order kernels) or 2 (table kernels)");
    return (int)path;
}

void run_forward(int op, const Tensor &feats, const OptTensor &unq_inv, const OptTensor &perm, const Tensor &seg,
                 const Tensor &preSum, const Tensor &slot_of, const Tensor &heavy_ids, int64_t num_heavy,
                 Tensor &scratch, Tensor &out, OptTensor &arg, int64_t max_cnt, int path, bool holds_gil = true) {
    const int64_t N = feats.size(0), C = feats.size(1), U = preSum.numel() - 1;
    const int64_t S = heavy_ids.numel();
    TORCH_CHECK(scratch.dim() == 1, "scratch must be 1-D (ScatterData.scratch(channel))");
    TORCH_CHECK(num_heavy >= 0 && num_heavy <= S, "num_heavy exceeds the number of special voxels");
    TORCH_CHECK(scratch.numel() >= num_heavy * C, "scratch holds ", scratch.numel(), " cells, the heavy voxels need ",
                num_heavy * C);
    TORCH_CHECK(seg.numel() == N, "plan was built for ", seg.numel(), " rows, feats has ", N);
    TORCH_CHECK(!perm.has_value() || perm->numel() == N, "perm length mismatch");
    TORCH_CHECK(!unq_inv.has_value() || unq_inv->numel() == N, "unq_inv length mismatch");
    TORCH_CHECK(slot_of.numel() == U, "slot_of length mismatch");
    TORCH_CHECK(out.size(0) == U && out.size(1) == C, "out must be [num_unq, channel]");
    const int dt = dtype_code(feats, "feats");
    void *st = cur_stream(feats);
    auto launch = [&]() {
        return txs_scatter_forward(op, dt, feats.data_ptr(), opt_i32p(unq_inv), opt_i32p(perm), i32p(seg),
                                   i32p(preSum), i32p(slot_of), i32p(heavy_ids), S, num_heavy,
                                   scratch.numel() ? scratch.data_ptr() : nullptr, scratch.numel(), out.data_ptr(),
                                   arg.has_value() ? arg->data_ptr<int32_t>() : nullptr, N, C, U, max_cnt, path,
                                   st);
    };
    int rc;
    if (holds_gil) {
        pybind11::gil_scoped_release nogil;
        rc = launch();
    } else {
        rc = launch();
    }
    check_status(rc, "scatter_forward");
}

// forward(op, feats, unq_inv|None, perm|None, seg, preSum, slot_of, heavy_ids, num_heavy, scratch, max_cnt,
//         path=0) -> (out, arg|None)
std::tuple<Tensor, OptTensor> forward_impl(int64_t op, const Tensor &feats, const OptTensor &unq_inv,
                                           const OptTensor &perm, const Tensor &seg, const Tensor &preSum,
                                           const Tensor &slot_of, const Tensor &heavy_ids, int64_t num_heavy,
                                           Tensor scratch, int64_t max_cnt, int64_t path, bool holds_gil) {
    check_dev(feats, "feats");
    TORCH_CHECK(feats.dim() == 2, "feats must be [num_total, channel]");
    check_i32(seg, "seg");
    check_i32(preSum, "preSum");
    check_i32(slot_of, "slot_of");
    check_i32(heavy_ids, "heavy_ids");
    if (perm.has_value()) check_i32(*perm, "perm");
    if (unq_inv.has_value()) check_i32(*unq_inv, "unq_inv");
    check_dev(scratch, "scratch");
    TORCH_CHECK(scratch.scalar_type() == at::kLong, "scratch must be int64");
    TORCH_CHECK(seg.device() == feats.device(), "plan and feats live on different devices");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(feats.device());
    const int64_t C = feats.size(1), U = preSum.numel() - 1;
    Tensor out = at::empty({U, C}, feats.options());
    OptTensor arg;
    if (op == TXS_MAX || op == TXS_MAX_REFTIE) arg = at::empty({U, C}, feats.options().dtype(at::kInt));
    run_forward((int)op, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, scratch, out, arg, max_cnt,
                check_path(path), holds_gil);
    return {out, arg};
}

std::tuple<Tensor, OptTensor> forward(int64_t op, const Tensor &feats, const OptTensor &unq_inv,
                                      const OptTensor &perm, const Tensor &seg, const Tensor &preSum,
                                      const Tensor &slot_of, const Tensor &heavy_ids, int64_t num_heavy,
                                      Tensor scratch, int64_t max_cnt, int64_t path) {
    return forward_impl(op, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, std::move(scratch),
                        max_cnt, path, /*holds_gil=*/true);
}

// backward(op, grad_out, arg|None, unq_inv|None, perm|None, seg, preSum, num_total, path=0) -> grad_in
Tensor backward_impl(int64_t op, const Tensor &grad_out, const OptTensor &arg, const OptTensor &unq_inv,
                     const OptTensor &perm, const Tensor &seg, const Tensor &preSum, int64_t num_total, int64_t path,
                     bool holds_gil) {
    check_dev(grad_out, "grad_out");
    TORCH_CHECK(grad_out.dim() == 2, "grad_out must be [num_unq, channel]");
    check_i32(seg, "seg");
    check_i32(preSum, "preSum");
    if (perm.has_value()) check_i32(*perm, "perm");
    if (unq_inv.has_value()) check_i32(*unq_inv, "unq_inv");
    const int64_t U = preSum.numel() - 1, C = grad_out.size(1), N = num_total;
    TORCH_CHECK(grad_out.size(0) == U, "grad_out has ", grad_out.size(0), " rows, plan has ", U, " voxels");
    TORCH_CHECK(seg.numel() == N, "plan row count mismatch");
    TORCH_CHECK(!perm.has_value() || perm->numel() == N, "perm length mismatch");
    TORCH_CHECK(!unq_inv.has_value() || unq_inv->numel() == N, "unq_inv length mismatch");
    TORCH_CHECK(seg.device() == grad_out.device(), "plan and grad_out live on different devices");
    if (op == TXS_MAX || op == TXS_MAX_REFTIE) {
        TORCH_CHECK(arg.has_value(), "scatter_max backward needs arg");
        check_i32(*arg, "arg");
        TORCH_CHECK(arg->dim() == 2 && arg->size(0) == U && arg->size(1) == C, "arg must be [num_unq, channel]");
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(grad_out.device());
    const int dt = dtype_code(grad_out, "grad_out");
    const int pth = check_path(path);
    Tensor gin = at::empty({N, C}, grad_out.options());
    void *st = cur_stream(grad_out);
    auto launch = [&]() {
        return txs_scatter_backward((int)op, dt, grad_out.data_ptr(), opt_i32p(arg), opt_i32p(unq_inv),
                                    opt_i32p(perm), i32p(seg), i32p(preSum), gin.data_ptr(), N, C, U, pth, st);
    };
    int rc;
    if (holds_gil) {
        pybind11::gil_scoped_release nogil;
        rc = launch();
    } else {
        rc = launch();
    }
    check_status(rc, "scatter_backward");
    return gin;
}

Tensor backward(int64_t op, const Tensor &grad_out, const OptTensor &arg, const OptTensor &unq_inv,
                const OptTensor &perm, const Tensor &seg, const Tensor &preSum, int64_t num_total, int64_t path) {
    return backward_impl(op, grad_out, arg, unq_inv, perm, seg, preSum, num_total, path, /*holds_gil=*/true);
}

// The operators as one autograd node written in C++ (what ScatterSumFunction /
// ScatterMeanFunction / ScatterMaxFunction of scatter_op.py:24-111 are in Python): the node's
// forward and backward call the same launch functions, without the Python-side
// autograd.Function machinery, which costs more host time per call than a small input's
// kernels take on the GPU.  The gradient goes to feats only; arg is not differentiable.
struct ScatterNode : public torch::autograd::Function<ScatterNode> {
    static torch::autograd::variable_list forward(torch::autograd::AutogradContext *ctx, const Tensor &feats,
                                                  int64_t op, const OptTensor &unq_inv, const OptTensor &perm,
                                                  const Tensor &seg, const Tensor &preSum, const Tensor &slot_of,
                                                  const Tensor &heavy_ids, int64_t num_heavy, const Tensor &scratch,
                                                  int64_t max_cnt, int64_t path) {
        auto [out, arg] = forward_impl(op, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, scratch,
                                       max_cnt, path, /*holds_gil=*/PyGILState_Check() != 0);
        ctx->saved_data["op"] = op;
        ctx->saved_data["path"] = path;
        ctx->saved_data["num_total"] = feats.size(0);
        const Tensor none;
        ctx->save_for_backward({arg.has_value() ? *arg : none, unq_inv.has_value() ? *unq_inv : none,
                                perm.has_value() ? *perm : none, seg, preSum});
        ctx->set_materialize_grads(false);  // no zero tensor for the integer output's gradient slot
        if (arg.has_value()) {
            ctx->mark_non_differentiable({*arg});
            return {out, *arg};
        }
        return {out};
    }

    static torch::autograd::variable_list backward(torch::autograd::AutogradContext *ctx,
                                                   torch::autograd::variable_list grads) {
        torch::autograd::variable_list result(12);  // one slot per forward argument; only feats gets a gradient
        if (grads.empty() || !grads[0].defined()) return result;
        const auto saved = ctx->get_saved_variables();
        auto opt = [](const Tensor &t) -> OptTensor { return t.defined() ? OptTensor(t) : std::nullopt; };
        const int64_t op = ctx->saved_data["op"].toInt();
        // the engine's worker threads run this without the interpreter lock
        result[0] = backward_impl(op, grads[0].contiguous(), opt(saved[0]), opt(saved[1]), opt(saved[2]), saved[3],
                                  saved[4], ctx->saved_data["num_total"].toInt(), ctx->saved_data["path"].toInt(),
                                  /*holds_gil=*/PyGILState_Check() != 0);
        return result;
    }
};

// scatter(op, feats, <plan arguments of forward>) -> (out, arg | None), differentiable in feats
std::tuple<Tensor, OptTensor> scatter_autograd(int64_t op, const Tensor &feats, const OptTensor &unq_inv,
                                               const OptTensor &perm, const Tensor &seg, const Tensor &preSum,
                                               const Tensor &slot_of, const Tensor &heavy_ids, int64_t num_heavy,
                                               const Tensor &scratch, int64_t max_cnt, int64_t path) {
    auto res = ScatterNode::apply(feats, op, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, scratch,
                                  max_cnt, path);
    OptTensor arg;
    if (res.size() > 1) arg = res[1];
    return {res[0], arg};
}

// ---- the reference module's three functions (scatter.cpp:20-64) ------------

// The reference module's entry points take only CSR offsets, every call.  The plan that
// goes with a preSum tensor is kept for the next calls (the reference's ScatterData
// makes preSum once and then calls sum/max many times): a few entries, keyed by the
// tensor object, its memory, length and version counter.
struct CsrPlan {
    // The preSum tensor the plan was built from, held weakly: the entry dies with the
    // tensor (so the cache pins device memory only for tensors still in use) and a later
    // tensor that happens to get the same address can never match it.
    c10::weak_intrusive_ptr<c10::TensorImpl> owner;
    const void *data = nullptr;
    Tensor seg, slot_of, heavy_ids;
    uint32_t version = 0;
    int64_t numel = 0, num_total = 0, num_heavy = 0;
    // zeroed heavy-voxel tables, one per (channel count, stream): calls on one stream are
    // ordered, calls on different streams must not share a table
    std::vector<std::tuple<int64_t, void *, Tensor>> scratch;
    explicit CsrPlan(const Tensor &preSum) : owner(preSum.getIntrusivePtr()) {}
};
constexpr size_t kCsrPlanCacheSize = 8;
constexpr size_t kCsrPlanScratchKept = 4;
std::vector<CsrPlan> &csr_plan_cache() {
    // touched under the GIL only; never destroyed, so no device tensor is freed after
    // the runtime has shut down at interpreter exit
    static auto *cache = new std::vector<CsrPlan>();
    return *cache;
}

void drop_orphaned_csr_plans() {
    auto &cache = csr_plan_cache();
    cache.erase(std::remove_if(cache.begin(), cache.end(), [](const CsrPlan &p) { return p.owner.expired(); }),
                cache.end());
}

// Plans built from memory that `preSum` covers are void once it is rewritten (getPreSum
// writes through a raw pointer).
void drop_csr_plans_of(const Tensor &preSum) {
    auto &cache = csr_plan_cache();
    const char *lo = (const char *)preSum.data_ptr();
    const char *hi = lo + preSum.numel() * (int64_t)sizeof(int32_t);
    cache.erase(std::remove_if(cache.begin(), cache.end(),
                               [&](const CsrPlan &p) {
                                   const char *a = (const char *)p.data;
                                   const char *b = a + p.numel * (int64_t)sizeof(int32_t);
                                   return p.owner.expired() || (a < hi && lo < b);
                               }),
                cache.end());
}

CsrPlan &csr_plan_for(const Tensor &preSum, int64_t num_total) {
    auto &cache = csr_plan_cache();
    drop_orphaned_csr_plans();
    const uint32_t version = preSum.unsafeGetTensorImpl()->version_counter().current_version();
    for (size_t i = 0; i < cache.size(); ++i) {
        CsrPlan &p = cache[i];
        if (p.owner._unsafe_get_target() == preSum.unsafeGetTensorImpl() && p.data == preSum.data_ptr() &&
            p.numel == preSum.numel() && p.version == version && p.num_total == num_total) {
            if (i != 0) std::rotate(cache.begin(), cache.begin() + i, cache.begin() + i + 1);  // most recent first
            return cache.front();
        }
    }
    auto [seg, slot_of, heavy_ids, hs] = plan_from_presum(preSum, num_total, txs_default_heavy_threshold());
    CsrPlan p(preSum);
    p.data = preSum.data_ptr();
    p.numel = preSum.numel();
    p.seg = seg;
    p.slot_of = slot_of;
    p.heavy_ids = heavy_ids;
    p.version = version;
    p.num_total = num_total;
    p.num_heavy = hs[TXS_STAT_NUM_HEAVY];
    if (cache.size() >= kCsrPlanCacheSize) cache.pop_back();
    cache.insert(cache.begin(), std::move(p));
    return cache.front();
}

void csr_reduce(int op, Tensor feats, Tensor preSum, Tensor out, OptTensor arg, int64_t max_cnt) {
    check_dev(feats, "feats");
    check_i32(preSum, "preSum");
    check_dev(out, "out");
    TORCH_CHECK(feats.dim() == 2 && out.dim() == 2, "feats and out must be 2-D");
    TORCH_CHECK(out.scalar_type() == feats.scalar_type(), "out dtype must match feats");
    TORCH_CHECK(preSum.numel() == out.size(0) + 1, "preSum must have out.size(0)+1 entries");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(feats.device());
    const int64_t C = feats.size(1);
    void *st = cur_stream(feats);
    // Everything the launch needs is copied out of the cache entry (tensor handles, by
    // value) while the GIL is held: run_forward releases it, and another Python thread
    // may then insert into or reorder the cache.
    Tensor seg, slot_of, heavy_ids, scratch;
    int64_t num_heavy = 0;
    {
        CsrPlan &plan = csr_plan_for(preSum, feats.size(0));
        for (auto &entry : plan.scratch)
            if (std::get<0>(entry) == C && std::get<1>(entry) == st) scratch = std::get<2>(entry);
        if (!scratch.defined()) {
            scratch = make_scratch(feats.size(0), C, preSum.numel() - 1, plan.num_heavy, feats);
            // the newest few are kept: a table can hold tens of MB of partial tables
            if (plan.scratch.size() >= kCsrPlanScratchKept) plan.scratch.erase(plan.scratch.begin());
            plan.scratch.emplace_back(C, st, scratch);
        }
        seg = plan.seg;
        slot_of = plan.slot_of;
        heavy_ids = plan.heavy_ids;
        num_heavy = plan.num_heavy;
    }
    OptTensor perm, unq_inv;  // grouped rows: the per-position ids are the row-order ids
    run_forward(op, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, scratch, out, arg, max_cnt,
                TXS_PATH_AUTO);
}

void clear_csr_plan_cache() { csr_plan_cache().clear(); }
int64_t csr_plan_cache_size() {
    drop_orphaned_csr_plans();
    return (int64_t)csr_plan_cache().size();
}

// sum(feats, preSum, out, max_cnt): max_cnt only shaped the reference's thread
// blocks (scatter_kernel.cu:179); it does not change a sum and is not needed here.
void sum_ref(Tensor feats, Tensor preSum, Tensor out, int64_t max_cnt) {
    csr_reduce(TXS_SUM, feats, preSum, out, std::nullopt, max_cnt);
}

// max(feats, preSum, out, arg, max_cnt): the reference module's own entry point.
// max_cnt selected the reference's block width (scatter_kernel.cu:187) and with
// it the row reported among equal maxima; the same row is reported here.
void max_ref(Tensor feats, Tensor preSum, Tensor out, Tensor arg, int64_t max_cnt) {
    check_i32(arg, "arg");
    TORCH_CHECK(arg.sizes() == out.sizes(), "arg must have the shape of out");
    csr_reduce(TXS_MAX_REFTIE, feats, preSum, out, arg, max_cnt);
}

void get_presum_ref(Tensor unq_inv, Tensor preSum) {
    check_i32(unq_inv, "unq_inv");
    check_i32(preSum, "preSum");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(unq_inv.device());
    check_status(txs_get_presum(i32p(unq_inv), i32w(preSum), unq_inv.numel(), preSum.numel(),
                                cur_stream(unq_inv)),
                 "getPreSum");
    // preSum was rewritten through a raw pointer: say so to autograd's version counter
    // (the plans kept for sum/max are keyed on it) and drop the plans built from the old
    // contents of this storage
    preSum.unsafeGetTensorImpl()->bump_version();
    drop_csr_plans_of(preSum);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("sum", &sum_ref, "scatter_sum over CSR offsets, in place (HIP)");
    m.def("max", &max_ref, "scatter_max with arg over CSR offsets, in place (HIP)");
    m.def("getPreSum", &get_presum_ref, "CSR offsets from a sorted unq_inv (HIP)");
    m.def("build_plan", &build_plan, "build_plan(unq_inv, num_unq, heavy_threshold, unq_cnts|None, assume_sorted=False)",
          pybind11::arg("unq_inv"), pybind11::arg("num_unq"), pybind11::arg("heavy_threshold"),
          pybind11::arg("unq_cnts"), pybind11::arg("assume_sorted") = false);
    m.def("plan_from_presum", &plan_from_presum, "index preparation from CSR offsets");
    m.def("voxel_keys", &voxel_keys, "voxel_keys(points, range_lo, voxel_size, dims) -> (coors, keys, stats)");
    m.def("unique_plan", &unique_plan, "unique_plan(keys, key_bound, heavy_threshold, stats|None)");
    m.def("ingroup_inds", &ingroup_inds, "ingroup_inds(seg, perm|None, preSum, num_unq)");
    m.def("group_ranks", &group_ranks, "group_ranks(group_inds) -> int64 rank of every element inside its group");
    m.def("dynamic_point_pool", &dynamic_point_pool,
          "dynamic_point_pool(rois, pts, extra_wlh, max_pts_per_box, max_all_pts, rois_batch=None, pts_batch=None)",
          pybind11::arg("rois"), pybind11::arg("pts"), pybind11::arg("extra_wlh"), pybind11::arg("max_pts_per_box"),
          pybind11::arg("max_all_pts"), pybind11::arg("rois_batch") = pybind11::none(),
          pybind11::arg("pts_batch") = pybind11::none());
    m.def("grid_hash_build", &grid_hash_build, "build_table(coors, values) -> table");
    m.def("grid_hash_probe", &grid_hash_probe, "probe_table(coors, table) -> values");
    m.def("make_scratch", &make_scratch, "make_scratch(num_total, channel, num_unq, num_heavy, like): zeroed forward scratch");
    m.def("clear_csr_plan_cache", &clear_csr_plan_cache, "drop the plans kept for sum/max over CSR offsets");
    m.def("csr_plan_cache_size", &csr_plan_cache_size, "number of plans currently kept for sum/max over CSR offsets");
    m.def("forward", &forward,
          "forward(op, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, scratch, max_cnt, path=0)",
          pybind11::arg("op"), pybind11::arg("feats"), pybind11::arg("unq_inv"), pybind11::arg("perm"),
          pybind11::arg("seg"), pybind11::arg("preSum"), pybind11::arg("slot_of"), pybind11::arg("heavy_ids"),
          pybind11::arg("num_heavy"), pybind11::arg("scratch"), pybind11::arg("max_cnt"), pybind11::arg("path") = 0);
    m.def("scatter", &scatter_autograd,
          "scatter(op, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_heavy, scratch, max_cnt, path=0) -> "
          "(out, arg|None): forward(...) as an autograd node, differentiable in feats",
          pybind11::arg("op"), pybind11::arg("feats"), pybind11::arg("unq_inv"), pybind11::arg("perm"),
          pybind11::arg("seg"), pybind11::arg("preSum"), pybind11::arg("slot_of"), pybind11::arg("heavy_ids"),
          pybind11::arg("num_heavy"), pybind11::arg("scratch"), pybind11::arg("max_cnt"), pybind11::arg("path") = 0);
    m.def("backward", &backward, "backward(op, grad_out, arg, unq_inv, perm, seg, preSum, num_total, path=0)",
          pybind11::arg("op"), pybind11::arg("grad_out"), pybind11::arg("arg"), pybind11::arg("unq_inv"),
          pybind11::arg("perm"), pybind11::arg("seg"), pybind11::arg("preSum"), pybind11::arg("num_total"),
          pybind11::arg("path") = 0);
    m.def("kernel_name", [](bool backward, int64_t op, const Tensor &like, int64_t num_total, int64_t num_unq,
                            bool table_allowed) {
        char buf[64];
        check_status(txs_kernel_name(backward, (int)op, dtype_code(like, "like"), num_total, like.size(1), num_unq, 16,
                                     table_allowed, buf, 64),
                     "kernel_name");
        return std::string(buf);
    }, "kernel_name(backward, op, like, num_total, num_unq, table_allowed): the kernel a call on `like`-shaped rows launches");
    m.attr("PATH_AUTO") = (int)TXS_PATH_AUTO;
    m.attr("PATH_VOXEL_ORDER") = (int)TXS_PATH_VOXEL_ORDER;
    m.attr("PATH_TABLE") = (int)TXS_PATH_TABLE;
    m.def("abi_version", &txs_abi_version);
    m.def("default_heavy_threshold", &txs_default_heavy_threshold);
    m.attr("SUM") = (int)TXS_SUM;
    m.attr("MEAN") = (int)TXS_MEAN;
    m.attr("MAX") = (int)TXS_MAX;
    m.attr("MAX_REFTIE") = (int)TXS_MAX_REFTIE;

    // The reference's other three extension modules, with their own names and positional
    // signatures, so that operator_py/ingroup_inds_op.py, dynamic_point_pool_op.py and
    // grid_hash.py bind as they are (torchex_amd/_native.py registers them in sys.modules).
    auto ig = m.def_submodule("ingroup_indices", "the reference's ingroup_indices module (ingroup_inds.cpp:52-54)");
    ig.def("forward", &ingroup_inds_ref, "forward(group_inds, out_inds): rank of every element inside its group, in place");
    auto dp = m.def_submodule("dynamic_point_pool_ext",
                              "the reference's dynamic_point_pool_ext module (dynamic_point_pool.cpp:166-169)");
    dp.def("forward", &dpp_forward_ref,
           "forward(rois, pts, extra_wlh, max_num_pts_per_box, out_pts_idx, out_roi_idx, out_pts_feats), in place");
    dp.def("dynamic_point_pool_mixed_gpu", &dpp_mixed_ref,
           "dynamic_point_pool_mixed_gpu(rois, rois_batch, pts, pts_batch, extra_wlh, max_num_pts_per_box, "
           "out_pts_idx, out_roi_idx, out_pts_feats), in place");
    auto gh = m.def_submodule("grid_hash_ext", "the reference's grid_hash_ext module (grid_hash.cpp:115-118)");
    gh.def("build_table", &grid_hash_build, "build_table(coors, values) -> table");
    gh.def("probe_table", &grid_hash_probe, "probe_table(coors, table) -> values");
}
