"""Voxel scatter-reductions with the call surface of TorchEx's scatter operators.

Mirrors ``torchex/operator_py/scatter_op.py``: ``ScatterData(unq_inv, unq_cnts)``
bundles the index data once per voxelization, and ``scatter_sum`` /
``scatter_mean`` / ``scatter_max`` are ``autograd.Function.apply`` callables taking
``(feats, data)``.  Differences from the reference, all extensions:

* ``unq_inv`` may be in any order (the reference needs rows grouped by voxel:
  its ``getPreSum`` finds run boundaries, ``scatter_kernel.cu:85-100``);
* ``feats`` may be float32, float16 or bfloat16 (sums accumulate in fp32);
* ``scatter_max`` has a working backward (``scatter_op.py:106-111`` raises as
  written; the intended ``zeros.scatter_(0, arg, g)`` is what runs here);
* ``scatter_mean`` is one fused kernel rather than sum followed by a divide.

Which row ``scatter_max`` reports among equal maxima: when ``unq_inv`` arrives
grouped by voxel -- the only order the reference accepts (``scatter_op.py:18-19``) --
the row the reference kernel itself reports (``scatter_kernel.cu:41-83,146-152``), so a
program written for the reference sees the same ``arg``; for any other order, where the
reference is undefined, the smallest row index.  ``max_tie_rule`` forces either.

There is no PyTorch fallback: everything runs in the HIP kernels behind
``scatter_ext``.
"""
import torch
from torch.autograd import Function

from ._native import scatter_ext

_SUM, _MEAN, _MAX = scatter_ext.SUM, scatter_ext.MEAN, scatter_ext.MAX


def _check_tie_rule(rule):
    if rule not in (None, "first", "reference"):
        raise ValueError("max_tie_rule must be None, 'first' or 'reference'")


def _resolve_tie_rule(rule, grouped):
    """Which row scatter_max reports among equal maxima.  ``None`` (the default) means:
    the reference kernel's own winner when the rows arrived grouped by voxel, which is
    the only input the reference defines (scatter_op.py:18-19), and the smallest row
    index otherwise."""
    if rule is None:
        return "reference" if grouped else "first"
    return rule


_SCRATCH_KEPT = 4   # forward workspaces a ScatterData keeps (most recently used)


class ScatterData:
    """Index bundle shared by the scatter operators (``scatter_op.py:7-21``).

    Public attributes as in the reference: ``unq_inv`` (int32 ``[N]``),
    ``unq_cnts`` (``[U, 1]``, dtype kept), ``preSum`` (int32 ``[U+1]``),
    ``max_cnt`` (int), ``num_unq`` (int).  Additional cached attributes used by
    the kernels: ``perm`` (int32 ``[N]`` row at each voxel-sorted position, or
    ``None`` when ``unq_inv`` is already non-decreasing), ``seg`` (int32 ``[N]``
    voxel at each sorted position, bit 31 marking voxels reduced through
    atomics), ``slot_of`` / ``heavy_ids`` (table of those voxels).

    ``heavy_threshold`` (default 64, at least 16): voxels with more rows are reduced
    through atomics.  With the default, a plan whose only heavy voxels are a handful just
    above it (at most 64 of them, none above 96 rows) keeps them ordinary, so that a
    forward call is a single kernel; ``num_heavy`` is then 0.

    ``max_tie_rule``: ``"reference"`` reports, among equal maxima, the row the reference
    kernel reports for the voxel's rows taken in ascending order; ``"first"`` the
    smallest row index; ``None`` (default) picks ``"reference"`` for grouped input and
    ``"first"`` otherwise.  The rule in force is kept as ``self.max_tie_rule``.

    ``path`` (attribute, default ``scatter_ext.PATH_AUTO``) lets a caller force the
    voxel-order kernels (``PATH_VOXEL_ORDER``) or the row-order table kernels for inputs
    with few voxels (``PATH_TABLE``; raises where they do not apply).

    ``assume_sorted=True`` states that ``unq_inv`` is already grouped (the order the
    reference requires): the sort is then not queued at all; the statement is
    verified on the device and an unsorted ``unq_inv`` raises.
    """

    def __init__(self, unq_inv, unq_cnts, heavy_threshold=None, max_tie_rule=None,
                 assume_sorted=False) -> None:
        assert unq_inv.ndim in (
            1, 2), f"unq_inv in ScatterData should be 1 or 2-dims, but got {unq_inv.ndim}-dims"
        assert unq_cnts.ndim in (
            1, 2), f"unq_cnts in ScatterData should be 1 or 2-dims, but got {unq_cnts.ndim}-dims"
        self.unq_inv = unq_inv.int()
        if unq_cnts.ndim == 1:
            self.unq_cnts = unq_cnts.unsqueeze(-1)
        else:
            self.unq_cnts = unq_cnts
        _check_tie_rule(max_tie_rule)
        if heavy_threshold is None:
            heavy_threshold = scatter_ext.default_heavy_threshold()
        self.heavy_threshold = int(heavy_threshold)
        flat = self.unq_inv.reshape(-1).contiguous()
        num_unq = self.unq_cnts.shape[0]
        cnts64 = self.unq_cnts.reshape(-1).long().contiguous()
        (self.preSum, self.perm, self.seg, self.slot_of, self.heavy_ids,
         stats) = scatter_ext.build_plan(flat, num_unq, self.heavy_threshold, cnts64, bool(assume_sorted))
        # same consistency check as the reference (scatter_op.py:19), made on
        # the recomputed histogram so that a stale unq_cnts is caught too
        assert stats[5] == 0, "unq_cnts is not the histogram of unq_inv"
        self.num_total = flat.shape[0]
        self.is_sorted = self.perm is None
        # voxel id of every row in row order, for the row-order (few-voxel) kernels; grouped
        # rows need none: their per-position ids are the row-order ids
        self.row_ids = None if self.is_sorted else flat
        self.path = scatter_ext.PATH_AUTO
        self.max_tie_rule = _resolve_tie_rule(max_tie_rule, self.is_sorted)
        self.max_cnt = int(stats[2])
        self.num_special = int(stats[3])
        self.num_heavy = int(stats[7])
        self.num_unq = num_unq
        self._scratch = {}

    @classmethod
    def from_keys(cls, keys, key_bound, heavy_threshold=None, max_tie_rule=None, _stats=None):
        """ScatterData straight from voxel keys (any non-negative int ids below
        ``key_bound``, e.g. linear voxel ids): computes what ``torch.unique(keys,
        return_inverse=True, return_counts=True)`` returns -- kept as ``unq_keys``,
        ``unq_inv``, ``unq_cnts`` -- and the scatter plan from ONE sort of the keys,
        where ``torch.unique`` followed by ``ScatterData(...)`` sorts twice."""
        _check_tie_rule(max_tie_rule)
        self = cls.__new__(cls)
        if heavy_threshold is None:
            heavy_threshold = scatter_ext.default_heavy_threshold()
        self.heavy_threshold = int(heavy_threshold)
        flat = keys.reshape(-1)
        if flat.dtype not in (torch.int32, torch.int64):
            flat = flat.int()
        flat = flat.contiguous()
        (self.unq_keys, self.unq_inv, cnts, self.preSum, self.perm, self.seg, self.slot_of,
         self.heavy_ids, stats) = scatter_ext.unique_plan(flat, int(key_bound), self.heavy_threshold, _stats)
        self.unq_cnts = cnts.unsqueeze(-1)
        self.num_total = flat.shape[0]
        self.is_sorted = self.perm is None
        self.row_ids = None if self.is_sorted else self.unq_inv
        self.path = scatter_ext.PATH_AUTO
        self.max_tie_rule = _resolve_tie_rule(max_tie_rule, self.is_sorted)
        self.max_cnt = int(stats[2])
        self.num_special = int(stats[3])
        self.num_heavy = int(stats[7])
        self.num_unq = int(stats[6])
        self._scratch = {}
        return self

    @classmethod
    def from_points(cls, points, voxel_size, pc_range, heavy_threshold=None, max_tie_rule=None):
        """Dynamic voxelization in one go: voxel coordinates as the reference's
        ``voxelize_single`` computes them (``test/test_incremental_mask.py:20-26``),
        x-major linear keys (``operator_py/incremental_points.py:18-19``), unique and
        scatter plan.  Points outside ``pc_range`` raise.  Extra attributes:
        ``coors`` (int32 ``[N, 3]``), ``spatial_size``."""
        coors, keys, stats, dims = _voxel_keys(points, voxel_size, pc_range)
        self = cls.from_keys(keys, dims[0] * dims[1] * dims[2], heavy_threshold, max_tie_rule, _stats=stats)
        self.coors = coors
        self.spatial_size = dims
        return self

    def scratch(self, channel):
        """Forward workspace: the zeroed table the heavy voxels are merged in (one row each,
        left zeroed again by the kernels) and, for inputs with few voxels, room for the
        partial tables of the row-order kernels.  Buffers are kept for reuse -- one per
        channel count and per stream (calls queued on one stream are ordered, and forwards
        that run concurrently on different streams each get a workspace of their own), the
        ``_SCRATCH_KEPT`` most recently used at most."""
        key = (channel, torch.cuda.current_stream(self.seg.device).stream_id)
        buf = self._scratch.pop(key, None)
        if buf is None:
            buf = scatter_ext.make_scratch(self.num_total, channel, self.num_unq, self.num_heavy, self.seg)
            # the few most recently used are kept (a buffer can hold tens of MB of partial
            # tables); one that is dropped was only ever used on its own stream, so the
            # allocator may hand its memory on as soon as that stream's queued work allows
            while len(self._scratch) >= _SCRATCH_KEPT:
                self._scratch.pop(next(iter(self._scratch)))
        self._scratch[key] = buf          # most recently used last
        return buf

    def forward_args(self, channel):
        """Plan arguments of ``scatter_ext.forward`` after ``(op, feats)``."""
        return (self.row_ids, self.perm, self.seg, self.preSum, self.slot_of, self.heavy_ids, self.num_heavy,
                self.scratch(channel), self.max_cnt, self.path)

    def backward_args(self):
        """Plan arguments of ``scatter_ext.backward`` after ``(op, grad_out, arg)``."""
        return (self.row_ids, self.perm, self.seg, self.preSum, self.num_total, self.path)


def _check_feats(feats, data):
    if feats.dim() != 2:
        raise RuntimeError(f"feats must be [num_total, channel], got {tuple(feats.shape)}")
    if feats.shape[0] != data.num_total:
        raise RuntimeError(
            f"feats has {feats.shape[0]} rows but ScatterData was built for {data.num_total}")


def _forward(op, feats, data):
    _check_feats(feats, data)
    return scatter_ext.forward(op, feats, *data.forward_args(feats.shape[1]))


def _backward(op, g, arg, data):
    return scatter_ext.backward(op, g.contiguous(), arg, *data.backward_args())


class ScatterSumFunction(Function):

    @staticmethod
    def forward(ctx, feats: torch.Tensor, data: ScatterData):
        """scatter_sum forward (``scatter_op.py:27-44``).
        Args:
            feats (torch.Tensor, float32/float16/bfloat16): [num_total, channel]
            data (ScatterData)
        Returns: [num_unq, channel], dtype of feats
        """
        out, _ = _forward(_SUM, feats, data)
        ctx.data = data
        return out

    @staticmethod
    def backward(ctx, g):
        # g[unq_inv] (scatter_op.py:47-50)
        return _backward(_SUM, g, None, ctx.data), None


class ScatterMeanFunction(Function):

    @staticmethod
    def forward(ctx, feats: torch.Tensor, data: ScatterData):
        """scatter_mean forward (``scatter_op.py:56-71``): sum / unq_cnts, with
        the division by the fp32-converted count fused into the reduction."""
        out, _ = _forward(_MEAN, feats, data)
        ctx.data = data
        return out

    @staticmethod
    def backward(ctx, g):
        # (g / unq_cnts)[unq_inv] (scatter_op.py:74-78)
        return _backward(_MEAN, g, None, ctx.data), None


class ScatterMaxFunction(Function):

    @staticmethod
    def forward(ctx, feats: torch.Tensor, data: ScatterData):
        """scatter_max forward (``scatter_op.py:84-103``).
        Returns ``(out [num_unq, channel], arg [num_unq, channel] int32)`` where
        ``arg`` is the row index into ``feats`` of the winning element.  When
        several rows tie, ``data.max_tie_rule`` decides: ``"reference"`` (the
        default for grouped ``unq_inv``) reports the row the reference kernel
        reports, ``"first"`` (the default for any other order) the smallest row.
        """
        op = scatter_ext.MAX_REFTIE if data.max_tie_rule == "reference" else _MAX
        out, arg = _forward(op, feats, data)
        ctx.save_for_backward(arg)
        ctx.mark_non_differentiable(arg)
        # no zero tensor is made for the gradient slot of the integer output
        ctx.set_materialize_grads(False)
        ctx.data = data
        return out, arg

    @staticmethod
    def backward(ctx, g_out, g_arg):
        # zeros(N, C).scatter_(0, arg, g_out) (scatter_op.py:106-111, as intended)
        if g_out is None:
            return None, None
        (arg,) = ctx.saved_tensors
        return _backward(_MAX, g_out, arg, ctx.data), None


class GetPreSumFunction(Function):

    @staticmethod
    def forward(ctx, unq_inv: torch.Tensor):
        """CSR offsets from a SORTED ``unq_inv`` (``scatter_op.py:117-131``)."""
        if unq_inv.dtype != torch.int32:
            unq_inv = unq_inv.int()
        num_unq = int(unq_inv[-1]) + 2
        preSum = unq_inv.new_zeros(num_unq)
        scatter_ext.getPreSum(unq_inv.contiguous(), preSum)
        ctx.mark_non_differentiable(preSum)
        return preSum

    @staticmethod
    def backward(ctx, g):
        return None


def _voxel_keys(points, voxel_size, pc_range):
    import math
    lo = [float(v) for v in pc_range[:3]]
    hi = [float(v) for v in pc_range[3:6]]
    vs = [float(v) for v in voxel_size]
    dims = [max(1, int(math.ceil((h - l) / v - 1e-6))) for l, h, v in zip(lo, hi, vs)]
    coors, keys, stats = scatter_ext.voxel_keys(points, lo, vs, dims)
    return coors, keys, stats, dims


def voxelize(points, voxel_size, pc_range):
    """Voxel coordinates of every point: ``torch.div(points[:, :3] - pc_range[:3],
    voxel_size, rounding_mode='floor').int()`` (the reference's ``voxelize_single``,
    ``test/test_incremental_mask.py:20-26``), int32 ``[N, 3]``, computed by one HIP
    kernel.  No range check is made here (as in the reference)."""
    return _voxel_keys(points, voxel_size, pc_range)[0]


def ingroup_inds(group_inds):
    """Rank of every element inside its group (``operator_py/ingroup_inds_op.py``).
    ``group_inds``: integer ``[N]`` group ids; returns ``[N]`` of the same dtype.
    Ranks ascend with the element index inside a group; the reference hands
    them out with an atomic counter, i.e. in arbitrary order."""
    if group_inds.numel() == 0:
        return torch.zeros_like(group_inds)
    # index preparation of the ids + one rank kernel; the largest id is read on the host (as
    # the reference does for every call) only when an id reaches the number of elements
    out = scatter_ext.group_ranks(group_inds)
    return out.to(group_inds.dtype).reshape(group_inds.shape)


# The reference binds ``scatter_sum = ScatterSumFunction.apply`` etc. (scatter_op.py:138-141).
# Same call form and results here; the autograd node behind these three is the C++ one in
# scatter_ext (``scatter_ext.scatter``), which spares the host the Python-side
# ``autograd.Function`` machinery on every call -- on small inputs that costs more than the
# kernels.  The ``*Function`` classes above stay usable through ``.apply``.

def scatter_sum(feats, data):
    """``scatter_sum(feats, data) -> [num_unq, channel]`` (``scatter_op.py:27-50``)."""
    _check_feats(feats, data)
    return scatter_ext.scatter(_SUM, feats, *data.forward_args(feats.shape[1]))[0]


def scatter_mean(feats, data):
    """``scatter_mean(feats, data) -> [num_unq, channel]`` (``scatter_op.py:56-78``)."""
    _check_feats(feats, data)
    return scatter_ext.scatter(_MEAN, feats, *data.forward_args(feats.shape[1]))[0]


def scatter_max(feats, data):
    """``scatter_max(feats, data) -> (out, arg)`` (``scatter_op.py:84-111``); the tie rule is
    ``data.max_tie_rule`` as described for ``ScatterMaxFunction``."""
    _check_feats(feats, data)
    op = scatter_ext.MAX_REFTIE if data.max_tie_rule == "reference" else _MAX
    return scatter_ext.scatter(op, feats, *data.forward_args(feats.shape[1]))


getPreSum = GetPreSumFunction.apply
