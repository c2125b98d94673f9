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

There is no PyTorch fallback: everything runs in the HIP kernels behind
``scatter_ext``.
"""
import torch
from torch.autograd import Function

from ._native import scatter_ext

_SUM, _MEAN, _MAX = scatter_ext.SUM, scatter_ext.MEAN, scatter_ext.MAX


class ScatterData:
    """Index bundle shared by the scatter operators (``scatter_op.py:7-21``).

    Public attributes as in the reference: ``unq_inv`` (int32 ``[N]``),
    ``unq_cnts`` (``[U, 1]``, dtype kept), ``preSum`` (int32 ``[U+1]``),
    ``max_cnt`` (int), ``num_unq`` (int).  Additional cached attributes used by
    the kernels: ``perm`` (int32 ``[N]`` row at each voxel-sorted position, or
    ``None`` when ``unq_inv`` is already non-decreasing), ``seg`` (int32 ``[N]``
    voxel at each sorted position, bit 31 marking voxels reduced through
    atomics), ``slot_of`` / ``heavy_ids`` (table of those voxels).
    """

    def __init__(self, unq_inv, unq_cnts, heavy_threshold=None, max_tie_rule="first") -> None:
        assert unq_inv.ndim in (
            1, 2), f"unq_inv in ScatterData should be 1 or 2-dims, but got {unq_inv.ndim}-dims"
        assert unq_cnts.ndim in (
            1, 2), f"unq_cnts in ScatterData should be 1 or 2-dims, but got {unq_cnts.ndim}-dims"
        self.unq_inv = unq_inv.int()
        if unq_cnts.ndim == 1:
            self.unq_cnts = unq_cnts.unsqueeze(-1)
        else:
            self.unq_cnts = unq_cnts
        if max_tie_rule not in ("first", "reference"):
            raise ValueError("max_tie_rule must be 'first' or 'reference'")
        # which row scatter_max reports among equal maxima: the smallest row
        # index, or the row the reference kernel's shuffle tree would keep
        self.max_tie_rule = max_tie_rule
        if heavy_threshold is None:
            heavy_threshold = scatter_ext.default_heavy_threshold()
        self.heavy_threshold = int(heavy_threshold)
        flat = self.unq_inv.reshape(-1).contiguous()
        num_unq = self.unq_cnts.shape[0]
        cnts64 = self.unq_cnts.reshape(-1).long().contiguous()
        (self.preSum, self.perm, self.seg, self.slot_of, self.heavy_ids,
         stats) = scatter_ext.build_plan(flat, num_unq, self.heavy_threshold, cnts64)
        # same consistency check as the reference (scatter_op.py:19), made on
        # the recomputed histogram so that a stale unq_cnts is caught too
        assert stats[5] == 0, "unq_cnts is not the histogram of unq_inv"
        self.num_total = flat.shape[0]
        self.is_sorted = self.perm is None
        self.max_cnt = int(stats[2])
        self.num_special = int(stats[3])
        self.num_unq = num_unq
        self._scratch = {}

    def scratch(self, channel):
        """Zeroed table the special voxels are merged in; the kernels leave it
        zeroed again, so one buffer per channel count is kept for reuse."""
        buf = self._scratch.get(channel)
        if buf is None:
            buf = scatter_ext.make_scratch(self.num_special, channel, self.seg)
            self._scratch[channel] = buf
        return buf


def _check_feats(feats, data):
    if feats.dim() != 2:
        raise RuntimeError(f"feats must be [num_total, channel], got {tuple(feats.shape)}")
    if feats.shape[0] != data.num_total:
        raise RuntimeError(
            f"feats has {feats.shape[0]} rows but ScatterData was built for {data.num_total}")


def _forward(op, feats, data):
    _check_feats(feats, data)
    return scatter_ext.forward(op, feats, data.perm, data.seg, data.preSum, data.slot_of,
                               data.heavy_ids, data.scratch(feats.shape[1]), data.max_cnt)


def _backward(op, g, arg, data):
    return scatter_ext.backward(op, g.contiguous(), arg, data.perm, data.seg, data.preSum,
                                data.num_total)


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
        several rows tie, the smallest row wins (``data.max_tie_rule ==
        "first"``, the default) or the row the reference kernel would report
        for the voxel's rows in ascending order (``"reference"``).
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


scatter_sum = ScatterSumFunction.apply
scatter_mean = ScatterMeanFunction.apply
scatter_max = ScatterMaxFunction.apply
getPreSum = GetPreSumFunction.apply
