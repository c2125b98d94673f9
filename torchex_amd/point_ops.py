"""Callers on either side of the scatter path, with the reference's call surface:
``dynamic_point_pool`` (``torchex/operator_py/dynamic_point_pool_op.py``) and
``grid_hash_build`` / ``grid_hash_probe`` / ``GridHash``
(``torchex/operator_py/grid_hash.py``).  All device work runs in HIP kernels behind
``scatter_ext``; there is no PyTorch fallback.
"""
import torch

from ._native import scatter_ext


def dynamic_point_pool(rois, pts, extra_wlh, max_inbox_point, max_all_pts=50000, rois_batch=None,
                       pts_batch=None):
    """Points inside the boxes enlarged by ``extra_wlh`` (dynamic_point_pool_op.py:17-57).

    Args:
        rois (Tensor): float32 ``[N, 7]`` boxes in LiDAR coordinates, ``(x, y, z)`` the
            bottom centre, then ``w, l, h, rz``.
        pts (Tensor): float32 ``[npoints, 3]``.
        extra_wlh (sequence of 3 floats), max_inbox_point (int), max_all_pts (int).
        rois_batch, pts_batch (Tensor, optional, both or neither): integer ``[N]`` /
            ``[npoints]`` sample index of every box and point; a point is then matched
            only with the boxes of its own sample (the extension's
            ``dynamic_point_pool_mixed_gpu``, src/dynamic_point_pool/dynamic_point_pool.cpp:108-164).
    Returns ``(out_pts_idx int64 [M], out_roi_idx int64 [M], out_pts_feats float32 [M, 13])``.
    Entries come in (box, point) order; the reference's atomic counters leave the order
    (and, under a cap, the surviving subset) to thread timing.  With no hit at all the
    reference returns one placeholder entry (-1, -1, zeros); so does this.
    """
    assert len(rois) > 0
    assert (rois_batch is None) == (pts_batch is None)
    if rois_batch is not None:
        rois_batch = rois_batch.int().contiguous()
        pts_batch = pts_batch.int().contiguous()
    idx, roi, feats = scatter_ext.dynamic_point_pool(
        rois.contiguous(), pts.contiguous(), [float(v) for v in extra_wlh], int(max_inbox_point),
        int(max_all_pts), rois_batch, pts_batch)
    if idx.numel() == 0:   # the reference fakes a non-empty output (dynamic_point_pool_op.py:41-45)
        idx = pts.new_full((1,), -1, dtype=torch.long)
        roi = pts.new_full((1,), -1, dtype=torch.long)
        feats = pts.new_zeros((1, 13), dtype=torch.float)
    return idx, roi, feats


def grid_hash_build(coors, values):
    """Hash table ``[up_2n(N), 2]`` int32 of (key, value), -1 in empty slots
    (``grid_hash.py:25-38``, ``grid_hash.cpp:49-78``).  Keys must be unique."""
    return scatter_ext.grid_hash_build(coors.contiguous(), values.contiguous())


def grid_hash_probe(coors, table):
    """Value stored for each key; -1 for a key that is absent (``grid_hash.py:40-53``;
    the reference's kernel asserts on an absent key)."""
    return scatter_ext.grid_hash_probe(coors.contiguous(), table.contiguous())


def _flatten_3dim_coors(coors, sizes):
    # grid_hash.py:7-15
    x, y, z = coors[:, 0], coors[:, 1], coors[:, 2]
    return x * (sizes[1] * sizes[2]) + y * sizes[2] + z


class GridHash:
    """Map from voxel coordinates to compact indices (``grid_hash.py:59-104``):
    ``GridHash(coors)`` indexes the distinct rows of ``coors`` (``[N, 3]`` or flat ``[N]``
    integer keys) in sorted order, ``probe(coors)`` returns their indices.

    The reference makes the rows unique with ``torch.unique(coors, dim=0)``; here the keys
    are linearised first and made unique by the same single radix sort that serves the
    scatter plan, which orders them identically (row-lexicographic == linear key order).
    """

    def __init__(self, coors, debug=False):
        if coors.ndim == 1:
            self.dim_size = None
            keys = coors
        else:
            assert coors.ndim == 2 and coors.size(1) == 3
            self.dim_size = tuple(int(v) + 1 for v in coors.amax(0).tolist())   # grid_hash.py:17-23
            assert self.dim_size[0] * self.dim_size[1] * self.dim_size[2] < 2 ** 31
            keys = _flatten_3dim_coors(coors.long(), self.dim_size)
        if keys.numel() == 0:
            raise ValueError("GridHash needs at least one coordinate")
        bound = int(keys.max()) + 1 if self.dim_size is None else \
            self.dim_size[0] * self.dim_size[1] * self.dim_size[2]
        unq_keys = scatter_ext.unique_plan(keys.int().contiguous(), bound,
                                           scatter_ext.default_heavy_threshold(), None)[0]
        unq_keys = unq_keys.contiguous()
        values = torch.arange(len(unq_keys), device=unq_keys.device, dtype=unq_keys.dtype)
        self.table = grid_hash_build(unq_keys, values)
        self.valid_mask = self.table[:, 0] != -1
        self.valid_table = self.table[self.valid_mask]
        if debug:
            assert self.valid_mask.sum() == len(unq_keys)
            assert self.valid_table[:, 1].max() + 1 == len(unq_keys)
            assert len(self.valid_table[:, 1]) == len(torch.unique(self.valid_table[:, 1]))
            if not self.valid_mask.all():
                assert (self.table[~self.valid_mask, 0] == -1).all()

    def probe(self, coors):
        if coors.ndim == 2:
            assert coors.size(1) == 3
            coors = _flatten_3dim_coors(coors, self.dim_size)
        else:
            assert coors.ndim == 1
        if coors.dtype != torch.int32:
            coors = coors.int()
        return grid_hash_probe(coors, self.table)
