"""The scatter operators written with stock ``torch`` CPU ops (test infrastructure).

Independent of ``scatter_oracle.c``: these go through ``Tensor.scatter_reduce_``
/ ``index_add_``, so they cross-check the C oracle with a library routine, and
they are the CPU path that ``bench.py`` times next to the GPU kernels.

Semantics follow the reference wrappers in
``torchex/operator_py/scatter_op.py`` (sum :27-50, mean :56-78, max :84-111)
for an ``unq_inv`` in arbitrary order.
"""
import torch


def _idx(unq_inv, C):
    return unq_inv.long().unsqueeze(1).expand(-1, C)


def scatter_sum(feats, unq_inv, num_unq, acc_dtype=None):
    """``out[u] = sum_{i: inv[i]==u} feats[i]`` (scatter_op.py:40-41)."""
    f = feats if acc_dtype is None else feats.to(acc_dtype)
    out = torch.zeros((num_unq, f.shape[1]), dtype=f.dtype)
    out.index_add_(0, unq_inv.long(), f)
    return out


def scatter_mean(feats, unq_inv, unq_cnts, acc_dtype=None):
    """``sum / unq_cnts`` with ``unq_cnts`` broadcast as ``[U, 1]`` (scatter_op.py:68-69)."""
    num_unq = unq_cnts.shape[0]
    s = scatter_sum(feats, unq_inv, num_unq, acc_dtype)
    return s / unq_cnts.reshape(-1, 1)


def scatter_max(feats, unq_inv, num_unq):
    """Max with first-occurrence arg (row index into ``feats``), NaN-free input.

    ``amax`` gives the values; the winner is the smallest row whose value
    equals the max (``-0.0 == +0.0`` ties as in the reference's float compare).
    """
    N, C = feats.shape
    idx = _idx(unq_inv, C)
    out = torch.zeros((num_unq, C), dtype=feats.dtype)
    out.scatter_reduce_(0, idx, feats, "amax", include_self=False)
    rows = torch.arange(N, dtype=torch.int64).unsqueeze(1).expand(-1, C)
    cand = torch.where(feats == out[unq_inv.long()], rows, torch.full_like(rows, N))
    arg = torch.full((num_unq, C), N, dtype=torch.int64)
    arg.scatter_reduce_(0, idx, cand, "amin", include_self=True)
    # value bits follow the winning row (matters only for signed zeros)
    out = torch.gather(feats, 0, arg.clamp(max=max(N - 1, 0))) if N > 0 else out
    return out, arg.to(torch.int32)


def sum_backward(g, unq_inv):
    """scatter_op.py:47-50."""
    return g[unq_inv.long()]


def mean_backward(g, unq_cnts, unq_inv):
    """scatter_op.py:74-78."""
    return (g / unq_cnts.reshape(-1, 1))[unq_inv.long()]


def max_backward(g, arg, n):
    """scatter_op.py:106-111 as intended: zeros(N, C).scatter_(0, arg, g)."""
    gin = torch.zeros((n, g.shape[1]), dtype=g.dtype)
    gin.scatter_(0, arg.long(), g)
    return gin


def step_mean_max(feats, unq_inv, unq_cnts, g_mean, g_max):
    """One forward+backward of scatter_mean and scatter_max on CPU tensors: the
    same work ``bench.py`` times on the GPU."""
    U = unq_cnts.shape[0]
    mean = scatter_mean(feats, unq_inv, unq_cnts)
    gi_mean = mean_backward(g_mean, unq_cnts, unq_inv)
    mx, arg = scatter_max(feats, unq_inv, U)
    gi_max = max_backward(g_max, arg, feats.shape[0])
    return mean, gi_mean, mx, arg, gi_max


def voxelize(points, voxel_size, pc_range):
    """The reference's ``voxelize_single`` verbatim in spirit
    (``test/test_incremental_mask.py:20-26``), on CPU tensors."""
    vs = torch.tensor(voxel_size, dtype=torch.float32)
    rng = torch.tensor(pc_range, dtype=torch.float32)
    return torch.div(points[:, :3] - rng[None, :3], vs[None, :], rounding_mode='floor').int()


def flatten_coors(coors, sizes):
    """``operator_py/grid_hash.py:7-15`` / ``operator_py/incremental_points.py:18-19``."""
    x, y, z = coors[:, 0].long(), coors[:, 1].long(), coors[:, 2].long()
    return x * (sizes[1] * sizes[2]) + y * sizes[2] + z
