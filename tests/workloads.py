"""Seeded synthetic inputs for the voxel scatter path: test and benchmark
infrastructure (used by the tests, ``bench.py`` and the smoke entry point), not part
of the product package.

Every workload is generated on the CPU with ``torch.Generator().manual_seed``
and returned as CPU tensors, so a CPU checker and the GPU kernels see identical
data.  Voxel keys are int64 linear ids ``(ix * Y + iy) * Z + iz`` (x-major, the
linearisation of the reference's ``operator_py/incremental_points.py:18-19``);
``unq_inv`` / ``unq_cnts`` come from ``torch.unique(keys, return_inverse=True,
return_counts=True)`` and the point order stays as generated (unsorted).
"""
import math
from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class Workload:
    name: str
    feats: torch.Tensor      # [N, C] float32
    unq_inv: torch.Tensor    # [N] int64, as torch.unique returns it
    unq_cnts: torch.Tensor   # [U] int64
    sorted: bool = False

    @property
    def N(self):
        return self.feats.shape[0]

    @property
    def C(self):
        return self.feats.shape[1]

    @property
    def U(self):
        return self.unq_cnts.shape[0]


def _unique(keys):
    _, inv, cnt = torch.unique(keys, return_inverse=True, return_counts=True)
    return inv, cnt


def reference_test_groups(channel=128, num_group=500, cnt_min=100, cnt_max=5000, seed=0,
                          perm_seed=0):
    """The data of the reference's own test (``test/test_scatter.py:8-24``): 500
    groups in sorted order, sizes from ``np.random.seed(0); randint(100, 5000)``,
    each group a random permutation of ``0..cnt-1`` replicated over the channels.
    Returns the workload and, per group, the position of the maximum.
    """
    rs = np.random.RandomState(seed)
    cnts = np.array([rs.randint(cnt_min, cnt_max) for _ in range(num_group)], dtype=np.int64)
    g = torch.Generator().manual_seed(perm_seed)
    cols, invs = [], []
    for gid, c in enumerate(cnts.tolist()):
        cols.append(torch.randperm(c, generator=g).to(torch.float32))
        invs.append(torch.full((c,), gid, dtype=torch.int64))
    col = torch.cat(cols)
    feats = col.unsqueeze(1).expand(-1, channel).contiguous()
    return Workload("reference_test_groups", feats, torch.cat(invs), torch.from_numpy(cnts), True)


def uniform_box(N=200_000, C=64, seed=1):
    """Uniform points in a 150 m x 150 m x 6 m box, 0.32 x 0.32 x 6 m voxels."""
    g = torch.Generator().manual_seed(seed)
    xy = torch.rand((N, 2), generator=g) * 150.0 - 75.0
    z = torch.rand((N,), generator=g) * 6.0 - 3.0
    X = Y = int(math.ceil(150.0 / 0.32))
    ix = ((xy[:, 0] + 75.0) / 0.32).floor().long().clamp_(0, X - 1)
    iy = ((xy[:, 1] + 75.0) / 0.32).floor().long().clamp_(0, Y - 1)
    iz = ((z + 3.0) / 6.0).floor().long().clamp_(0, 0)
    keys = (ix * Y + iy) * 1 + iz
    feats = torch.randn((N, C), generator=g)
    inv, cnt = _unique(keys)
    return Workload("uniform_box", feats, inv, cnt)


def _lidar_keys(N, g, pillars=False):
    u = torch.rand((N,), generator=g, dtype=torch.float64)
    r = 1.0 / (0.5 - u * (0.5 - 1.0 / 75.0))           # inverse CDF of p(r) ~ r^-2 on [2, 75]
    th = torch.rand((N,), generator=g, dtype=torch.float64) * (2.0 * math.pi)
    x = r * torch.cos(th)
    y = r * torch.sin(th)
    z = torch.rand((N,), generator=g, dtype=torch.float64) * 6.0 - 2.0
    X = Y = 750
    Z = 30
    ix = ((x + 75.0) / 0.2).floor().long().clamp_(0, X - 1)
    iy = ((y + 75.0) / 0.2).floor().long().clamp_(0, Y - 1)
    iz = ((z + 2.0) / 0.2).floor().long().clamp_(0, Z - 1)
    if pillars:   # one voxel per 0.2 m x 0.2 m column, whatever z
        return ix * Y + iy, X * Y
    return (ix * Y + iy) * Z + iz, X * Y * Z


def lidar_sweep(N=1_000_000, C=128, seed=2):
    """LiDAR-like skew: range density ~ 1/r^2 on [2 m, 75 m], 0.2 m cubic voxels."""
    g = torch.Generator().manual_seed(seed)
    keys, _ = _lidar_keys(N, g)
    feats = torch.randn((N, C), generator=g)
    inv, cnt = _unique(keys)
    return Workload("lidar_sweep", feats, inv, cnt)


def lidar_pillars(N=1_000_000, C=128, seed=2):
    """The points of ``lidar_sweep`` (same seed, same draws) binned into 0.2 m x 0.2 m
    pillars over the full height: the heavy-tailed occupancy a real sweep has near the
    sensor (about 89k pillars, the fullest above 1.4k points, two thirds of the points in
    pillars of more than 64)."""
    g = torch.Generator().manual_seed(seed)
    keys, _ = _lidar_keys(N, g, pillars=True)
    feats = torch.randn((N, C), generator=g)
    inv, cnt = _unique(keys)
    return Workload("lidar_pillars", feats, inv, cnt)


def zipf_contention(N=2_000_000, C=16, num_ids=1024, s=1.2, seed=4):
    """Zipf(s) draw over ``num_ids`` voxel ids: a few voxels get >100k points."""
    g = torch.Generator().manual_seed(seed)
    k = torch.arange(1, num_ids + 1, dtype=torch.float64)
    p = k.pow(-s)
    cdf = torch.cumsum(p / p.sum(), 0)
    ids = torch.searchsorted(cdf, torch.rand((N,), generator=g, dtype=torch.float64)).clamp_(max=num_ids - 1)
    feats = torch.rand((N, C), generator=g) * 2.0 - 1.0
    inv, cnt = _unique(ids)
    return Workload("zipf_contention", feats, inv, cnt)


def multi_sweep(N_per=1_000_000, sweeps=4, C=32, seed0=50):
    """Several LiDAR sweeps with the batch index folded into the voxel key."""
    keys, feats = [], []
    for b in range(sweeps):
        g = torch.Generator().manual_seed(seed0 + b)
        k, vol = _lidar_keys(N_per, g)
        keys.append(k + b * vol)
        feats.append(torch.randn((N_per, C), generator=g))
    inv, cnt = _unique(torch.cat(keys))
    return Workload("multi_sweep", torch.cat(feats), inv, cnt)


def upstream_grad(U, C, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn((U, C), generator=g)


def algorithmic_bytes(op, N, C, U, elem_bytes=4):
    """Bytes the operator must move: features once, int32 ``unq_inv`` once,
    int64 counts (mean), outputs once; ``arg`` is int32."""
    e = elem_bytes
    table = {
        "sum_fwd": N * C * e + 4 * N + U * C * e,
        "mean_fwd": N * C * e + 4 * N + 8 * U + U * C * e,
        "max_fwd": N * C * e + 4 * N + U * C * e + 4 * U * C,
        "sum_bwd": U * C * e + 4 * N + N * C * e,
        "mean_bwd": U * C * e + 8 * U + 4 * N + N * C * e,
        "max_bwd": U * C * e + 4 * U * C + 4 * N + N * C * e,
    }
    return table[op]
