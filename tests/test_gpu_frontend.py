"""GPU parity of the callers on either side of the scatter path: voxelization, the fused
unique + plan, and ingroup_inds.  Integer work: everything is compared bit-exact, against
the C oracle and against stock torch CPU routines (torch.div floor mode, torch.unique)."""
import sys

import numpy as np
import pytest
import torch

from oracle import c_oracle as orc
from oracle import torch_oracle as tor
from torchex_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def tx():
    import torchex_amd
    return torchex_amd


def _edge_points(n, seed):
    g = torch.Generator().manual_seed(seed)
    pts = torch.rand((n, 5), generator=g) * 160.0 - 80.0
    pts[:, 2] = torch.rand((n,), generator=g) * 6.0 - 2.0
    edges = torch.arange(-80.0, 80.0, 0.25)[:640]
    pts[:640, 0] = edges                                             # exactly on cell edges
    pts[640:1280, 1] = torch.nextafter(edges, torch.tensor(-1e9))    # one ulp below
    pts[1280:1920, 0] = torch.nextafter(edges, torch.tensor(1e9))    # one ulp above
    return pts


def test_voxelize_matches_torch_floor_division():
    T = tx()
    voxel_size, pc_range = [0.25, 0.25, 0.4], [-80, -80, -2, 80, 80, 4]
    pts = _edge_points(200_000, 41)
    pts[5] = torch.tensor([-80.5, 90.0, 7.0, 0, 0])    # outside the range: coordinates still as torch gives
    say("[case] voxelize", tuple(pts.shape))
    got = T.voxelize(pts.to(DEV), voxel_size, pc_range).cpu()
    want = tor.voxelize(pts, voxel_size, pc_range)
    assert got.dtype == torch.int32 and torch.equal(got, want)
    oc, _ = orc.voxelize(pts.numpy(), voxel_size, pc_range[:3], [640, 640, 15])
    assert np.array_equal(got.numpy(), oc)


@pytest.mark.parametrize("case", ["lidar", "sorted", "few_keys", "single", "sparse_ids"])
def test_from_keys_equals_torch_unique_and_scatter_data(case):
    T = tx()
    g = torch.Generator().manual_seed(7)
    if case == "lidar":
        keys, bound = workloads._lidar_keys(300_000, g)
    elif case == "sorted":
        keys = torch.sort(torch.randint(0, 5000, (50_000,), generator=g)).values
        bound = 5000
    elif case == "few_keys":
        keys = torch.randint(0, 7, (40_000,), generator=g) * 1000 + 3
        bound = 7003
    elif case == "single":
        keys = torch.full((1000,), 12345)
        bound = 20000
    else:
        keys = torch.randint(0, 2**30, (100_000,), generator=g)
        bound = 2**30
    N = keys.shape[0]
    say(f"[case] from_keys {case} N={N} bound={bound}")
    unq, inv, cnt = torch.unique(keys, return_inverse=True, return_counts=True)
    data = T.ScatterData.from_keys(keys.to(DEV), bound)
    assert torch.equal(data.unq_keys.cpu().long(), unq)
    assert torch.equal(data.unq_inv.cpu().long(), inv)
    assert torch.equal(data.unq_cnts.cpu().reshape(-1), cnt) and data.unq_cnts.dtype == torch.int64
    assert data.num_unq == unq.shape[0] and data.max_cnt == int(cnt.max())
    inv32 = inv.numpy().astype(np.int32)
    pre = orc.presum(cnt.numpy())
    assert np.array_equal(data.preSum.cpu().numpy(), pre)
    perm = data.perm.cpu().numpy() if data.perm is not None else np.arange(N, dtype=np.int32)
    assert np.array_equal(perm, orc.stable_perm(inv32, pre))
    assert np.array_equal(data.seg.cpu().numpy() & 0x7fffffff, inv32[perm])
    if case == "sorted":
        assert data.perm is None
    # the operators give exactly what they give on ScatterData(torch.unique(...))
    feats = torch.randn((N, 16), generator=g).to(DEV)
    ref = T.ScatterData(inv.to(DEV), cnt.to(DEV))
    a, b = T.scatter_max(feats, data), T.scatter_max(feats, ref)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    light = (cnt <= data.heavy_threshold).to(DEV)
    assert torch.equal(T.scatter_mean(feats, data)[light], T.scatter_mean(feats, ref)[light])
    fg = feats.clone().requires_grad_(True)
    T.scatter_mean(fg, data).sum().backward()
    assert torch.equal(fg.grad, (1.0 / cnt.float()).to(DEV)[inv.to(DEV)].unsqueeze(1).expand(-1, 16))


def test_from_points_end_to_end_and_range_check():
    T = tx()
    voxel_size, pc_range = [0.2, 0.2, 0.2], [-75, -75, -2, 75, 75, 4]
    g = torch.Generator().manual_seed(9)
    N = 400_000
    u = torch.rand((N,), generator=g, dtype=torch.float64)
    r = 1.0 / (0.5 - u * (0.5 - 1.0 / 75.0))
    th = torch.rand((N,), generator=g, dtype=torch.float64) * 6.283185307179586
    pts = torch.stack([r * torch.cos(th), r * torch.sin(th),
                       torch.rand((N,), generator=g, dtype=torch.float64) * 6.0 - 2.0], 1).float()
    pts = pts.clamp(min=-74.99, max=74.99)
    pts[:, 2] = pts[:, 2].clamp(-1.99, 3.99)
    say("[case] from_points", N)
    data = T.ScatterData.from_points(pts.to(DEV), voxel_size, pc_range)
    assert data.spatial_size == [750, 750, 30]
    coors = tor.voxelize(pts, voxel_size, pc_range)
    assert torch.equal(data.coors.cpu(), coors)
    keys = tor.flatten_coors(coors, (750, 750, 30))
    unq, inv, cnt = torch.unique(keys, return_inverse=True, return_counts=True)
    assert torch.equal(data.unq_keys.cpu().long(), unq) and torch.equal(data.unq_inv.cpu().long(), inv)
    assert torch.equal(data.unq_cnts.cpu().reshape(-1), cnt)
    feats = torch.randn((N, 32), generator=g)
    mx, arg = T.scatter_max(feats.to(DEV), data)
    wm, wa = orc.scatter_max_first(feats.numpy(), inv.numpy().astype(np.int32), unq.shape[0])
    assert np.array_equal(arg.cpu().numpy(), wa) and np.array_equal(mx.cpu().numpy(), wm)
    bad = pts.clone()
    bad[17, 0] = 80.0
    with pytest.raises(RuntimeError, match="outside the grid"):
        T.ScatterData.from_points(bad.to(DEV), voxel_size, pc_range)
    with pytest.raises(RuntimeError, match="outside the grid"):
        T.ScatterData.from_keys(torch.tensor([1, 5, 9], device=DEV), 9)


def test_ingroup_inds():
    T = tx()
    g = torch.Generator().manual_seed(13)
    for n, ngroups in [(1, 1), (1000, 1), (50_000, 300), (200_000, 150_000)]:
        ids = torch.randint(0, ngroups, (n,), generator=g)
        say(f"[case] ingroup_inds n={n} groups={ngroups}")
        out = T.ingroup_inds(ids.to(DEV))
        assert out.dtype == ids.dtype and out.shape == ids.shape
        assert np.array_equal(out.cpu().numpy(), orc.ingroup_inds(ids.numpy()))
    # the reference's contract: inside each group the ranks are a permutation of 0..cnt-1
    ids = torch.randint(0, 50, (20_000,), generator=g)
    out = T.ingroup_inds(ids.to(DEV)).cpu()
    for gid in range(50):
        r = torch.sort(out[ids == gid]).values
        assert torch.equal(r, torch.arange(r.shape[0]))
    assert T.ingroup_inds(torch.zeros(0, dtype=torch.long, device=DEV)).numel() == 0
    # int32 ids keep their dtype; sorted ids take the identity path
    s = torch.sort(ids).values.int()
    assert T.ingroup_inds(s.to(DEV)).dtype == torch.int32
    assert np.array_equal(T.ingroup_inds(s.to(DEV)).cpu().numpy(), orc.ingroup_inds(s.numpy()).astype(np.int32))
