"""GPU parity of the callers on either side of the scatter path: voxelization, the fused
unique + plan, and ingroup_inds.  Integer work: everything is compared bit-exact, against
the C oracle and against stock torch CPU routines (torch.div floor mode, torch.unique)."""
import sys

import numpy as np
import pytest
import torch

from oracle import c_oracle as orc
from oracle import torch_oracle as tor
from tests import workloads

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


@pytest.mark.parametrize("case", ["lidar", "pillars", "sorted", "few_keys", "single", "sparse_ids"])
def test_from_keys_equals_torch_unique_and_scatter_data(case):
    T = tx()
    g = torch.Generator().manual_seed(7)
    if case == "lidar":       # the voxel keys of the LiDAR-like sweep at its full size
        keys, bound = workloads._lidar_keys(1_000_000, g)
    elif case == "pillars":   # fewer cells than points
        keys, bound = workloads._lidar_keys(1_000_000, g, pillars=True)
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


@pytest.mark.parametrize("seed", range(12))
def test_from_keys_seeded(seed):
    """Key sets nobody chose by hand: grids smaller and far larger than the input (both routes
    of from_keys), dense, clustered and heavy-tailed occupancy, int32 and int64 keys."""
    T = tx()
    g = torch.Generator().manual_seed(4000 + seed)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    N = [1, 7, 300, 5_000, 40_000, 120_000, 250_000, 33_333, 65_536, 65_537, 99_999, 500_000][seed]
    bound = [1, 3, 10_000, 2**31 - 32770, 1_000, 7_000_000, 100_000, 2**20, 70_000, 12_345_678, 64, 20_000_000][seed]
    kind = seed % 3
    if kind == 0:
        keys = torch.randint(0, bound, (N,), generator=g)
    elif kind == 1:      # clustered: a few hundred distinct keys, some of them crowded
        pool = torch.randint(0, bound, (min(bound, ri(1, 300)),), generator=g)
        keys = pool[(torch.rand((N,), generator=g) ** 3 * pool.numel()).long()]
    else:                # mostly distinct, with runs of equal neighbours
        keys = torch.randint(0, bound, (N,), generator=g)
        keys[1::2] = keys[0::2][: keys[1::2].numel()]
    if seed % 2:
        keys = keys.int()
    if seed == 3:        # one past the largest key bound the library takes
        with pytest.raises(RuntimeError):
            T.ScatterData.from_keys(keys.to(DEV), bound + 1)
    say(f"[case] from_keys seeded {seed} N={N} bound={bound} dtype={keys.dtype}")
    unq, inv, cnt = torch.unique(keys.long(), return_inverse=True, return_counts=True)
    data = T.ScatterData.from_keys(keys.to(DEV), bound)
    assert torch.equal(data.unq_keys.cpu().long(), unq)
    assert torch.equal(data.unq_inv.cpu().long(), inv)
    assert torch.equal(data.unq_cnts.cpu().reshape(-1), cnt)
    assert data.num_unq == unq.shape[0] and data.max_cnt == int(cnt.max())
    inv32 = inv.numpy().astype(np.int32)
    pre = orc.presum(cnt.numpy())
    assert np.array_equal(data.preSum.cpu().numpy(), pre)
    perm = data.perm.cpu().numpy() if data.perm is not None else np.arange(N, dtype=np.int32)
    assert np.array_equal(perm, orc.stable_perm(inv32, pre))
    assert np.array_equal(data.seg.cpu().numpy() & 0x7fffffff, inv32[perm])
    # the plan drives the operators as the plan of ScatterData(torch.unique(...)) does
    feats = torch.randn((N, 8), generator=g).to(DEV)
    ref = T.ScatterData(inv.to(DEV), cnt.to(DEV))
    assert (data.num_special, data.num_heavy) == (ref.num_special, ref.num_heavy)
    a, b = T.scatter_max(feats, data), T.scatter_max(feats, ref)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert np.array_equal(T.ingroup_inds(keys.to(DEV)).cpu().numpy(), orc.ingroup_inds(keys.long().numpy()))


def test_from_keys_occupancy_map_and_sort_agree():
    """from_keys numbers the keys with an occupancy map of the grid when the grid is not much
    larger than the input and sorts them otherwise.  The same keys under a small and under a huge
    bound must give the same triple and plan; int32 and int64 keys alike; the last key of a grid
    whose size is not a multiple of 32; keys below zero or at the bound raise on both routes."""
    T = tx()
    g = torch.Generator().manual_seed(17)
    N, bound = 200_000, 1_000_003
    keys = torch.randint(0, bound, (N,), generator=g)
    keys[:64] = torch.arange(bound - 64, bound)          # the top of the grid, up to bound - 1
    keys[64:96] = 0
    unq, inv, cnt = torch.unique(keys, return_inverse=True, return_counts=True)
    results = []
    for kdev, b in ((keys.to(DEV), bound), (keys.int().to(DEV), bound), (keys.to(DEV), 2 ** 30),
                    (keys.int().to(DEV), 2 ** 30)):
        say(f"[case] from_keys routes: dtype={kdev.dtype} bound={b}")
        d = T.ScatterData.from_keys(kdev, b)
        assert torch.equal(d.unq_keys.cpu().long(), unq) and torch.equal(d.unq_inv.cpu().long(), inv)
        assert torch.equal(d.unq_cnts.cpu().reshape(-1), cnt) and d.unq_cnts.dtype == torch.int64
        assert d.unq_inv.dtype == torch.int32 and d.unq_keys.dtype == torch.int32
        assert d.num_unq == unq.shape[0] and d.max_cnt == int(cnt.max())
        results.append(d)
    a = results[0]
    for d in results[1:]:
        assert torch.equal(d.preSum, a.preSum) and torch.equal(d.perm, a.perm) and torch.equal(d.seg, a.seg)
        assert torch.equal(d.slot_of, a.slot_of) and torch.equal(d.heavy_ids, a.heavy_ids)
        assert (d.num_special, d.num_heavy) == (a.num_special, a.num_heavy)
    for bad_key in (-1, bound):
        bad = keys.clone()
        bad[1234] = bad_key
        for b in (bound, 2 ** 30) if bad_key < 0 else (bound,):
            with pytest.raises(RuntimeError, match="outside the grid"):
                T.ScatterData.from_keys(bad.to(DEV), b)
    # an int64 key whose low 32 bits would pass for a valid one: rejected on both routes
    # (occupancy map for a grid near the input's size, sort for a much larger bound)
    for b in (bound, 2 ** 30):
        bad = keys.clone()
        bad[77] = 2 ** 32 + 5
        with pytest.raises(RuntimeError, match="outside the grid"):
            T.ScatterData.from_keys(bad.to(DEV), b)
        bad[77] = -(2 ** 32) + 5
        with pytest.raises(RuntimeError, match="outside the grid"):
            T.ScatterData.from_keys(bad.to(DEV), b)
    # every cell of a small grid occupied, and a grid of one cell
    full = torch.randperm(4096, generator=g).repeat(3)
    d = T.ScatterData.from_keys(full.to(DEV), 4096)
    assert d.num_unq == 4096 and torch.equal(d.unq_keys.cpu().long(), torch.arange(4096))
    assert torch.equal(d.unq_inv.cpu().long(), full) and int(d.unq_cnts.min()) == 3 == d.max_cnt
    d = T.ScatterData.from_keys(torch.zeros(500, dtype=torch.int64, device=DEV), 1)
    assert d.num_unq == 1 and d.max_cnt == 500 and d.perm is None


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
    # (400k elements in 2048 groups: two buckets of 200k rows, slices of two placement rounds)
    for n, ngroups in [(1, 1), (1000, 1), (50_000, 300), (200_000, 150_000), (400_000, 2048)]:
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
    # ids at or beyond the number of elements (not the inverse of a unique) take the pass that
    # reads the largest id first; any shape is ranked as its flattened view
    sparse = torch.randint(0, 40, (5_000,), generator=g) * 1_000_003 % 2_000_000_000
    assert int(sparse.max()) >= 5_000
    assert np.array_equal(T.ingroup_inds(sparse.to(DEV)).cpu().numpy(), orc.ingroup_inds(sparse.numpy()))
    two_d = torch.randint(0, 7, (40, 25), generator=g)
    out = T.ingroup_inds(two_d.to(DEV))
    assert out.shape == two_d.shape
    assert np.array_equal(out.cpu().numpy().reshape(-1), orc.ingroup_inds(two_d.reshape(-1).numpy()))
    with pytest.raises(RuntimeError, match="non-negative"):
        T.ingroup_inds(torch.tensor([3, -1, 2], device=DEV))
    # few groups over many elements (cluster or batch ids): all ids share one bucket of the first
    # attempt, which guesses the number of elements as their bound; the second attempt, with the
    # true bound, must rank them (and quickly: the time is bounded loosely here)
    import time
    many = torch.randint(0, 1000, (1_000_000,), generator=g)
    want = orc.ingroup_inds(many.numpy())
    md = many.to(DEV)
    assert np.array_equal(T.ingroup_inds(md).cpu().numpy(), want)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    T.ingroup_inds(md)
    torch.cuda.synchronize()
    assert time.perf_counter() - t0 < 0.01, "few groups over many elements must not take the slow route"
    # ... and few groups with huge ids: one crowded bucket also under the true bound
    far = many * 1_000_000 + 7
    assert np.array_equal(T.ingroup_inds(far.to(DEV)).cpu().numpy(), want)


# ---------------------------------------------------------- dynamic point pool --

def _boxes_and_points(seed, B, P):
    g = torch.Generator().manual_seed(seed)
    rois = torch.zeros((B, 7))
    rois[:, 0:2] = torch.rand((B, 2), generator=g) * 100 - 50
    rois[:, 2] = torch.rand((B,), generator=g) * 2 - 1
    rois[:, 3:6] = torch.rand((B, 3), generator=g) * 4 + 1
    rois[:, 6] = torch.rand((B,), generator=g) * 6.283 - 3.1415
    pts = torch.zeros((P, 3))
    pts[:, 0:2] = torch.rand((P, 2), generator=g) * 120 - 60
    pts[:, 2] = torch.rand((P,), generator=g) * 6 - 2
    per = P // (2 * B)
    for b in range(B):
        pts[b * per:(b + 1) * per, 0:2] = rois[b, 0:2] + (torch.rand((per, 2), generator=g) - 0.5) * 7
        pts[b * per:(b + 1) * per, 2] = rois[b, 2] + torch.rand((per,), generator=g) * rois[b, 5]
    return rois, pts[torch.randperm(P, generator=g)]


@pytest.mark.parametrize("B,P,cap,max_all,extra", [
    (40, 60_000, 512, 50_000, [0.0, 0.0, 0.0]),      # the reference test's call: dynamic_point_pool(boxes, pc, [0,0,0], 512)
    (40, 60_000, 100_000, 1_000_000, [0.5, 0.5, 0.3]),
    (7, 1_000, 16, 60, [1.0, 0.2, 0.4]),             # both caps bite
    (300, 200_000, 64, 50_000, [0.4, 0.4, 0.2]),
    (1, 300, 512, 50_000, [0.0, 0.0, 0.0]),
])
def test_dynamic_point_pool(B, P, cap, max_all, extra):
    """Bit-exact against the oracle: same hits, same (box, point) order, same 13 floats
    (both sides take the rotation terms from double-precision cos/sin and keep products
    and sums as separate fp32 roundings)."""
    T = tx()
    rois, pts = _boxes_and_points(B * 7 + P, B, P)
    say(f"[case] dynamic_point_pool B={B} P={P} cap={cap} max_all={max_all}")
    idx, roi, feats = T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), extra, cap, max_all)
    wi, wr, wf = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, cap, max_all)
    assert idx.dtype == torch.int64 and roi.dtype == torch.int64 and feats.shape[1] == 13
    assert wi.shape[0] > 0
    assert np.array_equal(idx.cpu().numpy(), wi) and np.array_equal(roi.cpu().numpy(), wr)
    assert np.array_equal(feats.cpu().numpy().view(np.uint32), wf.view(np.uint32))
    assert idx.shape[0] <= max_all and torch.bincount(roi).max().item() <= cap


@pytest.mark.parametrize("cap,max_all", [(10 ** 6, 10 ** 6), (5, 300)])
def test_dynamic_point_pool_mixed_batches(cap, max_all):
    """Boxes and points of several samples in one call (the reference extension's
    dynamic_point_pool_mixed_gpu): bit-exact against the oracle, never a pair across
    samples, and with every index in one sample the same as the plain op."""
    T = tx()
    rois, pts = _boxes_and_points(123, 60, 50_000)
    g = torch.Generator().manual_seed(9)
    rb = torch.randint(0, 4, (60,), generator=g)
    pb = torch.randint(0, 4, (50_000,), generator=g)
    extra = [0.4, 0.4, 0.2]
    say(f"[case] dynamic_point_pool mixed cap={cap} max_all={max_all}")
    idx, roi, feats = T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), extra, cap, max_all,
                                           rois_batch=rb.to(DEV), pts_batch=pb.to(DEV))
    wi, wr, wf = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, cap, max_all, rb.numpy(), pb.numpy())
    assert wi.shape[0] > 50
    assert np.array_equal(idx.cpu().numpy(), wi) and np.array_equal(roi.cpu().numpy(), wr)
    assert np.array_equal(feats.cpu().numpy().view(np.uint32), wf.view(np.uint32))
    assert torch.equal(rb[roi.cpu()], pb[idx.cpu()])
    zr, zp = torch.zeros_like(rb).to(DEV), torch.zeros_like(pb).to(DEV)
    a = T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), extra, cap, max_all, rois_batch=zr, pts_batch=zp)
    b = T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), extra, cap, max_all)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    with pytest.raises(AssertionError):
        T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), extra, cap, max_all, rois_batch=zr)


def test_dynamic_point_pool_corner_points():
    """Points placed a hair inside and outside the corners and edge midpoints of the
    rotated (enlarged) boxes: the farthest places from a box centre that still count,
    i.e. where a too tight early reject would lose hits.  Includes shrinking margins."""
    T = tx()
    g = torch.Generator().manual_seed(17)
    B = 64
    rois = torch.zeros((B, 7))
    rois[:, 0:2] = torch.rand((B, 2), generator=g) * 60 - 30
    rois[:, 3:6] = torch.rand((B, 3), generator=g) * 6 + 0.5
    rois[:, 6] = torch.rand((B,), generator=g) * 6.283 - 3.1415
    for extra in ([0.0, 0.0, 0.0], [0.6, 0.4, 0.2], [-0.2, -0.1, 0.0]):
        ex = torch.tensor(extra)
        pts = []
        for b in range(B):
            cx, cy, zb, w, l, h, rz = rois[b].tolist()
            rot = rz + np.pi / 2
            c, s_ = np.cos(rot), np.sin(rot)
            for dims in ((l, w), (l + extra[1], w + extra[0])):
                for ux, uy in ((1, 1), (1, -1), (-1, 1), (-1, -1), (1, 0), (0, 1), (-1, 0), (0, -1)):
                    for scale in (1 - 1e-6, 1 - 1e-4, 1 + 1e-6, 1 + 1e-4):
                        lx, ly = ux * dims[0] / 2 * scale, uy * dims[1] / 2 * scale
                        # inverse of the local transform: world = centre + R^T (lx, ly)
                        pts.append([cx + lx * c + ly * s_, cy - lx * s_ + ly * c, zb + h / 2])
        pts = torch.tensor(pts, dtype=torch.float32)
        say(f"[case] dynamic_point_pool corners extra={extra} P={pts.shape[0]}")
        idx, roi, feats = T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), extra, 100_000, 1_000_000)
        wi, wr, wf = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, 100_000, 1_000_000)
        assert wi.shape[0] > B * 8     # the inner copies are hits
        assert np.array_equal(idx.cpu().numpy(), wi) and np.array_equal(roi.cpu().numpy(), wr)
        assert np.array_equal(feats.cpu().numpy().view(np.uint32), wf.view(np.uint32))


def test_dynamic_point_pool_no_hits_returns_the_reference_placeholder():
    T = tx()
    rois = torch.tensor([[1000.0, 1000.0, 0.0, 2.0, 4.0, 1.5, 0.3]], device=DEV)
    pts = torch.rand((500, 3), device=DEV)
    idx, roi, feats = T.dynamic_point_pool(rois, pts, [0, 0, 0], 512)
    assert idx.tolist() == [-1] and roi.tolist() == [-1] and feats.shape == (1, 13) and (feats == 0).all()
    with pytest.raises(RuntimeError):
        T.dynamic_point_pool(rois.cpu(), pts, [0, 0, 0], 512)


def test_dynamic_point_pool_feeds_the_scatter_path():
    """The pairs this op emits are what FSD-style code then reduces per RoI: unique the
    roi ids and scatter the per-pair numbers (here through ScatterData.from_keys)."""
    T = tx()
    rois, pts = _boxes_and_points(99, 50, 80_000)
    idx, roi, feats = T.dynamic_point_pool(rois.to(DEV), pts.to(DEV), [0.3, 0.3, 0.2], 512, 200_000)
    data = T.ScatterData.from_keys(roi, 50)
    assert data.is_sorted                               # (box, point) order: no permutation needed
    mx, arg = T.scatter_max(feats.contiguous(), data)
    unq, inv = torch.unique(roi.cpu(), return_inverse=True)
    # grouped rows: the default reports the reference kernel's winner among equal maxima
    assert data.max_tie_rule == "reference"
    wm, wa = orc.scatter_max_reforder(feats.cpu().numpy(), inv.numpy().astype(np.int32), unq.shape[0])
    assert np.array_equal(arg.cpu().numpy(), wa) and np.array_equal(mx.cpu().numpy(), wm)
    d1 = T.ScatterData.from_keys(roi, 50, max_tie_rule="first")
    mx, arg = T.scatter_max(feats.contiguous(), d1)
    wm, wa = orc.scatter_max_first(feats.cpu().numpy(), inv.numpy().astype(np.int32), unq.shape[0])
    assert np.array_equal(arg.cpu().numpy(), wa) and np.array_equal(mx.cpu().numpy(), wm)


# -------------------------------------------------------------------- grid hash --

def test_grid_hash_build_and_probe_against_oracle():
    T = tx()
    rng = np.random.default_rng(17)
    for n in (1, 2, 1000, 1024, 4097, 300_000):
        keys = rng.choice(2 ** 30, size=n, replace=False).astype(np.int32)
        vals = rng.permutation(n).astype(np.int32)
        say(f"[case] grid_hash n={n}")
        table = T.grid_hash_build(torch.from_numpy(keys).to(DEV), torch.from_numpy(vals).to(DEV))
        assert table.dtype == torch.int32 and table.shape == (orc.grid_hash_build(keys, vals).shape[0], 2)
        tb = table.cpu().numpy()
        stored = tb[tb[:, 0] != -1]
        assert stored.shape[0] == n and (tb[tb[:, 0] == -1, 1] == -1).all()
        assert set(map(tuple, stored.tolist())) == set(zip(keys.tolist(), vals.tolist()))
        # absent keys too; few of them when the table is completely full (n a power of two),
        # where an absent key has to visit every slot
        n_absent = 8 if (n & (n - 1)) == 0 else n + 5
        queries = np.concatenate([keys, rng.integers(0, 2 ** 30, size=n_absent).astype(np.int32)])
        out = T.grid_hash_probe(torch.from_numpy(queries).to(DEV), table).cpu().numpy()
        # the table built in a different insertion order answers every query identically
        assert np.array_equal(out, orc.grid_hash_probe(queries, orc.grid_hash_build(keys, vals)))
        # and the oracle's probe reads the GPU-built table the same way (open-addressing invariant)
        assert np.array_equal(orc.grid_hash_probe(queries, tb), out)


def test_grid_hash_absent_keys():
    """Keys that are not in the table.  With free slots in the table (N not a power of two)
    the probe of an absent key stops at the first empty slot of its sequence, so 200k of them
    cost about as much as 200k present ones.  On a completely full table (N a power of two,
    the table has exactly N slots as in the reference, grid_hash.cpp:28-37) there is no empty
    slot and an absent key is looked for in all N slots -- the reference does that for every
    absent key on any table (functions.cuh:54-63) -- so only 32 are asked for here:
    32 x 262,144 slot reads."""
    T = tx()
    rng = np.random.default_rng(23)
    for n, n_absent in ((300_000, 200_000), (1 << 18, 32)):
        keys = rng.choice(2 ** 30, size=n, replace=False).astype(np.int32)
        vals = rng.permutation(n).astype(np.int32)
        absent = np.setdiff1d(rng.integers(0, 2 ** 30, size=n_absent + 64).astype(np.int32), keys)[:n_absent]
        queries = np.concatenate([absent, keys[:1000]])
        want = np.concatenate([np.full(absent.shape[0], -1, np.int32), vals[:1000]])
        table = T.grid_hash_build(torch.from_numpy(keys).to(DEV), torch.from_numpy(vals).to(DEV))
        free = int((table[:, 0] == -1).sum())
        say(f"[case] grid_hash absent keys n={n} table={table.shape[0]} free={free} absent={absent.shape[0]}")
        assert (free == 0) == ((n & (n - 1)) == 0)
        out = T.grid_hash_probe(torch.from_numpy(queries).to(DEV), table).cpu().numpy()
        assert np.array_equal(out, want)


def test_grid_hash_class_follows_the_reference_test():
    """test/test_grid_hash.py:17-44 (smaller, seeded): probe(unique rows) == arange, the
    table maps its own keys to their values, and the mapping is stable under re-indexing."""
    T = tx()
    import random
    random.seed(2)
    g = torch.Generator().manual_seed(0)
    for _ in range(6):
        all_size = random.randint(1, 200000)
        high = random.randint(10, 1024)
        coors = torch.randint(0, high, (all_size, 3), generator=g).int()
        unq_coors = torch.unique(coors, dim=0)
        hasher = T.GridHash(coors.to(DEV), debug=True)
        out = hasher.probe(unq_coors.to(DEV))
        assert (out.cpu() == torch.arange(len(out))).all()
        valid_values = hasher.valid_table[:, 1]
        assert (hasher.probe(hasher.table[hasher.valid_mask, 0]) == valid_values).all()
        index = torch.randint(0, max(all_size - 1, 1), (random.randint(1, 200000),), generator=g)
        values_1 = hasher.probe(coors.to(DEV))
        values_2 = hasher.probe(coors[index].to(DEV))
        assert (values_1[index.to(DEV)] == values_2).all()
    # flat keys
    keys = torch.randint(0, 5000, (20000,), generator=g)
    h = T.GridHash(keys.to(DEV))
    unq, inv = torch.unique(keys, return_inverse=True)
    assert torch.equal(h.probe(keys.to(DEV)).cpu().long(), inv)


# ------------------------------- the reference's extension-module names and signatures --
#
# The reference's wrappers bind three more modules by name: `import ingroup_indices`
# (operator_py/ingroup_inds_op.py:4), `import dynamic_point_pool_ext`
# (operator_py/dynamic_point_pool_op.py:7), `import grid_hash_ext` (operator_py/grid_hash.py:2).
# Each test below does what the body of the wrapper's forward() does, with
# caller-allocated outputs where the reference has them, and checks against the oracle.

def test_reference_module_ingroup_indices_forward_in_place():
    tx()
    import ingroup_indices
    g = torch.Generator().manual_seed(31)
    for n, ngroups in [(1, 1), (70_000, 900), (300_000, 200_000)]:
        group_inds = torch.randint(0, ngroups, (n,), generator=g).to(DEV)
        say(f"[case] ingroup_indices.forward n={n} groups={ngroups}")
        out_inds = torch.zeros_like(group_inds) - 1                  # ingroup_inds_op.py:15
        assert ingroup_indices.forward(group_inds, out_inds) is None  # :17
        assert out_inds.dtype == torch.int64
        assert np.array_equal(out_inds.cpu().numpy(), orc.ingroup_inds(group_inds.cpu().numpy()))
    with pytest.raises(RuntimeError, match="int64"):
        ingroup_indices.forward(group_inds, torch.zeros(n, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="one entry per element"):
        ingroup_indices.forward(group_inds, torch.zeros(n + 1, dtype=torch.int64, device=DEV))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ingroup_indices.forward(group_inds.cpu(), torch.zeros(n, dtype=torch.int64))


@pytest.mark.parametrize("B,P,cap,max_all,extra", [
    (40, 60_000, 512, 50_000, [0.0, 0.0, 0.0]),
    (7, 1_000, 16, 60, [1.0, 0.2, 0.4]),             # both caps bite
])
def test_reference_module_dynamic_point_pool_ext_forward_in_place(B, P, cap, max_all, extra):
    tx()
    import dynamic_point_pool_ext
    rois, pts = _boxes_and_points(B * 11 + P, B, P)
    rois, pts = rois.to(DEV), pts.to(DEV)
    say(f"[case] dynamic_point_pool_ext.forward B={B} P={P} cap={cap} max_all={max_all}")
    out_pts_idx = -1 * pts.new_ones(max_all, dtype=torch.long)          # dynamic_point_pool_op.py:33-35
    out_roi_idx = -1 * pts.new_ones(max_all, dtype=torch.long)
    out_pts_feats = pts.new_zeros(max_all, 13, dtype=torch.float)
    assert dynamic_point_pool_ext.forward(rois, pts, extra, cap, out_pts_idx, out_roi_idx, out_pts_feats) is None
    valid_mask = out_pts_idx >= 0                                        # :40
    wi, wr, wf = orc.dynamic_point_pool(rois.cpu().numpy(), pts.cpu().numpy(), extra, cap, max_all)
    M = wi.shape[0]
    assert M > 0 and int(valid_mask.sum()) == M and bool(valid_mask[:M].all())   # compact, from index 0
    assert np.array_equal(out_pts_idx[valid_mask].cpu().numpy(), wi)
    assert np.array_equal(out_roi_idx[valid_mask].cpu().numpy(), wr)
    assert np.array_equal(out_pts_feats[valid_mask].cpu().numpy().view(np.uint32), wf.view(np.uint32))
    # what lies behind the last entry keeps the caller's fill
    assert (out_roi_idx[M:] == -1).all() and (out_pts_feats[M:] == 0).all()
    with pytest.raises(RuntimeError, match="13"):
        dynamic_point_pool_ext.forward(rois, pts, extra, cap, out_pts_idx, out_roi_idx,
                                       pts.new_zeros(max_all, 12, dtype=torch.float))


def test_reference_module_dynamic_point_pool_ext_mixed_in_place():
    tx()
    import dynamic_point_pool_ext
    rois, pts = _boxes_and_points(321, 60, 50_000)
    g = torch.Generator().manual_seed(5)
    rb = torch.randint(0, 3, (60,), generator=g).int()
    pb = torch.randint(0, 3, (50_000,), generator=g).int()
    extra, cap, max_all = [0.4, 0.4, 0.2], 64, 20_000
    oi = torch.full((max_all,), -1, dtype=torch.long, device=DEV)
    orr = torch.full((max_all,), -1, dtype=torch.long, device=DEV)
    of = torch.zeros((max_all, 13), device=DEV)
    say("[case] dynamic_point_pool_ext.dynamic_point_pool_mixed_gpu")
    dynamic_point_pool_ext.dynamic_point_pool_mixed_gpu(rois.to(DEV), rb.to(DEV), pts.to(DEV), pb.to(DEV), extra, cap,
                                                        oi, orr, of)
    wi, wr, wf = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, cap, max_all, rb.numpy(), pb.numpy())
    M = wi.shape[0]
    assert M > 50 and int((oi >= 0).sum()) == M
    assert np.array_equal(oi[:M].cpu().numpy(), wi) and np.array_equal(orr[:M].cpu().numpy(), wr)
    assert np.array_equal(of[:M].cpu().numpy().view(np.uint32), wf.view(np.uint32))


def test_reference_module_grid_hash_ext():
    tx()
    import grid_hash_ext
    rng = np.random.default_rng(29)
    n = 50_000
    keys = rng.choice(2 ** 30, size=n, replace=False).astype(np.int32)
    vals = rng.permutation(n).astype(np.int32)
    say(f"[case] grid_hash_ext n={n}")
    table = grid_hash_ext.build_table(torch.from_numpy(keys).to(DEV), torch.from_numpy(vals).to(DEV))  # grid_hash.py:31
    assert table.dtype == torch.int32 and tuple(table.shape) == (65536, 2)
    queries = np.concatenate([keys[::3], rng.integers(0, 2 ** 30, size=999).astype(np.int32)])
    out = grid_hash_ext.probe_table(torch.from_numpy(queries).to(DEV), table)                           # :44
    assert np.array_equal(out.cpu().numpy(), orc.grid_hash_probe(queries, orc.grid_hash_build(keys, vals)))
