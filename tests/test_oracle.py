"""Pins the CPU oracle (oracle/scatter_oracle.c) without the reference's code:
known-answer data of the reference's own test, hand-worked fixtures, brute force
on tiny inputs, a library routine (torch index_add / scatter_reduce in fp64) and
invariants.  Each check is chosen so that a dropped term, a wrong index or a
swapped operand fails it."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as orc
from oracle import torch_oracle as tor
from tests import workloads


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bits_equal(a, b):
    """float32 equality on the bit pattern, NaNs compared as NaNs"""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    assert a.shape == b.shape
    both_nan = np.isnan(a) & np.isnan(b)
    assert np.array_equal(bits(a)[~both_nan], bits(b)[~both_nan])


# ---------------------------------------------------------------- helpers ----

def test_up_2n_and_block_width():
    # scatter_kernel.cu:14-24 : next power of two, 1 -> 1
    for n in [1, 2, 3, 4, 5, 31, 32, 33, 1023, 1024, 1025, 4996]:
        want = 1 if n == 1 else 1 << (n - 1).bit_length()
        assert orc.up_2n(n) == want
    assert orc.block_width(1) == 32
    assert orc.block_width(20) == 32
    assert orc.block_width(33) == 64
    assert orc.block_width(1000) == 1024
    assert orc.block_width(4996) == 1024


def test_get_presum_ref_is_cumsum_of_bincount_on_sorted_input():
    rng = np.random.default_rng(3)
    cnt = rng.integers(1, 40, size=200)
    inv = np.repeat(np.arange(200), cnt).astype(np.int32)
    want = np.concatenate([[0], np.cumsum(cnt)]).astype(np.int32)
    assert np.array_equal(orc.get_presum_ref(inv), want)
    assert np.array_equal(orc.presum(orc.counts(inv, 200)), want)


def test_counts_rejects_out_of_range():
    with pytest.raises(ValueError):
        orc.counts(np.array([0, 3], dtype=np.int32), 3)


def test_stable_perm_matches_stable_argsort():
    rng = np.random.default_rng(4)
    inv = rng.integers(0, 50, size=5000).astype(np.int32)
    pre = orc.presum(orc.counts(inv, 50))
    assert np.array_equal(orc.stable_perm(inv, pre), np.argsort(inv, kind="stable").astype(np.int32))


# ------------------------------------- the reference's own known-answer data --

def _reference_groups(reference_counts, num_group, channel):
    counts = np.array(reference_counts["counts"][:num_group], dtype=np.int64)
    g = torch.Generator().manual_seed(11)
    cols, invs, argpos = [], [], []
    start = 0
    for gid, c in enumerate(counts.tolist()):
        p = torch.randperm(c, generator=g)
        cols.append(p.to(torch.float32))
        invs.append(np.full(c, gid, dtype=np.int32))
        argpos.append(start + int(torch.argmax(p)))
        start += c
    feats = torch.cat(cols).unsqueeze(1).expand(-1, channel).contiguous().numpy()
    return feats, np.concatenate(invs), counts, np.array(argpos, dtype=np.int32)


def test_fixture_counts_match_numpy_recipe(reference_counts):
    np.random.seed(0)
    again = [int(np.random.randint(100, 5000)) for _ in range(500)]
    assert again == reference_counts["counts"]
    assert reference_counts["num_total"] == 1229413 and reference_counts["max_cnt"] == 4996


def test_reference_test_closed_forms(reference_counts):
    """test/test_scatter.py:17-23: each group is a permutation of 0..n-1 in every
    channel, so sum = n(n-1)/2 (< 2^24, exact in fp32 in any order), mean = (n-1)/2,
    max = n-1 at the position of n-1."""
    C = 3
    feats, inv, counts, argpos = _reference_groups(reference_counts, 80, C)
    U = counts.shape[0]
    n = counts.astype(np.float64)
    want_sum = np.repeat((n * (n - 1) / 2)[:, None], C, 1)
    want_mean = np.repeat(((n - 1) / 2)[:, None], C, 1)
    want_max = np.repeat((n - 1)[:, None], C, 1)
    want_arg = np.repeat(argpos[:, None], C, 1)
    pre = orc.get_presum_ref(inv)
    max_cnt = int(counts.max())
    assert max_cnt > 1024  # the multi-iteration strided path of the reference is exercised

    s = orc.scatter_sum_ref(feats, pre, max_cnt)
    assert np.array_equal(s.astype(np.float64), want_sum)
    assert np.array_equal(orc.mean_from_sum(s, counts).astype(np.float64), want_mean)
    m, a = orc.scatter_max_ref(feats, pre, max_cnt)
    assert np.array_equal(m.astype(np.float64), want_max)
    assert np.array_equal(a, want_arg)

    assert np.array_equal(orc.scatter_sum_f64(feats, inv, U), want_sum)
    m2, a2 = orc.scatter_max_first(feats, inv, U)
    assert np.array_equal(m2.astype(np.float64), want_max)
    assert np.array_equal(a2, want_arg)


# ----------------------------------------------------- hand-worked fixtures --

def test_hand_cases(hand_cases):
    for c in hand_cases:
        inv, feats = c["inv"], c["feats"]
        U = int(inv.max()) + 1
        cnt = orc.counts(inv, U)
        m, a = orc.scatter_max_first(feats, inv, U)
        assert_bits_equal(m, c["max"]), c["name"]
        assert np.array_equal(a, c["arg"]), c["name"]
        if "arg_ref" in c:   # grouped rows: what the reference kernel itself reports
            assert np.all(np.diff(inv) >= 0)
            mr, ar = orc.scatter_max_ref(feats, orc.presum(cnt), int(cnt.max()))
            assert np.array_equal(ar, c["arg_ref"]), c["name"]
            assert_bits_equal(mr, c.get("max_ref", c["max"])), c["name"]
        if "sum" in c:
            s64 = orc.scatter_sum_f64(feats, inv, U)
            np.testing.assert_allclose(s64, c["sum"], rtol=1e-6, atol=0)
            s32 = orc.scatter_sum_reforder(feats, inv, U)
            np.testing.assert_allclose(s32, c["sum"], rtol=1e-6, atol=0)
            np.testing.assert_allclose(orc.mean_from_sum(s32, cnt), c["mean"], rtol=1e-6)
        if "g" in c:
            g = c["g"]
            assert np.array_equal(orc.sum_backward(g, inv), c["sum_bwd"])
            np.testing.assert_allclose(orc.mean_backward(g, cnt, inv), c["mean_bwd"], rtol=1e-6)
            assert np.array_equal(orc.max_backward(g, a, inv.shape[0]), c["max_bwd"])


def test_reference_init_pair_for_all_minus_inf_group():
    """scatter_kernel.cu:139-148: the running max starts at -FLT_MAX with '>=', so a
    group holding only -inf keeps (-FLT_MAX, -1) in the reference.  The spec oracle
    treats -inf as an ordinary value (first row wins); this test records both."""
    feats = np.array([[-np.inf], [-np.inf]], dtype=np.float32)
    pre = np.array([0, 2], dtype=np.int32)
    m, a = orc.scatter_max_ref(feats, pre, 2)
    assert m[0, 0] == -np.finfo(np.float32).max and a[0, 0] == -1
    m, a = orc.scatter_max_first(feats, np.zeros(2, np.int32), 1)
    assert m[0, 0] == -np.inf and a[0, 0] == 0
    # a voxel of NaNs only: both keep the initial pair
    feats = np.array([[np.nan], [np.nan]], dtype=np.float32)
    m, a = orc.scatter_max_ref(feats, pre, 2)
    assert m[0, 0] == -np.finfo(np.float32).max and a[0, 0] == -1
    m, a = orc.scatter_max_first(feats, np.zeros(2, np.int32), 1)
    assert m[0, 0] == -np.finfo(np.float32).max and a[0, 0] == -1


def test_reference_tie_rule_large_group_hand_worked():
    """Worked from scatter_kernel.cu:146-152 ('>=' inside a thread: the later row of
    a thread wins) and :41-83 (strict '>' across lanes: the lower lane wins).
    2050 equal values with block width 1024: thread 0 sees rows 0, 1024, 2048 and
    keeps 2048; every other lane ties with it and loses, so arg = 2048.  With at most
    1024 rows each thread holds one row and lane 0 wins: arg = first row."""
    big = np.full((2050, 1), 3.5, dtype=np.float32)
    m, a = orc.scatter_max_ref(big, np.array([0, 2050], np.int32), 2050)
    assert m[0, 0] == 3.5 and a[0, 0] == 2048
    small = np.full((1000, 1), 3.5, dtype=np.float32)
    m, a = orc.scatter_max_ref(small, np.array([0, 1000], np.int32), 1000)
    assert a[0, 0] == 0
    # the maximum in a non-zero residue: rows 5 and 1029 hold the max -> thread 5 keeps 1029
    x = np.zeros((2050, 1), dtype=np.float32)
    x[5] = x[1029] = x[7] = 9.0
    m, a = orc.scatter_max_ref(x, np.array([0, 2050], np.int32), 2050)
    assert m[0, 0] == 9.0 and a[0, 0] == 1029
    _, a1 = orc.scatter_max_first(x, np.zeros(2050, np.int32), 1)
    assert a1[0, 0] == 5


def _bitrev(x, nbits):
    r = 0
    for b in range(nbits):
        r |= ((x >> b) & 1) << (nbits - 1 - b)
    return r


def _reference_tie_winner(vals, B):
    """Closed form of the reference's arg-max among equal maxima, derived from the
    shuffle tree on paper: a thread keeps the LAST maximal row of its residue class
    ('>=' at scatter_kernel.cu:148); a shfl_down tree with strict '>' lets lane 0 end
    with the candidate whose lane index is smallest in BIT-REVERSED order (step 16
    ranks lane 0 before 16, step 8 ranks {0,16} before {8,24}, ...), first over the
    5 lane bits inside a warp, then over the warp index bits across warps."""
    n = len(vals)
    vmax = max(vals)
    nvw = B // 32
    wbits = nvw.bit_length() - 1
    best = None
    for tid in range(min(B, n)):
        rows = [r for r in range(tid, n, B) if vals[r] == vmax]
        if not rows:
            continue
        key = (_bitrev(tid // 32, wbits), _bitrev(tid % 32, 5))
        if best is None or key < best[0]:
            best = (key, rows[-1])
    return best[1]


def test_reference_tie_rule_is_bit_reversed_lane_order():
    # hand-worked: 17 rows, width 32; rows 8 and 16 tie at the max.  Step 16 moves
    # row 16 into lane 0 (4 > 3); at step 8 lane 8 offers an equal 4 and loses.
    x = np.full((17, 1), 3.0, dtype=np.float32)
    x[8] = x[16] = 4.0
    m, a = orc.scatter_max_ref(x, np.array([0, 17], np.int32), 17)
    assert m[0, 0] == 4.0 and a[0, 0] == 16
    _, a1 = orc.scatter_max_first(x, np.zeros(17, np.int32), 1)
    assert a1[0, 0] == 8
    # lane-exact emulation == closed form, over random tie-heavy groups and widths
    rng = np.random.default_rng(12)
    for n, max_cnt in [(5, 5), (31, 31), (32, 40), (33, 64), (100, 100), (700, 700),
                       (1024, 1024), (1500, 1500), (3000, 4996)]:
        for _ in range(6):
            vals = rng.integers(0, 3, size=n).astype(np.float32)
            _, a = orc.scatter_max_ref(vals[:, None].copy(), np.array([0, n], np.int32), max_cnt)
            assert a[0, 0] == _reference_tie_winner(vals.tolist(), orc.block_width(max_cnt)), (n, max_cnt)


# ------------------------------------------------------------- brute force ---

def _brute(feats, inv, U):
    N, C = feats.shape
    s = [[0.0] * C for _ in range(U)]
    m = [[None] * C for _ in range(U)]
    a = [[-1] * C for _ in range(U)]
    for i in range(N):
        u = int(inv[i])
        for c in range(C):
            v = float(feats[i, c])
            s[u][c] += v
            if m[u][c] is None or v > m[u][c]:
                m[u][c] = v
                a[u][c] = i
    return np.array(s), np.array(m, dtype=np.float64), np.array(a, dtype=np.int32)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_brute_force_tiny(seed):
    rng = np.random.default_rng(seed)
    N, C, U = 64, 3, 7
    inv = np.concatenate([np.arange(U), rng.integers(0, U, size=N - U)]).astype(np.int32)
    rng.shuffle(inv)
    feats = rng.integers(-4, 5, size=(N, C)).astype(np.float32)  # small ints: many ties, exact sums
    s, m, a = _brute(feats, inv, U)
    assert np.array_equal(orc.scatter_sum_f64(feats, inv, U), s)
    assert np.array_equal(orc.scatter_sum_reforder(feats, inv, U).astype(np.float64), s)
    mo, ao = orc.scatter_max_first(feats, inv, U)
    assert np.array_equal(mo.astype(np.float64), m) and np.array_equal(ao, a)
    # the reference's lane-tree picks a different row among equal maxima (see
    # test_reference_tie_rule_is_bit_reversed_lane_order) but the same value, and
    # the same row wherever the maximum is unique
    mr, ar = orc.scatter_max_reforder(feats, inv, U)
    assert np.array_equal(mr.astype(np.float64), m)
    n_at_max = np.zeros((U, C), dtype=np.int64)
    np.add.at(n_at_max, inv, (feats == m[inv]).astype(np.int64))
    assert np.array_equal(ar[n_at_max == 1], a[n_at_max == 1])
    assert np.array_equal(np.take_along_axis(feats, ar.astype(np.int64), 0), mr)


# -------------------------------------------------- library routine + bounds --

def test_against_torch_library_routines():
    w = workloads.uniform_box(N=20000, C=8, seed=5)
    f, inv, cnt = w.feats.numpy(), w.unq_inv.numpy().astype(np.int32), w.unq_cnts.numpy()
    U = w.U
    s64 = orc.scatter_sum_f64(f, inv, U)
    t64 = tor.scatter_sum(w.feats, w.unq_inv, U, acc_dtype=torch.float64).numpy()
    np.testing.assert_allclose(s64, t64, rtol=1e-12, atol=1e-12)
    # fp32 in the reference's order stays within the textbook bound n*eps*sum|x|
    s32 = orc.scatter_sum_reforder(f, inv, U)
    sabs = orc.scatter_sum_f64(np.abs(f), inv, U)
    bound = cnt[:, None] * np.finfo(np.float32).eps * sabs + 1e-30
    assert np.all(np.abs(s32 - s64) <= bound)
    m, a = orc.scatter_max_first(f, inv, U)
    tm, ta = tor.scatter_max(w.feats, w.unq_inv, U)
    assert_bits_equal(m, tm.numpy())
    assert np.array_equal(a, ta.numpy())
    mr, ar = orc.scatter_max_reforder(f, inv, U)  # N(0,1) data: no ties, rules agree
    assert_bits_equal(mr, m)
    assert np.array_equal(ar, a)
    mean = orc.mean_from_sum(s32, cnt)
    tmean = (torch.from_numpy(s32) / w.unq_cnts.reshape(-1, 1)).numpy()  # scatter_op.py:69
    assert_bits_equal(mean, tmean)


def test_ties_against_torch_amin_construction():
    rng = np.random.default_rng(9)
    N, C, U = 30000, 4, 300
    inv = rng.integers(0, U, size=N).astype(np.int32)
    inv[:U] = np.arange(U)
    feats = rng.integers(0, 6, size=(N, C)).astype(np.float32)  # heavy ties
    m, a = orc.scatter_max_first(feats, inv, U)
    tm, ta = tor.scatter_max(torch.from_numpy(feats), torch.from_numpy(inv), U)
    assert np.array_equal(m, tm.numpy()) and np.array_equal(a, ta.numpy())
    # invariants of an arg-max
    assert np.array_equal(inv[a], np.repeat(np.arange(U)[:, None], C, 1))
    assert np.array_equal(np.take_along_axis(feats, a.astype(np.int64), 0), m)


def test_invariants_ones_and_total():
    w = workloads.zipf_contention(N=50000, C=4, num_ids=64, seed=6)
    f, inv, cnt = w.feats.numpy(), w.unq_inv.numpy().astype(np.int32), w.unq_cnts.numpy()
    ones = np.ones_like(f)
    # all-ones features give the counts exactly (the check in the reference's
    # commented-out main, scatter_kernel.cu:254-259)
    assert np.array_equal(orc.scatter_sum_reforder(ones, inv, w.U), np.repeat(cnt[:, None], 4, 1))
    s = orc.scatter_sum_f64(f, inv, w.U)
    np.testing.assert_allclose(s.sum(0), f.astype(np.float64).sum(0), rtol=1e-10)
    # permuting the points does not change the spec result
    p = np.random.default_rng(1).permutation(f.shape[0])
    np.testing.assert_allclose(orc.scatter_sum_f64(f[p], inv[p], w.U), s, rtol=1e-10, atol=1e-9)


# ---------------------------------------------------------------- backward ---

def test_backward_against_torch_ops_and_autograd():
    w = workloads.uniform_box(N=5000, C=6, seed=8)
    inv = w.unq_inv.numpy().astype(np.int32)
    cnt = w.unq_cnts.numpy()
    g = workloads.upstream_grad(w.U, w.C, 108)
    assert np.array_equal(orc.sum_backward(g.numpy(), inv), tor.sum_backward(g, w.unq_inv).numpy())
    assert_bits_equal(orc.mean_backward(g.numpy(), cnt, inv),
                      tor.mean_backward(g, w.unq_cnts, w.unq_inv).numpy())
    _, a = orc.scatter_max_first(w.feats.numpy(), inv, w.U)
    assert np.array_equal(orc.max_backward(g.numpy(), a, w.N),
                          tor.max_backward(g, torch.from_numpy(a), w.N).numpy())
    # autograd of the textbook formulation gives the same gradients
    x = w.feats.double().requires_grad_(True)
    idx = w.unq_inv.unsqueeze(1).expand(-1, w.C)
    torch.zeros(w.U, w.C, dtype=torch.float64).scatter_reduce(0, idx, x, "sum", include_self=False) \
        .backward(g.double())
    assert np.array_equal(x.grad.float().numpy(), orc.sum_backward(g.numpy(), inv))
    x.grad = None
    torch.zeros(w.U, w.C, dtype=torch.float64).scatter_reduce(0, idx, x, "amax", include_self=False) \
        .backward(g.double())
    # no ties in N(0,1) data: amax's gradient goes to the single winner
    assert np.array_equal(x.grad.float().numpy(), orc.max_backward(g.numpy(), a, w.N))


# ------------------------------------------- callers on either side of the path --

def test_ingroup_inds_oracle():
    rng = np.random.default_rng(21)
    g = rng.integers(0, 37, size=4000).astype(np.int64)
    out = orc.ingroup_inds(g)
    # what the reference guarantees: inside each group the ranks are 0..cnt-1, each once
    for gid in range(37):
        r = np.sort(out[g == gid])
        assert np.array_equal(r, np.arange(r.shape[0]))
    # in index order: rank = number of earlier elements of the same group (brute force)
    brute = np.array([int((g[:i] == g[i]).sum()) for i in range(300)])
    assert np.array_equal(out[:300], brute)


def test_voxelize_oracle_against_torch_floor_division():
    g = torch.Generator().manual_seed(31)
    pts = torch.rand((20000, 4), generator=g) * 160.0 - 80.0
    # points exactly on cell edges and just beside them, negative and positive
    edges = torch.arange(-80.0, 80.0, 0.25)[:640]
    pts[:640, 0] = edges
    pts[640:1280, 1] = torch.nextafter(edges, torch.tensor(-1e9))
    pts[1280:1920, 2] = torch.nextafter(edges, torch.tensor(1e9)) * 0.05
    voxel_size, pc_range = [0.25, 0.25, 0.4], [-80, -80, -2, 80, 80, 4]
    want = tor.voxelize(pts, voxel_size, pc_range).numpy()
    coors, keys = orc.voxelize(pts.numpy(), voxel_size, pc_range[:3], [640, 640, 15])
    assert np.array_equal(coors, want)
    inr = ((want >= 0) & (want < np.array([640, 640, 15]))).all(1)
    wk = tor.flatten_coors(torch.from_numpy(want), (640, 640, 15)).numpy()
    assert np.array_equal(keys[inr], wk[inr].astype(np.int32))
    # Python's floor division is not floor(a / b) in general; the textbook cases agree
    for a, b in [(7.0, 2.0), (-7.0, 2.0), (7.0, -2.0), (0.3, 0.1), (-0.3, 0.1), (1.0, 0.1)]:
        c, _ = orc.voxelize(np.array([[a, 0, 0]], np.float32), [b, 1, 1], [0, 0, 0], [1 << 20, 1, 1])
        assert c[0, 0] == int(np.float32(a) // np.float32(b)), (a, b)


def _boxes_and_points(seed, B=12, P=4000):
    g = torch.Generator().manual_seed(seed)
    rois = torch.zeros((B, 7))
    rois[:, 0:2] = torch.rand((B, 2), generator=g) * 40 - 20
    rois[:, 2] = torch.rand((B,), generator=g) * 2 - 1
    rois[:, 3:6] = torch.rand((B, 3), generator=g) * 4 + 1
    rois[:, 6] = torch.rand((B,), generator=g) * 6.283 - 3.1415
    pts = torch.zeros((P, 3))
    pts[:, 0:2] = torch.rand((P, 2), generator=g) * 50 - 25
    pts[:, 2] = torch.rand((P,), generator=g) * 6 - 2
    # plant points around every box so that each has hits
    per = P // (2 * B)
    for b in range(B):
        pts[b * per:(b + 1) * per, 0:2] = rois[b, 0:2] + (torch.rand((per, 2), generator=g) - 0.5) * 6
        pts[b * per:(b + 1) * per, 2] = rois[b, 2] + torch.rand((per,), generator=g) * rois[b, 5]
    return rois, pts


def test_dynamic_point_pool_oracle_geometry():
    """Pins the restated box test against an independent formulation: rotate the point
    into the box frame with a rotation matrix in float64 and compare the in-box /
    in-margin classification and the 13 numbers (float tolerance: the formulas differ
    in rounding, not in meaning)."""
    rois, pts = _boxes_and_points(3)
    extra = [0.6, 0.4, 0.2]
    idx, roi, feats = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, 10 ** 6, 10 ** 6)
    assert idx.shape[0] > 500
    R, Pn = rois.double().numpy(), pts.double().numpy()
    want = []
    for b in range(R.shape[0]):
        cx, cy, cz, w, l, h, rz = R[b]
        a = rz + np.pi / 2
        dx, dy, dz = Pn[:, 0] - cx, Pn[:, 1] - cy, Pn[:, 2] - (cz + h / 2)
        lx = dx * np.cos(a) - dy * np.sin(a)
        ly = dx * np.sin(a) + dy * np.cos(a)
        inside = (np.abs(lx) < l / 2) & (np.abs(ly) < w / 2) & (np.abs(dz) < h / 2)
        large = (np.abs(lx) < (l + extra[1]) / 2) & (np.abs(ly) < (w + extra[0]) / 2) & \
                (np.abs(dz) <= (h + extra[2]) / 2)
        for p in np.nonzero(large)[0]:
            want.append((b, p, lx[p], ly[p], dz[p], 0.0 if inside[p] else 1.0, w, l, h))
    got = {(int(r), int(i)): f for i, r, f in zip(idx, roi, feats)}
    near = 0
    for (b, p, lx, ly, dz, margin, w, l, h) in want:
        edge = min(abs(abs(lx) - l / 2), abs(abs(ly) - w / 2), abs(abs(dz) - h / 2),
                   abs(abs(lx) - (l + extra[1]) / 2), abs(abs(ly) - (w + extra[0]) / 2),
                   abs(abs(dz) - (h + extra[2]) / 2))
        if edge < 1e-4:      # a float-rounding distance from a face: either answer is right
            near += 1
            continue
        f = got[(b, p)]
        np.testing.assert_allclose(f[3:6], [lx, ly, dz], atol=2e-5)
        np.testing.assert_allclose(f[6:12], [lx + l / 2, ly + w / 2, dz + h / 2, -lx + l / 2, -ly + w / 2,
                                             -dz + h / 2], atol=3e-5)
        assert f[12] == margin and np.array_equal(f[0:3], pts.numpy()[p])
    assert len(got) >= len(want) - near and near < 20
    # (box, point) order, and the caps keep the first hits in that order
    order = np.lexsort((idx, roi))
    assert np.array_equal(order, np.arange(idx.shape[0]))
    i2, r2, f2 = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, 7, 50)
    assert i2.shape[0] == 50 and np.bincount(r2).max() <= 7
    keep = np.concatenate([np.nonzero(roi == b)[0][:7] for b in range(rois.shape[0])])[:50]
    assert np.array_equal(i2, idx[keep]) and np.array_equal(f2, feats[keep])


def test_dynamic_point_pool_oracle_mixed_batches():
    """A batch held in one pair of tensors (generate_pts_mask_for_box3d_mixed,
    dynamic_point_pool_kernel.cu:173-212) gives what the single-sample op gives sample by
    sample: the pairs of sample s are the op's output on that sample's boxes and points, with
    the indices mapped back; a pair of different samples never appears."""
    rois, pts = _boxes_and_points(5)
    g = torch.Generator().manual_seed(6)
    rb = torch.randint(0, 3, (rois.shape[0],), generator=g).numpy().astype(np.int32)
    pb = torch.randint(0, 3, (pts.shape[0],), generator=g).numpy().astype(np.int32)
    extra = [0.5, 0.5, 0.3]
    idx, roi, feats = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, 10 ** 6, 10 ** 6, rb, pb)
    assert idx.shape[0] > 100 and np.array_equal(rb[roi], pb[idx])
    parts = []
    for s_ in range(3):
        bsel, psel = np.nonzero(rb == s_)[0], np.nonzero(pb == s_)[0]
        i1, r1, f1 = orc.dynamic_point_pool(rois.numpy()[bsel], pts.numpy()[psel], extra, 10 ** 6, 10 ** 6)
        parts.append((psel[i1], bsel[r1], f1))
    wi = np.concatenate([p[0] for p in parts])
    wr = np.concatenate([p[1] for p in parts])
    wf = np.concatenate([p[2] for p in parts])
    order = np.lexsort((wi, wr))               # the mixed op emits in (box, point) order
    assert np.array_equal(idx, wi[order]) and np.array_equal(roi, wr[order])
    assert np.array_equal(feats.view(np.uint32), wf[order].view(np.uint32))
    # all in one sample: the plain op
    z_r, z_p = np.zeros_like(rb), np.zeros_like(pb)
    a = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, 9, 400, z_r, z_p)
    b = orc.dynamic_point_pool(rois.numpy(), pts.numpy(), extra, 9, 400)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


def test_grid_hash_oracle():
    rng = np.random.default_rng(5)
    keys = rng.choice(10 ** 7, size=3000, replace=False).astype(np.int32)
    vals = np.arange(3000, dtype=np.int32)
    table = orc.grid_hash_build(keys, vals)
    assert table.shape == (4096, 2)
    # a dictionary is the specification: every key maps to its value, others to -1
    assert np.array_equal(orc.grid_hash_probe(keys, table), vals)
    missing = np.setdiff1d(rng.integers(0, 10 ** 7, size=2000).astype(np.int32), keys)
    assert (orc.grid_hash_probe(missing, table) == -1).all()
    stored = table[table[:, 0] != -1]
    assert stored.shape[0] == 3000 and set(map(tuple, stored)) == set(zip(keys.tolist(), vals.tolist()))
    # probe sequence of functions.cuh:33-36: first slot key % size, step 2*key+1 (odd: full cycle)
    k = int(keys[0])
    first = k % 4096
    assert table[first, 0] != -1
    # a full table (N a power of two) still places every key
    keys2 = rng.choice(10 ** 6, size=1024, replace=False).astype(np.int32)
    t2 = orc.grid_hash_build(keys2, np.arange(1024, dtype=np.int32))
    assert (t2[:, 0] != -1).all() and np.array_equal(orc.grid_hash_probe(keys2, t2), np.arange(1024))


def test_property_random_small_inputs_against_python_loops():
    """Hypothesis-driven: the C oracle's spec functions against plain Python loops on
    small random inputs with planted ties, signed zeros and empty voxels."""
    from hypothesis import given, settings, strategies as st

    vals = st.sampled_from([-2.0, -1.0, -0.0, 0.0, 0.5, 1.0, 1.0, 3.0])

    @settings(max_examples=80, deadline=None)
    @given(st.integers(1, 6).flatmap(lambda U: st.tuples(
        st.just(U), st.lists(st.tuples(st.integers(0, U - 1), vals, vals), min_size=1, max_size=40))))
    def check(case):
        U, rows = case
        inv = np.array([r[0] for r in rows], dtype=np.int32)
        f = np.array([[r[1], r[2]] for r in rows], dtype=np.float32)
        N, C = f.shape
        s = orc.scatter_sum_f64(f, inv, U)
        mx, arg = orc.scatter_max_first(f, inv, U)
        cnt = orc.counts(inv, U)
        for u in range(U):
            members = [i for i in range(N) if inv[i] == u]
            assert cnt[u] == len(members)
            for c in range(C):
                assert s[u, c] == sum(float(f[i, c]) for i in members)
                if not members:
                    assert arg[u, c] == -1
                    continue
                best = members[0]
                for i in members[1:]:
                    if f[i, c] > f[best, c]:      # strict: the first of equal maxima stays
                        best = i
                assert arg[u, c] == best
                assert mx[u, c].tobytes() == f[best, c].tobytes()
        g = np.arange(U * C, dtype=np.float32).reshape(U, C) + 1
        gin = orc.max_backward(g, arg, N)
        for i in range(N):
            for c in range(C):
                assert gin[i, c] == (g[inv[i], c] if arg[inv[i], c] == i else 0.0)
        assert np.array_equal(orc.sum_backward(g, inv), g[inv])

    check()
