"""GPU parity: the HIP path (through scatter_ext -> C ABI) against the CPU oracle on
identical seeded inputs.

Bars: preSum / perm / counts / arg bit-exact; max values bit-exact; backward of sum,
mean and max bit-exact (copies and one correctly rounded division); forward sum and
mean within RTOL of the fp64 oracle, measured against the magnitude of the summands:
``|got - want| <= RTOL * sum_i |x_i|`` (``/ cnt`` for mean), RTOL = 1e-5 for fp32 and
2e-3 for fp16 / bf16 (fp32 accumulation).  A sum of zero-mean data has no meaningful
relative error against its own (possibly tiny) value, hence the summand scale.
For half-precision outputs the final rounding of the fp32 accumulator to the output
dtype adds up to half a unit in the last place of that dtype (2^-11 relative for fp16,
2^-8 for bf16 -- the latter alone is above 2e-3), so ``OUT_EPS * |want|`` is added.
"""
import sys

import numpy as np
import pytest
import torch

from oracle import c_oracle as orc
from tests import workloads

pytestmark = pytest.mark.gpu

RTOL = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 2e-3}
OUT_EPS = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}
DEV = "cuda:0"


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def tx():
    import torchex_amd
    return torchex_amd


def bits_equal(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    both_nan = np.isnan(a) & np.isnan(b)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32)[~both_nan], b.view(np.uint32)[~both_nan])


def run_case(name, feats, unq_inv, unq_cnts, dtype=torch.float32, grad_seed=100, check_plan=True,
             heavy_threshold=None, max_tie_rule=None, path=None):
    """feats fp32 CPU [N, C]; unq_inv int64 CPU; unq_cnts int64 CPU.  Returns the
    ScatterData for extra checks.  scatter_max is checked against the oracle of the tie
    rule in force: by default the reference kernel's own winner (lane-exact emulation)
    when the rows are grouped by voxel, the smallest row otherwise."""
    T = tx()
    N, C = feats.shape
    U = unq_cnts.shape[0]
    say(f"[case] {name} N={N} C={C} U={U} dtype={dtype}")
    f_in = feats.to(dtype)                 # what both sides see
    f32 = f_in.float().numpy()             # exact upcast for the oracle
    inv32 = unq_inv.numpy().astype(np.int32)
    cnt = unq_cnts.numpy()

    fg = f_in.to(DEV).requires_grad_(True)
    data = T.ScatterData(unq_inv.to(DEV), unq_cnts.to(DEV), heavy_threshold=heavy_threshold,
                         max_tie_rule=max_tie_rule)
    if path is not None:
        data.path = path
    grouped = N < 2 or bool((unq_inv[1:] >= unq_inv[:-1]).all())
    assert data.is_sorted == grouped
    assert data.max_tie_rule == (max_tie_rule or ("reference" if grouped else "first"))

    # ---- index preparation: integers, exact
    want_pre = orc.presum(orc.counts(inv32, U))
    assert np.array_equal(data.preSum.cpu().numpy(), want_pre), "preSum"
    assert data.num_unq == U and data.max_cnt == (int(cnt.max()) if U else 0)
    if check_plan and N:
        want_perm = orc.stable_perm(inv32, want_pre)
        got_perm = data.perm.cpu().numpy() if data.perm is not None else np.arange(N, dtype=np.int32)
        assert np.array_equal(got_perm, want_perm), "perm"
        seg = data.seg.cpu().numpy()
        assert np.array_equal(seg & 0x7fffffff, inv32[want_perm]), "seg ids"
        heavy = cnt > data.heavy_threshold
        # a handful of voxels just above the default threshold stay ordinary
        if data.heavy_threshold == 64 and 0 < int(heavy.sum()) <= 64 and int(cnt.max()) <= 96:
            heavy[:] = False
        special = heavy | (cnt == 0)
        assert np.array_equal(seg < 0, special[inv32[want_perm]]), "seg special bit"
        assert data.num_special == int(special.sum()) and data.num_heavy == int(heavy.sum())
        slot = data.slot_of.cpu().numpy()
        assert np.array_equal(slot >= 0, special), "slot_of"

    # ---- forward
    s = T.scatter_sum(fg, data)
    mean = T.scatter_mean(fg, data)
    mx, arg = T.scatter_max(fg, data)
    assert s.dtype == dtype and mean.dtype == dtype and mx.dtype == dtype and arg.dtype == torch.int32
    assert tuple(s.shape) == (U, C) and tuple(arg.shape) == (U, C)

    s64 = orc.scatter_sum_f64(f32, inv32, U)
    sabs = orc.scatter_sum_f64(np.abs(f32), inv32, U)
    rt, oe = RTOL[dtype], OUT_EPS[dtype]
    got = s.detach().float().cpu().numpy().astype(np.float64)
    finite = np.isfinite(sabs)
    assert np.all(np.abs(got - s64)[finite] <= (rt * sabs + oe * np.abs(s64))[finite] + 1e-30), \
        f"sum: worst {np.max((np.abs(got - s64) / (sabs + 1e-30))[finite]):.3e}"
    nz = cnt > 0
    gotm = mean.detach().float().cpu().numpy().astype(np.float64)
    wantm = s64[nz] / cnt[nz, None]
    fm = finite[nz]
    assert np.all(np.abs(gotm[nz] - wantm)[fm] <=
                  (rt * sabs[nz] / cnt[nz, None] + oe * np.abs(wantm))[fm] + 1e-30), "mean"
    assert np.all(np.isnan(gotm[~nz])), "mean of an empty voxel is 0/0 as in the reference"

    if data.max_tie_rule == "reference":
        want_max, want_arg = orc.scatter_max_reforder(f32, inv32, U)
    else:
        want_max, want_arg = orc.scatter_max_first(f32, inv32, U)
    got_arg = arg.cpu().numpy()
    assert np.array_equal(got_arg, want_arg), \
        f"arg: {int((got_arg != want_arg).sum())} of {want_arg.size} differ"
    got_max = mx.detach().float().cpu().numpy()
    if dtype == torch.float32:
        assert bits_equal(got_max, want_max), "max"
    else:  # lowest finite value of the dtype stands in for -FLT_MAX on winner-less cells
        has = want_arg >= 0
        assert bits_equal(got_max[has], want_max[has]), "max"
        assert np.all(got_max[~has] == float(torch.finfo(dtype).min))

    # ---- backward (upstream gradients N(0,1), rounded to the dtype)
    g = workloads.upstream_grad(U, C, grad_seed).to(dtype)
    g32 = g.float().numpy()
    gd = g.to(DEV)

    def grad_of(out):
        fg.grad = None
        out.backward(gd)
        return fg.grad.detach().float().cpu().numpy()

    assert bits_equal(grad_of(s), orc.sum_backward(g32, inv32)), "sum backward"
    want_mb = orc.mean_backward(g32, np.maximum(cnt, 1), inv32)
    if dtype != torch.float32:
        want_mb = torch.from_numpy(want_mb).to(dtype).float().numpy()
    assert bits_equal(grad_of(mean), want_mb), "mean backward"
    assert bits_equal(grad_of(mx), orc.max_backward(g32, want_arg, N)), "max backward"
    return data


# ------------------------------------------------------------ tiny and edges --

def test_hand_cases(hand_cases):
    T = tx()
    for c in hand_cases:
        say("[case] hand", c["name"])
        inv = torch.from_numpy(c["inv"]).long()
        U = int(inv.max()) + 1
        cnts = torch.bincount(inv, minlength=U)
        f = torch.from_numpy(c["feats"]).to(DEV)
        data = T.ScatterData(inv.to(DEV), cnts.to(DEV), max_tie_rule="first")
        mx, arg = T.scatter_max(f, data)
        assert bits_equal(mx.cpu().numpy(), c["max"]) and np.array_equal(arg.cpu().numpy(), c["arg"])
        if "arg_ref" in c:   # grouped rows: the default reports what the reference kernel reports
            dref = T.ScatterData(inv.to(DEV), cnts.to(DEV))
            assert dref.is_sorted and dref.max_tie_rule == "reference"
            mx, arg = T.scatter_max(f, dref)
            assert np.array_equal(arg.cpu().numpy(), c["arg_ref"]), c["name"]
            assert bits_equal(mx.cpu().numpy(), c.get("max_ref", c["max"])), c["name"]
        if "sum" in c:
            np.testing.assert_allclose(T.scatter_sum(f, data).cpu().numpy(), c["sum"], rtol=1e-6)
            np.testing.assert_allclose(T.scatter_mean(f, data).cpu().numpy(), c["mean"], rtol=1e-6)


@pytest.mark.parametrize("C", [1, 3, 13, 16, 32, 64, 128, 129, 260])
def test_channel_widths(C):
    g = torch.Generator().manual_seed(C)
    N, U = 3000, 97
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    run_case(f"channels{C}", torch.randn((N, C), generator=g), inv, torch.bincount(inv, minlength=U))


def test_single_voxel_single_point_and_singletons():
    g = torch.Generator().manual_seed(1)
    run_case("N1", torch.randn((1, 8), generator=g), torch.zeros(1, dtype=torch.long), torch.ones(1, dtype=torch.long))
    run_case("U1", torch.randn((500, 8), generator=g), torch.zeros(500, dtype=torch.long),
             torch.full((1,), 500, dtype=torch.long))
    inv = torch.randperm(777, generator=g)
    run_case("singletons", torch.randn((777, 12), generator=g), inv, torch.ones(777, dtype=torch.long))


def test_heavy_ties_integers():
    # small integer features: many equal maxima (first row must win), exact sums
    g = torch.Generator().manual_seed(2)
    N, U, C = 40000, 50, 20
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    feats = torch.randint(-3, 4, (N, C), generator=g).float()
    data = run_case("ties", feats, inv, torch.bincount(inv, minlength=U))
    assert data.num_special == U  # ~800 rows per voxel: all go through the atomic table
    T = tx()
    s = T.scatter_sum(feats.to(DEV), data).cpu().numpy().astype(np.float64)
    assert np.array_equal(s, orc.scatter_sum_f64(feats.numpy(), inv.numpy().astype(np.int32), U))


def test_all_equal_features_pure_tie():
    N, U, C = 5000, 9, 8
    inv = torch.arange(N) % U
    run_case("all_equal", torch.full((N, C), 2.5), inv, torch.bincount(inv, minlength=U))


def test_special_values():
    g = torch.Generator().manual_seed(3)
    N, U, C = 6000, 40, 8
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    f = torch.randn((N, C), generator=g)
    f[torch.rand((N, C), generator=g) < 0.05] = float("nan")
    f[torch.rand((N, C), generator=g) < 0.05] = float("-inf")
    f[torch.rand((N, C), generator=g) < 0.02] = float("inf")
    f[torch.rand((N, C), generator=g) < 0.05] = -0.0
    f[torch.rand((N, C), generator=g) < 0.05] = 0.0
    # voxels 0..2: only NaN / only -inf / NaN then -inf, light and heavy variants below
    f[inv == 0] = float("nan")
    f[inv == 1] = float("-inf")
    f[inv == 2] = float("nan")
    rows2 = torch.nonzero(inv == 2).flatten()
    f[rows2[len(rows2) // 2:]] = float("-inf")
    T = tx()
    for thr in (None, 1 << 20):   # through the atomic table, and all in registers
        say("[case] special values, heavy_threshold", thr)
        data = T.ScatterData(inv.to(DEV), torch.bincount(inv, minlength=U).to(DEV), heavy_threshold=thr)
        mx, arg = T.scatter_max(f.to(DEV), data)
        wm, wa = orc.scatter_max_first(f.numpy(), inv.numpy().astype(np.int32), U)
        assert np.array_equal(arg.cpu().numpy(), wa)
        assert bits_equal(mx.cpu().numpy(), wm)
        assert (wa[0] == -1).all() and (wa[1] == int(torch.nonzero(inv == 1)[0])).all()
        # sums propagate NaN/inf like any fp32 sum
        s = T.scatter_sum(f.to(DEV), data).cpu().numpy()
        w = orc.scatter_sum_f64(f.numpy(), inv.numpy().astype(np.int32), U)
        assert np.array_equal(np.isnan(s), np.isnan(w))
        assert np.array_equal(np.isinf(s), np.isinf(w))


def test_sorted_input_takes_identity_path_and_matches_unsorted():
    T = tx()
    g = torch.Generator().manual_seed(4)
    N, U, C = 20000, 700, 32
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    feats = torch.randn((N, C), generator=g)
    order = torch.argsort(inv, stable=True)
    run_case("sorted_default_rule", feats[order], inv[order], torch.bincount(inv, minlength=U))
    d_sorted = run_case("sorted", feats[order], inv[order], torch.bincount(inv, minlength=U),
                        max_tie_rule="first")
    assert d_sorted.perm is None and d_sorted.is_sorted
    d_uns = T.ScatterData(inv.to(DEV), torch.bincount(inv, minlength=U).to(DEV))
    assert d_uns.perm is not None
    a = T.scatter_max(feats[order].to(DEV), d_sorted)
    b = T.scatter_max(feats.to(DEV), d_uns)
    assert torch.equal(a[0], b[0])
    assert torch.equal(order.to(DEV)[a[1].long()].int(), b[1])
    # same accumulation order on both paths -> identical sums for the register path
    sa = T.scatter_sum(feats[order].to(DEV), d_sorted)
    sb = T.scatter_sum(feats.to(DEV), d_uns)
    light = (torch.bincount(inv, minlength=U) <= d_uns.heavy_threshold).to(DEV)
    assert torch.equal(sa[light], sb[light])
    # mean is the sum divided once by the count (scatter_op.py:69)
    m = T.scatter_mean(feats.to(DEV), d_uns)
    assert torch.equal(m[light], (sb / d_uns.unq_cnts)[light])


def test_empty_voxels_and_empty_input():
    T = tx()
    g = torch.Generator().manual_seed(5)
    N, U, C = 1000, 30, 8
    inv = torch.randint(0, U, (N,), generator=g)
    inv[inv % 7 == 3] = 0   # leaves several ids unused
    cnts = torch.bincount(inv, minlength=U)
    assert (cnts == 0).any()
    run_case("empty_voxels", torch.randn((N, C), generator=g), inv, cnts)
    say("[case] N=0")
    data = T.ScatterData(torch.zeros(0, dtype=torch.long, device=DEV), torch.zeros(4, dtype=torch.long, device=DEV))
    f = torch.zeros((0, 8), device=DEV)
    assert torch.equal(T.scatter_sum(f, data), torch.zeros((4, 8), device=DEV))
    mx, arg = T.scatter_max(f, data)
    assert (arg == -1).all() and (mx == torch.finfo(torch.float32).min).all()


def test_heavy_threshold_boundary_runs():
    # voxel sizes around the chunk length and the heavy threshold, in every phase
    # relative to chunk boundaries
    sizes = [1, 31, 32, 33, 63, 64, 65, 1, 2, 127, 128, 129, 64, 64, 1, 200, 32, 32, 32, 64, 1, 1, 65, 5]
    sizes = sizes * 3 + [1] * 70 + [64] * 5 + [3] * 33
    cnts = torch.tensor(sizes, dtype=torch.long)
    U = len(sizes)
    inv_sorted = torch.repeat_interleave(torch.arange(U), cnts)
    g = torch.Generator().manual_seed(6)
    N = int(cnts.sum())
    feats = torch.randn((N, 16), generator=g)
    run_case("boundaries_sorted", feats, inv_sorted, cnts)
    p = torch.randperm(N, generator=g)
    run_case("boundaries_shuffled", feats, inv_sorted[p], cnts)
    run_case("boundaries_thr32", feats, inv_sorted[p], cnts, heavy_threshold=32)


@pytest.mark.parametrize("C", [8, 128])
def test_heavy_runs_shorter_than_the_long_chunk(C):
    """Runs of 17..24 rows with the heavy threshold at its minimum (16): every voxel is on the
    heavy path, the average run is long enough for the forward's 32-position chunk, and such a
    chunk then meets up to three heavy runs: one more partial than a lane group can park."""
    g = torch.Generator().manual_seed(61)
    U = 3000
    cnts = torch.randint(17, 25, (U,), generator=g)
    inv_sorted = torch.repeat_interleave(torch.arange(U), cnts)
    N = int(cnts.sum())
    assert N >= 8 * U
    feats = torch.randn((N, C), generator=g)
    feats[torch.rand((N, C), generator=g) < 0.2] = 1.5          # ties
    run_case("short_heavy_runs_sorted", feats, inv_sorted, cnts, heavy_threshold=16)
    p = torch.randperm(N, generator=g)
    data = run_case("short_heavy_runs_shuffled", feats, inv_sorted[p], cnts, heavy_threshold=16)
    assert data.num_heavy == U
    run_case("short_heavy_runs_f16", feats, inv_sorted[p], cnts, heavy_threshold=16, dtype=torch.float16)


@pytest.mark.parametrize("C,dtype", [(16, torch.float32), (128, torch.float32), (128, torch.float16), (3, torch.float32)])
def test_ordinary_runs_longer_than_a_tile(C, dtype):
    """A heavy threshold far above the run lengths: every voxel is reduced in registers, also
    those whose runs are longer than the ids a tile stages behind its end (64) and longer than
    whole tiles.  A tile then finds no run start behind its end and its last lane group walks on
    to the run's end; a tile that lies inside such a run finds none behind its start either and
    owns nothing; runs of a few rows sit between the long ones."""
    g = torch.Generator().manual_seed(77)
    sizes = []
    for _ in range(120):
        sizes += [int(torch.randint(65, 700, (1,), generator=g)), int(torch.randint(1, 9, (1,), generator=g)),
                  int(torch.randint(1, 4, (1,), generator=g))]
    sizes += [2500, 1, 64, 65, 129, 1, 1, 300]
    cnts = torch.tensor(sizes, dtype=torch.long)
    U = len(sizes)
    inv_sorted = torch.repeat_interleave(torch.arange(U), cnts)
    N = int(cnts.sum())
    feats = torch.randn((N, C), generator=g)
    feats[torch.rand((N, C), generator=g) < 0.05] = 2.0          # ties
    data = run_case("long_ordinary_runs_sorted", feats, inv_sorted, cnts, dtype=dtype, heavy_threshold=4000)
    assert data.num_heavy == 0
    p = torch.randperm(N, generator=g)
    run_case("long_ordinary_runs_shuffled", feats, inv_sorted[p], cnts, dtype=dtype, heavy_threshold=4000)
    run_case("long_ordinary_runs_first_tie", feats, inv_sorted, cnts, dtype=dtype, heavy_threshold=4000,
             max_tie_rule="first")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_few_short_heavy_voxels_stay_ordinary(dtype):
    """With the default threshold, a plan whose only heavy voxels are a handful just above it
    (64 at most, none above 96 rows) keeps them ordinary: no heavy table, no second kernel;
    their runs are reduced in registers and LDS, the rows beyond the ids a tile stages behind
    its end one by one.  One voxel more, or one longer voxel, and the heavy path is back."""
    g = torch.Generator().manual_seed(31)

    def make(long_sizes, n_short=3000):
        sizes = torch.randint(1, 9, (n_short,), generator=g)
        at = torch.randperm(n_short, generator=g)[:len(long_sizes)]
        sizes[at] = torch.tensor(long_sizes)
        inv_sorted = torch.repeat_interleave(torch.arange(n_short), sizes)
        N = int(sizes.sum())
        feats = torch.randn((N, 128), generator=g)
        feats[torch.rand((N, 128), generator=g) < 0.05] = 1.5     # ties
        return feats, inv_sorted, sizes

    few = [65, 66, 69, 70, 80, 95, 96, 96] + [65 + (7 * i) % 32 for i in range(40)]
    feats, inv_sorted, cnts = make(few)
    p = torch.randperm(inv_sorted.numel(), generator=g)
    data = run_case("few_short_heavy_shuffled", feats, inv_sorted[p], cnts, dtype=dtype)
    assert data.num_heavy == 0 and data.num_special == 0 and data.max_cnt == 96
    data = run_case("few_short_heavy_sorted", feats, inv_sorted, cnts, dtype=dtype)
    assert data.num_heavy == 0
    data = run_case("few_short_heavy_first_tie", feats, inv_sorted[p], cnts, dtype=dtype, max_tie_rule="first")
    assert data.num_heavy == 0
    # one voxel of 97 rows: the heavy path for all of them
    feats, inv_sorted, cnts = make(few[:-1] + [97])
    data = run_case("one_longer_heavy", feats, inv_sorted, cnts, dtype=dtype)
    assert data.num_heavy == len(few)
    # 65 voxels above the threshold: the same
    feats, inv_sorted, cnts = make([70] * 65)
    data = run_case("many_short_heavy", feats, inv_sorted, cnts, dtype=dtype)
    assert data.num_heavy == 65


@pytest.mark.parametrize("seed", range(24))
def test_seeded_shapes(seed):
    """Shapes nobody chose by hand: channel counts that leave lanes idle or need a second
    column block, run lengths from geometric, uniform and heavy-tailed draws, thresholds on
    both sides of the run lengths, all three dtypes, grouped and shuffled rows, empty voxels."""
    g = torch.Generator().manual_seed(9000 + seed)

    def ri(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=g))

    C = [1, 2, 3, 5, 7, 8, 12, 16, 24, 31, 32, 48, 64, 96, 100, 128, 160, 200, 256, 257, 300, 384, 512, 6][seed]
    U = ri(1, 4000)
    kind = seed % 3
    if kind == 0:      # short runs, some empty voxels
        cnts = torch.poisson(torch.full((U,), 1.5), generator=g).long()
    elif kind == 1:    # up to a few tiles long
        cnts = torch.randint(0, 3 * ri(8, 200), (U,), generator=g)
    else:              # heavy tail
        cnts = (torch.rand((U,), generator=g) ** 6 * ri(100, 3000)).long() + torch.randint(0, 2, (U,), generator=g)
    if int(cnts.sum()) == 0:
        cnts[0] = 1
    budget = 6_000_000 // C                      # rows the oracle gets through in a second or two
    while int(cnts.sum()) > budget:
        cnts = cnts // 2
    inv_sorted = torch.repeat_interleave(torch.arange(U), cnts)
    N = inv_sorted.numel()
    feats = torch.randn((N, C), generator=g)
    feats[torch.rand((N, C), generator=g) < 0.03] = 0.75       # ties
    thr = [None, 16, 32, 64, 100, 5000][ri(0, 5)]     # (16 is the smallest the library accepts)
    dtype = [torch.float32, torch.float16, torch.bfloat16][ri(0, 2)]
    inv = inv_sorted if seed % 4 == 0 else inv_sorted[torch.randperm(N, generator=g)]
    run_case(f"seeded_{seed}", feats, inv, cnts, dtype=dtype, heavy_threshold=thr, grad_seed=300 + seed)


# ------------------------------------------------- the reference's own test --

def test_reference_test_data_closed_forms(reference_counts):
    """test/test_scatter.py: 500 sorted groups, each channel a permutation of 0..n-1:
    sum = n(n-1)/2 exactly, mean = (n-1)/2 exactly, max = n-1, arg = its position."""
    T = tx()
    w = workloads.reference_test_groups(channel=128)
    assert w.unq_cnts.tolist() == reference_counts["counts"] and w.N == 1229413
    say("[case] reference test data", w.N, w.C)
    n = w.unq_cnts.double()
    col = w.feats[:, 0]
    starts = torch.cumsum(w.unq_cnts, 0) - w.unq_cnts
    argpos = torch.stack([s + torch.argmax(col[s:s + c]) for s, c in zip(starts.tolist(), w.unq_cnts.tolist())])
    f = w.feats.to(DEV)
    data = T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV))
    assert data.max_cnt == 4996 and data.perm is None
    assert data.preSum[-1].item() == w.N
    for _ in range(2):
        s = T.scatter_sum(f, data).cpu().double()
        assert torch.equal(s, (n * (n - 1) / 2).unsqueeze(1).expand(-1, 128))
        m = T.scatter_mean(f, data).cpu().double()
        assert torch.equal(m, ((n - 1) / 2).unsqueeze(1).expand(-1, 128))
        mx, arg = T.scatter_max(f, data)
        assert torch.equal(mx.cpu().double(), (n - 1).unsqueeze(1).expand(-1, 128))
        assert torch.equal(arg.cpu().long(), argpos.unsqueeze(1).expand(-1, 128))
    # the reference module's own entry points on the same tensors (scatter.cpp:66-70)
    import scatter_ext
    pre = T.getPreSum(w.unq_inv.to(DEV))
    assert torch.equal(pre, data.preSum)
    out = f.new_zeros((w.U, 128))
    scatter_ext.sum(f, pre, out, data.max_cnt)
    assert torch.equal(out.cpu().double(), (n * (n - 1) / 2).unsqueeze(1).expand(-1, 128))
    out = f.new_zeros((w.U, 128))
    arg = pre.new_zeros((w.U, 128))
    scatter_ext.max(f, pre, out, arg, data.max_cnt)
    assert torch.equal(arg.cpu().long(), argpos.unsqueeze(1).expand(-1, 128))
    assert torch.equal(out.cpu().double(), (n - 1).unsqueeze(1).expand(-1, 128))


# ------------------------------------------------------- benchmark workloads --

def test_uniform_box_and_reference_order_oracle():
    w = workloads.uniform_box()
    run_case("uniform_box", w.feats, w.unq_inv, w.unq_cnts)
    # this workload also against the reference's own fp32 summation order
    T = tx()
    data = T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV))
    s = T.scatter_sum(w.feats.to(DEV), data).cpu().numpy()
    inv32 = w.unq_inv.numpy().astype(np.int32)
    ref = orc.scatter_sum_reforder(w.feats.numpy(), inv32, w.U)
    sabs = orc.scatter_sum_f64(np.abs(w.feats.numpy()), inv32, w.U)
    assert np.all(np.abs(s.astype(np.float64) - ref) <= 1e-5 * sabs)
    mr, ar = orc.scatter_max_reforder(w.feats.numpy(), inv32, w.U)
    mx, arg = T.scatter_max(w.feats.to(DEV), data)
    assert bits_equal(mx.cpu().numpy(), mr) and np.array_equal(arg.cpu().numpy(), ar)


def test_lidar_sweep_fp32():
    w = workloads.lidar_sweep()
    run_case("lidar_sweep", w.feats, w.unq_inv, w.unq_cnts, grad_seed=102)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_lidar_sweep_half(dtype):
    w = workloads.lidar_sweep(N=1_000_000, C=128, seed=2)
    run_case("lidar_sweep_half", w.feats, w.unq_inv, w.unq_cnts, dtype=dtype, grad_seed=102)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_lidar_pillars(dtype):
    """Unsorted rows, 512-byte (256-byte) rows, and two thirds of the points in voxels that are
    split across lane groups and merged through LDS and the atomic table."""
    w = workloads.lidar_pillars()
    assert int(w.unq_cnts.max()) > 1000 and int((w.unq_cnts > 64).sum()) > 2000
    data = run_case("lidar_pillars", w.feats, w.unq_inv, w.unq_cnts, dtype=dtype, grad_seed=102)
    assert data.num_heavy == int((w.unq_cnts > 64).sum())


def test_lidar_pillars_grouped_rows():
    """The same points delivered grouped by voxel, the reference's input contract: the
    default tie rule is then the reference's (block width 1024 here, several rows per thread
    in the fullest pillars)."""
    w = workloads.lidar_pillars()
    order = torch.sort(w.unq_inv, stable=True)[1]
    data = run_case("lidar_pillars_grouped", w.feats[order], w.unq_inv[order], w.unq_cnts, grad_seed=102)
    assert data.max_tie_rule == "reference" and data.max_cnt > 1024


def test_zipf_contention():
    w = workloads.zipf_contention()
    assert int(w.unq_cnts.max()) > 100_000
    run_case("zipf", w.feats, w.unq_inv, w.unq_cnts)


def test_multi_sweep():
    w = workloads.multi_sweep()
    run_case("multi_sweep", w.feats, w.unq_inv, w.unq_cnts, check_plan=True)


# ------------------------------------------------------ size-independent laws --

def test_linearity_and_permutation_invariance_full_size():
    T = tx()
    w = workloads.lidar_sweep(N=1_000_000, C=32, seed=7)
    say("[case] laws", w.N, w.C, w.U)
    inv = w.unq_inv.to(DEV)
    data = T.ScatterData(inv, w.unq_cnts.to(DEV))
    f = w.feats.to(DEV)
    mx, arg = T.scatter_max(f, data)
    # arg points into the right voxel and at the winning value; no earlier row of the
    # voxel attains it
    assert torch.equal(inv[arg.long()], torch.arange(w.U, device=DEV).unsqueeze(1).expand(-1, w.C))
    assert torch.equal(torch.gather(f, 0, arg.long()), mx)
    assert (f <= mx[inv]).all()
    rows = torch.arange(w.N, device=DEV).unsqueeze(1)
    assert not ((f == mx[inv]) & (rows < arg[inv])).any()
    # integer-valued features: sums are exact, so linearity and shuffling are bit-exact
    fi = torch.randint(-8, 9, (w.N, w.C), generator=torch.Generator().manual_seed(1)).float().to(DEV)
    fj = torch.randint(-8, 9, (w.N, w.C), generator=torch.Generator().manual_seed(2)).float().to(DEV)
    assert torch.equal(T.scatter_sum(fi + fj, data), T.scatter_sum(fi, data) + T.scatter_sum(fj, data))
    p = torch.randperm(w.N, generator=torch.Generator().manual_seed(3)).to(DEV)
    data_p = T.ScatterData(inv[p], w.unq_cnts.to(DEV))
    assert torch.equal(T.scatter_sum(fi[p], data_p), T.scatter_sum(fi, data))
    mp, ap = T.scatter_max(f[p], data_p)
    assert torch.equal(mp, mx)
    ones = torch.ones((w.N, w.C), device=DEV)
    assert torch.equal(T.scatter_sum(ones, data), w.unq_cnts.to(DEV).float().unsqueeze(1).expand(-1, w.C))
    # backward of sum then forward again is multiplication by the counts
    g = torch.randint(-8, 9, (w.U, w.C), generator=torch.Generator().manual_seed(4)).float().to(DEV)
    x = torch.zeros((w.N, w.C), device=DEV, requires_grad=True)
    T.scatter_sum(x, data).backward(g)
    assert torch.equal(T.scatter_sum(x.grad, data), g * data.unq_cnts)


def test_repeatability():
    T = tx()
    w = workloads.lidar_sweep(N=300_000, C=64, seed=9)
    data = T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV))
    f = w.feats.to(DEV)
    m0, a0 = T.scatter_max(f, data)
    mean0 = T.scatter_mean(f, data)
    light = (w.unq_cnts <= data.heavy_threshold).to(DEV)
    for _ in range(5):
        m1, a1 = T.scatter_max(f, data)
        assert torch.equal(m0, m1) and torch.equal(a0, a1)
        assert torch.equal(T.scatter_mean(f, data)[light], mean0[light])


# --------------------------------------------------------------- error paths --

def test_error_paths():
    T = tx()
    import scatter_ext
    g = torch.Generator().manual_seed(8)
    N, U, C = 100, 5, 8
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    cnts = torch.bincount(inv, minlength=U)
    data = T.ScatterData(inv.to(DEV), cnts.to(DEV))
    f = torch.randn((N, C), generator=g)
    with pytest.raises(RuntimeError):
        T.scatter_sum(f, data)                                # CPU tensor (scatter.cpp:4-5)
    with pytest.raises(RuntimeError):
        T.scatter_sum(f.to(DEV).t().contiguous().t(), data)   # non-contiguous (scatter.cpp:6-7)
    with pytest.raises(RuntimeError):
        T.scatter_sum(f.double().to(DEV), data)               # unsupported dtype
    with pytest.raises(RuntimeError):
        T.scatter_max(f[:50].to(DEV), data)                   # row count mismatch
    with pytest.raises(RuntimeError):
        T.ScatterData((inv + 1).to(DEV), cnts.to(DEV))        # id out of range
    with pytest.raises(AssertionError):
        T.ScatterData(inv.to(DEV), (cnts + 1).to(DEV))        # counts are not the histogram
    with pytest.raises(AssertionError):
        T.ScatterData(inv.to(DEV).reshape(N, 1, 1), cnts.to(DEV))
    out = torch.zeros((U, C), device=DEV)
    with pytest.raises(RuntimeError):
        scatter_ext.sum(f.to(DEV), data.preSum.long(), out, data.max_cnt)  # preSum dtype
    with pytest.raises(RuntimeError):
        scatter_ext.sum(f.to(DEV), data.preSum[:-1].contiguous(), out, data.max_cnt)
    # a failed call leaves the device usable
    assert torch.isfinite(T.scatter_sum(f.to(DEV), data)).all()


def test_c_abi_direct_call():
    """Calls libtorchex_scatter.so through ctypes with raw device pointers, the way a
    non-torch host would bind it."""
    import ctypes
    from torchex_amd import _native
    lib = _native.cabi()
    T = tx()
    g = torch.Generator().manual_seed(10)
    N, U, C = 5000, 300, 32
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    feats = torch.randn((N, C), generator=g)
    data = T.ScatterData(inv.to(DEV), torch.bincount(inv, minlength=U).to(DEV))
    f = feats.to(DEV)
    out = torch.empty((U, C), device=DEV)
    arg = torch.empty((U, C), device=DEV, dtype=torch.int32)
    lib.txs_scatter_scratch_cells.restype = ctypes.c_int64
    vp = ctypes.c_void_p
    i64 = ctypes.c_int64
    cells = lib.txs_scatter_scratch_cells(i64(N), i64(C), i64(U), i64(data.num_heavy))
    assert cells == data.num_heavy * C      # 300 voxels of ~17 rows: no table mode, no partial tables
    scratch = torch.zeros((max(cells, 1),), device=DEV, dtype=torch.int64)
    stream = vp(torch.cuda.current_stream().cuda_stream)
    lib.txs_scatter_forward.restype = ctypes.c_int
    rc = lib.txs_scatter_forward(
        ctypes.c_int(2), ctypes.c_int(0), vp(f.data_ptr()), vp(data.row_ids.data_ptr()), vp(data.perm.data_ptr()),
        vp(data.seg.data_ptr()), vp(data.preSum.data_ptr()), vp(data.slot_of.data_ptr()),
        vp(data.heavy_ids.data_ptr() if data.num_special else 0), i64(data.num_special), i64(data.num_heavy),
        vp(scratch.data_ptr()), i64(cells), vp(out.data_ptr()), vp(arg.data_ptr()), i64(N), i64(C), i64(U),
        i64(data.max_cnt), ctypes.c_int(0), stream)
    assert rc == 0
    torch.cuda.synchronize()
    wm, wa = orc.scatter_max_first(feats.numpy(), inv.numpy().astype(np.int32), U)
    assert bits_equal(out.cpu().numpy(), wm) and np.array_equal(arg.cpu().numpy(), wa)
    assert (scratch == 0).all()
    gin = torch.empty((N, C), device=DEV)
    gup = torch.randn((U, C), generator=g).to(DEV)
    lib.txs_scatter_backward.restype = ctypes.c_int
    rc = lib.txs_scatter_backward(
        ctypes.c_int(2), ctypes.c_int(0), vp(gup.data_ptr()), vp(arg.data_ptr()), vp(data.row_ids.data_ptr()),
        vp(data.perm.data_ptr()), vp(data.seg.data_ptr()), vp(data.preSum.data_ptr()), vp(gin.data_ptr()),
        i64(N), i64(C), i64(U), ctypes.c_int(0), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert bits_equal(gin.cpu().numpy(), orc.max_backward(gup.cpu().numpy(), wa, N))
    # argument validation returns a status instead of launching
    rc = lib.txs_scatter_forward(
        ctypes.c_int(7), ctypes.c_int(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), i64(0), i64(0), vp(0),
        i64(0), vp(0), vp(0), i64(N), i64(C), i64(U), i64(1), ctypes.c_int(0), stream)
    assert rc == 3
    rc = lib.txs_scatter_forward(
        ctypes.c_int(0), ctypes.c_int(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), i64(0), i64(0), vp(0),
        i64(0), vp(0), vp(0), i64(N), i64(C), i64(U), i64(1), ctypes.c_int(0), stream)
    assert rc == 1


# ------------------------------------------- the reference's own tie rule ----

def _tie_heavy_groups(seed, sizes, C):
    g = torch.Generator().manual_seed(seed)
    cnts = torch.tensor(sizes, dtype=torch.long)
    inv = torch.repeat_interleave(torch.arange(len(sizes)), cnts)
    feats = torch.randint(0, 3, (int(cnts.sum()), C), generator=g).float()   # many equal maxima
    return feats, inv, cnts


@pytest.mark.parametrize("sizes", [
    [5, 17, 31, 32, 33, 64, 1, 2, 100, 7] * 20,                 # block width 128: one row per thread
    [700, 33, 1024, 5, 900, 64, 65, 1] * 6,                     # width 1024, everything within one pass
    [2050, 1500, 40, 4996, 100, 1025, 3000, 64, 7, 1100] * 2,   # width 1024, several rows per thread
])
def test_reference_tie_rule_mode(sizes):
    """max_tie_rule='reference' reports, among equal maxima, the row the reference kernel
    keeps (lane-exact emulation in the oracle), for sorted input directly and for
    shuffled input through the stable sort; the raw scatter_ext.max entry point, which
    receives max_cnt like the reference's, does the same."""
    T = tx()
    import scatter_ext
    C = 12
    feats, inv, cnts = _tie_heavy_groups(len(sizes), sizes, C)
    U, N = len(sizes), feats.shape[0]
    inv32 = inv.numpy().astype(np.int32)
    say(f"[case] reference tie rule N={N} U={U} max_cnt={max(sizes)}")
    want_max, want_arg = orc.scatter_max_reforder(feats.numpy(), inv32, U)
    first_max, first_arg = orc.scatter_max_first(feats.numpy(), inv32, U)
    assert (want_arg != first_arg).any()   # the two rules really differ on this data

    data = T.ScatterData(inv.to(DEV), cnts.to(DEV), max_tie_rule="reference")
    mx, arg = T.scatter_max(feats.to(DEV), data)
    assert np.array_equal(arg.cpu().numpy(), want_arg)
    assert bits_equal(mx.cpu().numpy(), want_max)
    # grouped rows are the reference's own input: the default reports its winner too
    d0 = T.ScatterData(inv.to(DEV), cnts.to(DEV))
    assert d0.max_tie_rule == "reference"
    mx, arg = T.scatter_max(feats.to(DEV), d0)
    assert np.array_equal(arg.cpu().numpy(), want_arg) and bits_equal(mx.cpu().numpy(), want_max)
    # the smallest-row rule on the same data
    d1 = T.ScatterData(inv.to(DEV), cnts.to(DEV), max_tie_rule="first")
    assert np.array_equal(T.scatter_max(feats.to(DEV), d1)[1].cpu().numpy(), first_arg)
    # all rows through the register path as well (no heavy voxels)
    d2 = T.ScatterData(inv.to(DEV), cnts.to(DEV), heavy_threshold=1 << 20, max_tie_rule="reference")
    assert np.array_equal(T.scatter_max(feats.to(DEV), d2)[1].cpu().numpy(), want_arg)

    # the reference module's entry point on the sorted rows
    out = torch.zeros((U, C), device=DEV)
    a = torch.zeros((U, C), device=DEV, dtype=torch.int32)
    scatter_ext.max(feats.to(DEV), data.preSum, out, a, data.max_cnt)
    assert np.array_equal(a.cpu().numpy(), want_arg) and bits_equal(out.cpu().numpy(), want_max)

    # shuffled rows: the reference defines nothing there and the default is the smallest row
    p = torch.randperm(N, generator=torch.Generator().manual_seed(5))
    dsh = T.ScatterData(inv[p].to(DEV), cnts.to(DEV))
    assert dsh.max_tie_rule == "first"
    assert np.array_equal(T.scatter_max(feats[p].to(DEV), dsh)[1].cpu().numpy(),
                          orc.scatter_max_first(feats[p].numpy(), inv32[p.numpy()], U)[1])
    # forced: winner = reference rule on the stably sorted voxel, as original row ids
    want_max_s, want_arg_s = orc.scatter_max_reforder(feats[p].numpy(), inv32[p.numpy()], U)
    ds = T.ScatterData(inv[p].to(DEV), cnts.to(DEV), max_tie_rule="reference")
    mx, arg = T.scatter_max(feats[p].to(DEV).requires_grad_(True), ds)
    assert np.array_equal(arg.cpu().numpy(), want_arg_s)
    assert bits_equal(mx.detach().cpu().numpy(), want_max_s)
    # backward follows whichever arg was reported
    gup = workloads.upstream_grad(U, C, 9)
    x = feats[p].to(DEV).requires_grad_(True)
    T.scatter_max(x, ds)[0].backward(gup.to(DEV))
    assert bits_equal(x.grad.cpu().numpy(), orc.max_backward(gup.numpy(), want_arg_s, N))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_reference_tie_rule_special_values_and_half_precision(dtype):
    """Grouped rows (the reference's input, so its tie rule is in force) full of equal values,
    signed zeros, infinities and NaN, in every dtype, through registers and through the heavy-voxel
    table: arg and the value's bits against the lane-exact emulation of the reference kernel."""
    g = torch.Generator().manual_seed(55)
    sizes = [1, 2, 17, 33, 64, 65, 100, 300, 1500, 40, 3, 700]
    U, C = len(sizes), 10
    inv = torch.repeat_interleave(torch.arange(U), torch.tensor(sizes))
    N = inv.numel()
    f = torch.randint(-3, 4, (N, C), generator=g).float()          # few distinct values: ties everywhere
    f[torch.rand((N, C), generator=g) < 0.10] = -0.0
    f[torch.rand((N, C), generator=g) < 0.05] = float("nan")
    f[torch.rand((N, C), generator=g) < 0.03] = float("inf")
    f[torch.rand((N, C), generator=g) < 0.05] = float("-inf")
    f[inv == 9] = float("-inf")                                     # a voxel without a finite value
    f[inv == 10] = float("nan")
    cnts = torch.tensor(sizes)
    for thr in (None, 1 << 20):
        with np.errstate(invalid="ignore"):   # inf - inf in the checks of the sums
            data = run_case(f"reference ties, special values, threshold {thr}", f, inv, cnts, dtype=dtype,
                            heavy_threshold=thr)
        assert data.max_tie_rule == "reference"


def test_reference_tie_rule_mode_matches_default_without_ties():
    T = tx()
    w = workloads.lidar_sweep(N=200_000, C=32, seed=12)
    f = w.feats.to(DEV)
    a = T.scatter_max(f, T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV), max_tie_rule="first"))
    b = T.scatter_max(f, T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV), max_tie_rule="reference"))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


# ------------------------------------------------------------ robustness ----

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("C", [1, 2, 8, 13, 16, 72])
def test_half_precision_channel_widths(C, dtype):
    g = torch.Generator().manual_seed(100 + C)
    N, U = 4000, 61
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    run_case(f"half_channels{C}", torch.randn((N, C), generator=g), inv, torch.bincount(inv, minlength=U),
             dtype=dtype)


def test_many_rows_few_channels():
    """Index range and tile geometry at the other extreme: 12M rows of 2 channels (one lane per
    row, 4096 positions per workgroup)."""
    T = tx()
    g = torch.Generator().manual_seed(77)
    N, U, C = 12_000_000, 900_000, 2
    inv = torch.randint(0, U, (N,), generator=g)
    feats = torch.randint(-50, 51, (N, C), generator=g).float()      # exact sums
    cnts = torch.bincount(inv, minlength=U)
    say(f"[case] many rows N={N} C={C} U={U}")
    data = T.ScatterData(inv.to(DEV), cnts.to(DEV))
    f = feats.to(DEV)
    s = T.scatter_sum(f, data).cpu()
    want = torch.zeros((U, C)).index_add_(0, inv, feats)
    assert torch.equal(s, want)
    mx, arg = T.scatter_max(f, data)
    wm, wa = orc.scatter_max_first(feats.numpy(), inv.numpy().astype(np.int32), U)
    assert np.array_equal(arg.cpu().numpy(), wa) and bits_equal(mx.cpu().numpy(), wm)
    gup = torch.randint(-5, 6, (U, C), generator=g).float().to(DEV)
    x = f.clone().requires_grad_(True)
    T.scatter_sum(x, data).backward(gup)
    assert torch.equal(x.grad, gup[inv.to(DEV)])


def test_misaligned_views_fall_back_to_narrow_vectors():
    """Tensors whose storage offset breaks 16-byte alignment still work (the launcher picks a
    narrower per-lane vector)."""
    T = tx()
    import scatter_ext
    g = torch.Generator().manual_seed(88)
    N, U, C = 5000, 123, 128
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:U] = torch.arange(U)
    feats = torch.randn((N, C), generator=g)
    data = T.ScatterData(inv.to(DEV), torch.bincount(inv, minlength=U).to(DEV))
    base = torch.empty(N * C + 3, device=DEV)
    for off in (1, 2, 3):
        f = base[off:off + N * C].view(N, C)
        f.copy_(feats)
        assert f.data_ptr() % 16 != 0 and f.is_contiguous()
        say(f"[case] misaligned feats offset {off} floats")
        mx, arg = T.scatter_max(f, data)
        wm, wa = orc.scatter_max_first(feats.numpy(), inv.numpy().astype(np.int32), U)
        assert np.array_equal(arg.cpu().numpy(), wa) and bits_equal(mx.cpu().numpy(), wm)
        gbase = torch.empty(U * C + 3, device=DEV)
        gup = gbase[off:off + U * C].view(U, C)
        gup.copy_(workloads.upstream_grad(U, C, 5))
        gin = scatter_ext.backward(scatter_ext.MAX, gup, arg, *data.backward_args())
        assert bits_equal(gin.cpu().numpy(), orc.max_backward(gup.cpu().numpy(), wa, N))


def test_runs_on_the_current_stream():
    T = tx()
    w = workloads.lidar_sweep(N=200_000, C=64, seed=21)
    inv, cnts, f = w.unq_inv.to(DEV), w.unq_cnts.to(DEV), w.feats.to(DEV)
    ref = T.scatter_max(f, T.ScatterData(inv, cnts))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        data = T.ScatterData(inv, cnts)
        outs = [T.scatter_max(f, data) for _ in range(3)]
        means = [T.scatter_mean(f, data) for _ in range(3)]
    side.synchronize()
    for mx, arg in outs:
        assert torch.equal(mx, ref[0]) and torch.equal(arg, ref[1])
    light = (w.unq_cnts <= data.heavy_threshold).to(DEV)
    assert torch.equal(means[0][light], means[2][light])


def test_hip_graph_capture_and_replay():
    """The forward and backward entry points only launch kernels (no memset node, no
    host synchronisation, scratch re-zeroed by a kernel), so they can be recorded into
    a HIP graph.  Every replay is checked against the eager result, with eager work
    and synchronisations between replays."""
    from torchex_amd._native import scatter_ext
    w = workloads.zipf_contention(N=300_000, C=32, num_ids=700, seed=31)   # every voxel on the atomic path
    w2 = workloads.lidar_sweep(N=200_000, C=64, seed=32)
    for wl in (w, w2):
        N, C, U = wl.N, wl.C, wl.U
        say(f"[case] graph replay {wl.name} N={N} C={C} U={U}")
        inv, cnts = wl.unq_inv.to(DEV), wl.unq_cnts.to(DEV)
        f = wl.feats.to(DEV)
        g = workloads.upstream_grad(U, C, 9).to(DEV)
        data = tx().ScatterData(inv, cnts)
        plan = data.forward_args(C)
        bplan = data.backward_args()

        def run():
            mean, _ = scatter_ext.forward(scatter_ext.MEAN, f, *plan)
            mx, arg = scatter_ext.forward(scatter_ext.MAX, f, *plan)
            g_mean = scatter_ext.backward(scatter_ext.MEAN, g, None, *bplan)
            g_max = scatter_ext.backward(scatter_ext.MAX, g, arg, *bplan)
            return mean, mx, arg, g_mean, g_max

        eager = [t.clone() for t in run()]
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run()                                   # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            captured = run()
        light = (wl.unq_cnts <= data.heavy_threshold).to(DEV)
        for rep in range(3):
            for t in captured:
                t.fill_(7)                          # eager work between replays; stale outputs would show
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            mean, mx, arg, g_mean, g_max = captured
            assert torch.equal(mx, eager[1]) and torch.equal(arg, eager[2]), f"replay {rep}: max"
            assert torch.equal(g_mean, eager[3]) and torch.equal(g_max, eager[4]), f"replay {rep}: backward"
            # voxels reduced through atomics may differ in the last bits between runs
            assert torch.equal(mean[light], eager[0][light]), f"replay {rep}: mean (register path)"
            assert torch.allclose(mean, eager[0], rtol=1e-5, atol=1e-5, equal_nan=True), f"replay {rep}: mean"
            # the scratch table is zero again after every replay
            assert not bool((data.scratch(C) != 0).any()), f"replay {rep}: scratch table not zero"


def test_random_small_shapes_sweep():
    """Seeded sweep over small random problems: row counts, channel widths, voxel counts,
    occupancy profiles (uniform, skewed, with empty voxels, grouped or shuffled) and
    heavy thresholds, each checked like every other case (plan, forward, backward)."""
    rs = np.random.RandomState(1234)
    for case in range(60):
        N = int(rs.choice([1, 2, 7, 15, 16, 17, 63, 64, 65, 129, 500, 1023, 2049, 4000]))
        C = int(rs.choice([1, 2, 3, 4, 5, 8, 12, 16, 31, 32, 33, 64, 100, 128]))
        U = int(rs.randint(1, N + 1))
        kind = case % 4
        if kind == 0:      # uniform ids (some voxels may stay empty)
            ids = rs.randint(0, U, size=N)
        elif kind == 1:    # skewed: most rows in a few voxels
            ids = np.minimum((rs.exponential(scale=max(U / 8.0, 1.0), size=N)).astype(np.int64), U - 1)
        elif kind == 2:    # one long run plus singletons
            ids = np.concatenate([np.zeros(N - N // 3, dtype=np.int64), rs.randint(0, U, size=N // 3)])
        else:              # every id at least once where possible
            ids = np.concatenate([np.arange(min(U, N)), rs.randint(0, U, size=N - min(U, N))])
        ids = np.sort(ids) if case % 3 == 0 else rs.permutation(ids)
        inv = torch.from_numpy(ids.astype(np.int64))
        cnts = torch.bincount(inv, minlength=U)
        feats = torch.from_numpy(rs.standard_normal((N, C)).astype(np.float32))
        if case % 5 == 0:  # plant ties
            feats = torch.round(feats * 2) / 2
        thr = int(rs.choice([16, 17, 33, 64]))
        dtype = [torch.float32, torch.float32, torch.float16, torch.bfloat16][case % 4] if case % 2 else torch.float32
        run_case(f"sweep{case}", feats, inv, cnts, dtype=dtype, grad_seed=case, heavy_threshold=thr)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_subnormal_values_are_kept(dtype):
    """Subnormal inputs are neither flushed on the way in nor on the way out (the
    output conversion of bf16 is a hardware instruction): max returns them bit for
    bit and a two-term sum equals the correctly rounded fp32 sum."""
    T = tx()
    tiny = {torch.float32: [1e-40, -3e-41, 2e-39, 5e-45],
            torch.bfloat16: [1e-40, -3e-41, 2e-39, 5e-45],
            torch.float16: [6e-8, -2e-7, 3e-6, 1e-7]}[dtype]
    v = torch.tensor(tiny, dtype=torch.float32).to(dtype)
    f = v.reshape(4, 1).repeat(1, 8).to(DEV)
    data = T.ScatterData(torch.tensor([0, 0, 1, 1], device=DEV), torch.tensor([2, 2], device=DEV))
    mx, arg = T.scatter_max(f, data)
    s = T.scatter_sum(f, data)
    want_max = torch.stack([torch.maximum(v[0], v[1]), torch.maximum(v[2], v[3])])
    want_sum = torch.stack([(v[0].float() + v[1].float()).to(dtype), (v[2].float() + v[3].float()).to(dtype)])
    for c in range(8):
        assert torch.equal(mx[:, c].cpu().view(torch.int16 if dtype != torch.float32 else torch.int32),
                           want_max.view(torch.int16 if dtype != torch.float32 else torch.int32))
        assert torch.equal(s[:, c].cpu().float(), want_sum.float())
    assert float(want_max.float().abs().min()) > 0.0   # the case really holds subnormals, not zeros


def test_mostly_empty_voxel_grid():
    """Ids scattered over a large dense grid: a million voxels, almost all empty, one
    heavy.  Empty voxels get their rows without owning scratch memory (one scratch row
    per heavy voxel only), and slot allocation does not queue on one counter."""
    U, N, C = 1_000_000, 30_000, 8
    g = torch.Generator().manual_seed(77)
    inv = torch.randint(0, U, (N,), generator=g)
    inv[:500] = 123_456                      # one voxel above the heavy threshold
    cnts = torch.bincount(inv, minlength=U)
    feats = torch.randn((N, C), generator=g)
    data = run_case("mostly_empty", feats, inv, cnts)
    assert data.num_heavy == 1 and data.num_special == int((cnts == 0).sum()) + 1
    assert tuple(data.scratch(C).shape) == (C,)
    # layout the kernels rely on: heavy voxels first, then the empty ones
    ids = data.heavy_ids.cpu()
    assert ids[0].item() == 123_456 and bool((cnts[ids[1:].long()] == 0).all())


def test_long_runs_of_empty_voxels_through_the_general_sequence():
    """CSR offsets from sorted ids when thousands of consecutive voxels are empty: the general
    sequence (here forced by one voxel that holds most of the rows) fills such runs block by
    block.  Offsets, order and the operators against the oracle; first and last voxel empty or
    not, run lengths around the 256-id block size."""
    import time
    g = torch.Generator().manual_seed(91)
    U, C = 3_000_000, 4
    used = torch.tensor([0, 1, 255, 256, 257, 511, 512, 513, 1000, 70_000, 70_255, 70_256, 70_767, 70_768,
                         2_000_000, 2_999_743, 2_999_744, 2_999_999])
    for name, drop in (("ends used", []), ("first and last empty", [0, U - 1])):
        ids = torch.tensor([u for u in used.tolist() if u not in drop])
        crowd = 300_000                                   # one voxel above the bucket kernels' limit
        inv = torch.cat([ids.repeat(3), torch.full((crowd,), 1000)])
        inv = inv[torch.randperm(inv.numel(), generator=g)]
        feats = torch.randint(-4, 5, (inv.numel(), C), generator=g).float()
        t0 = time.perf_counter()
        data = run_case(f"empty runs, {name}", feats, inv, torch.bincount(inv, minlength=U))
        assert data.max_cnt == crowd + 3 and data.num_special == U - ids.numel() + 1
        assert time.perf_counter() - t0 < 60


def test_reference_style_module_calls_reuse_their_plan():
    """scatter_ext.sum / max take only CSR offsets (the reference's signatures).  The
    plan behind a preSum tensor is kept between calls; it is rebuilt when the tensor is
    rewritten in place or used with another row count."""
    import scatter_ext
    scatter_ext.clear_csr_plan_cache()
    sizes = torch.tensor([3, 1, 70, 2, 5, 130, 1, 1, 9], dtype=torch.long)
    U, N, C = sizes.numel(), int(sizes.sum()), 12
    inv = torch.repeat_interleave(torch.arange(U), sizes)
    g = torch.Generator().manual_seed(8)
    feats = torch.randn((N, C), generator=g)
    pre = torch.zeros(U + 1, dtype=torch.int32, device=DEV)
    scatter_ext.getPreSum(inv.int().to(DEV), pre)
    f = feats.to(DEV)
    want = orc.scatter_sum_f64(feats.numpy(), inv.numpy().astype(np.int32), U)
    wm, wa = orc.scatter_max_reforder(feats.numpy(), inv.numpy().astype(np.int32), U)
    for _ in range(3):                                   # first call builds, the others reuse
        out = torch.zeros((U, C), device=DEV)
        scatter_ext.sum(f, pre, out, int(sizes.max()))
        assert np.allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
        mx = torch.zeros((U, C), device=DEV)
        arg = torch.zeros((U, C), device=DEV, dtype=torch.int32)
        scatter_ext.max(f, pre, mx, arg, int(sizes.max()))
        assert np.array_equal(arg.cpu().numpy(), wa) and bits_equal(mx.cpu().numpy(), wm)
    # the same tensor rewritten in place for other voxel sizes: the old plan must not be used
    sizes2 = torch.tensor([100, 1, 1, 2, 5, 10, 1, 1, 100], dtype=torch.long)
    assert int(sizes2.sum()) == N - 1
    inv2 = torch.repeat_interleave(torch.arange(U), sizes2)
    scatter_ext.getPreSum(inv2.int().to(DEV), pre)
    f2 = f[:N - 1].contiguous()
    out = torch.zeros((U, C), device=DEV)
    scatter_ext.sum(f2, pre, out, 100)
    want2 = orc.scatter_sum_f64(feats[:N - 1].numpy(), inv2.numpy().astype(np.int32), U)
    assert np.allclose(out.cpu().numpy(), want2, rtol=1e-5, atol=1e-5)
    # ... and rewritten in place for another grouping of the SAME number of rows and
    # voxels: nothing but the contents of preSum tells the two plans apart
    scatter_ext.clear_csr_plan_cache()
    scatter_ext.getPreSum(inv.int().to(DEV), pre)
    out = torch.zeros((U, C), device=DEV)
    scatter_ext.sum(f, pre, out, int(sizes.max()))           # plan for `sizes` is now cached
    sizes3 = torch.tensor([1, 1, 2, 70, 5, 9, 130, 3, 1], dtype=torch.long)
    assert int(sizes3.sum()) == N and sizes3.numel() == U
    inv3 = torch.repeat_interleave(torch.arange(U), sizes3)
    scatter_ext.getPreSum(inv3.int().to(DEV), pre)
    out = torch.zeros((U, C), device=DEV)
    scatter_ext.sum(f, pre, out, int(sizes3.max()))
    want3 = orc.scatter_sum_f64(feats.numpy(), inv3.numpy().astype(np.int32), U)
    assert np.allclose(out.cpu().numpy(), want3, rtol=1e-5, atol=1e-5)
    wm3, wa3 = orc.scatter_max_reforder(feats.numpy(), inv3.numpy().astype(np.int32), U)
    mx = torch.zeros((U, C), device=DEV)
    arg = torch.zeros((U, C), device=DEV, dtype=torch.int32)
    scatter_ext.max(f, pre, mx, arg, int(sizes3.max()))
    assert np.array_equal(arg.cpu().numpy(), wa3) and bits_equal(mx.cpu().numpy(), wm3)
    # a preSum tensor that is gone takes its plan (and the device memory it pins) with it
    del pre
    pre4 = torch.zeros(U + 1, dtype=torch.int32, device=DEV)
    scatter_ext.getPreSum(inv.int().to(DEV), pre4)
    scatter_ext.sum(f, pre4, torch.zeros((U, C), device=DEV), int(sizes.max()))
    assert scatter_ext.csr_plan_cache_size() == 1
    scatter_ext.clear_csr_plan_cache()


def test_assume_sorted_skips_the_sort_and_is_verified():
    """ScatterData(..., assume_sorted=True) on grouped input (the reference's contract)
    builds the same plan without queueing the sort; an input that is not sorted raises."""
    T = tx()
    w = workloads.lidar_sweep(N=100_000, C=32, seed=41)
    order = torch.sort(w.unq_inv, stable=True)[1]
    inv_s, f_s = w.unq_inv[order].to(DEV), w.feats[order].to(DEV)
    cnts = w.unq_cnts.to(DEV)
    a = T.ScatterData(inv_s, cnts)
    b = T.ScatterData(inv_s, cnts, assume_sorted=True)
    assert a.is_sorted and b.is_sorted and b.perm is None
    for name in ("preSum", "seg", "slot_of", "heavy_ids"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name
    assert (a.max_cnt, a.num_special, a.num_heavy) == (b.max_cnt, b.num_special, b.num_heavy)
    ma, aa = T.scatter_max(f_s, a)
    mb, ab = T.scatter_max(f_s, b)
    assert torch.equal(ma, mb) and torch.equal(aa, ab)
    assert torch.equal(T.scatter_mean(f_s, a), T.scatter_mean(f_s, b))
    with pytest.raises(RuntimeError, match="declared sorted"):
        T.ScatterData(w.unq_inv.to(DEV), cnts, assume_sorted=True)


# ------------------------------------------- drop-in behaviour on grouped rows --

@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_default_scatter_max_on_grouped_tie_heavy_rows_is_the_reference_winner(dtype):
    """``from torchex import scatter_max, ScatterData`` on rows grouped by voxel -- the only
    input the reference defines -- reports the row the reference kernel reports, also where
    many rows tie (values 0, 1, 2 only; block widths 32 .. 1024, several rows per thread)."""
    import torchex
    sizes = [5, 17, 31, 32, 33, 64, 1, 2, 100, 7, 700, 1024, 900, 65, 2050, 1500, 40, 4996, 1025, 3000] * 3
    C = 24
    feats, inv, cnts = _tie_heavy_groups(77, sizes, C)
    U = len(sizes)
    inv32 = inv.numpy().astype(np.int32)
    want_max, want_arg = orc.scatter_max_reforder(feats.numpy(), inv32, U)
    assert (want_arg != orc.scatter_max_first(feats.numpy(), inv32, U)[1]).any()
    data = torchex.ScatterData(inv.to(DEV), cnts.to(DEV))
    mx, arg = torchex.scatter_max(feats.to(dtype).to(DEV), data)
    assert mx.dtype == dtype
    assert np.array_equal(arg.cpu().numpy(), want_arg)
    assert bits_equal(mx.float().cpu().numpy(), want_max)


def test_reference_harness_form_with_torch_timer(capsys):
    """The reference's own test loop (test/test_scatter.py:27-51): ScatterData built outside
    the timers, ``with timer.timing(name)`` around each operator call, running means printed
    every ``freq`` calls; all three modes (the reference enables 'sum' only), checked against
    the closed forms of its data instead of torch_scatter."""
    from torchex import ScatterData, TorchTimer, scatter_max, scatter_mean, scatter_sum
    freq = 5
    timer_torchex = TorchTimer(freq)
    w = workloads.reference_test_groups(channel=128, num_group=60)
    feat, unq_inv, unq_cnts = w.feats.to(DEV), w.unq_inv.to(DEV), w.unq_cnts.to(DEV)
    data = ScatterData(unq_inv, unq_cnts)
    n = w.unq_cnts.double().unsqueeze(1)
    starts = torch.cumsum(w.unq_cnts, 0) - w.unq_cnts
    col = w.feats[:, 0]
    argpos = torch.stack([s + torch.argmax(col[s:s + c]) for s, c in zip(starts.tolist(), w.unq_cnts.tolist())])
    for mode in ("sum", "mean", "max"):
        for _ in range(2 * freq):
            with timer_torchex.timing(f"Torchex.scatter_{mode}"):
                if mode == "sum":
                    ans2 = scatter_sum(feat, data)
                elif mode == "mean":
                    ans2 = scatter_mean(feat, data)
                else:
                    ans2, arg2 = scatter_max(feat, data)
            want = {"sum": n * (n - 1) / 2, "mean": (n - 1) / 2, "max": n - 1}[mode]
            assert torch.equal(ans2.cpu().double(), want.expand(-1, 128))
            if mode == "max":
                assert torch.equal(arg2.cpu().long(), argpos.unsqueeze(1).expand(-1, 128))
    lines = [l for l in capsys.readouterr().out.splitlines() if l.startswith("Average time cost of Torchex.")]
    assert len(lines) == 6                      # 3 modes x (10 calls / freq 5)
    for l in lines:
        assert l.endswith("ms") and float(l.split(": ")[1][:-2]) > 0.0
    t = timer_torchex.timer_dict["Torchex.scatter_max"]
    assert t.exe_counter == 0 and t.print_freq == freq     # reset after each print


def test_get_presum_against_the_reference_restatement():
    """scatter_ext.getPreSum / getPreSum() against the oracle's restatement of the reference
    kernel (scatter_kernel.cu:85-100), including a tail of equal ids and single-row groups."""
    import scatter_ext
    T = tx()
    rs = np.random.RandomState(3)
    for sizes in ([1], [5], [1, 1, 1], [3, 1, 70, 2, 5, 130, 1, 1, 9], rs.randint(1, 400, size=3000).tolist()):
        inv = np.repeat(np.arange(len(sizes)), sizes).astype(np.int32)
        want = orc.get_presum_ref(inv)
        pre = torch.zeros(len(sizes) + 1, dtype=torch.int32, device=DEV)
        scatter_ext.getPreSum(torch.from_numpy(inv).to(DEV), pre)
        assert np.array_equal(pre.cpu().numpy(), want)
        assert np.array_equal(T.getPreSum(torch.from_numpy(inv).long().to(DEV)).cpu().numpy(), want)


def test_concurrent_streams_do_not_share_a_heavy_voxel_table():
    """Forwards of one ScatterData queued on two streams at the same time: each stream gets a
    heavy-voxel table of its own, so the results equal the single-stream ones."""
    T = tx()
    from torchex_amd._native import scatter_ext
    w = workloads.zipf_contention(N=400_000, C=32, num_ids=300, seed=5)     # every voxel heavy
    inv, cnts = w.unq_inv.to(DEV), w.unq_cnts.to(DEV)
    fa = w.feats.to(DEV)
    fb = (w.feats * 0.5 + 1.0).to(DEV)
    data = T.ScatterData(inv, cnts)
    data.path = scatter_ext.PATH_VOXEL_ORDER     # the kernels that merge heavy voxels through the table
    assert data.num_heavy == w.U
    ref_a, ref_b = T.scatter_max(fa, data), T.scatter_max(fb, data)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    for _ in range(6):
        with torch.cuda.stream(s1):
            outs_a.append(T.scatter_max(fa, data))
        with torch.cuda.stream(s2):
            outs_b.append(T.scatter_max(fb, data))
    torch.cuda.synchronize()
    for mx, arg in outs_a:
        assert torch.equal(mx, ref_a[0]) and torch.equal(arg, ref_a[1])
    for mx, arg in outs_b:
        assert torch.equal(mx, ref_b[0]) and torch.equal(arg, ref_b[1])
    assert len(data._scratch) == 3 and all(not bool((t != 0).any()) for t in data._scratch.values())


# ------------------------------------------------ few voxels: the row-order kernels --

def _kernel_of(data, feats, backward, op):
    from torchex_amd._native import scatter_ext
    return scatter_ext.kernel_name(backward, op, feats, data.num_total, data.num_unq, True)


def test_zipf_contention_takes_the_table_kernels_and_both_paths_agree():
    """The contention workload (1024 voxels, 64-byte rows) is reduced in row order through
    per-workgroup LDS tables; forcing the voxel-order kernels on the same plan gives the same
    max / arg / gradients bit for bit and sums within tolerance."""
    from torchex_amd._native import scatter_ext
    T = tx()
    w = workloads.zipf_contention()
    f = w.feats.to(DEV)
    data = T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV))
    assert _kernel_of(data, f, False, scatter_ext.MAX).startswith("table_fwd_kernel")
    assert _kernel_of(data, f, True, scatter_ext.MAX).startswith("table_bwd_kernel")
    g = workloads.upstream_grad(w.U, w.C, 3).to(DEV)
    res = {}
    for path in (scatter_ext.PATH_TABLE, scatter_ext.PATH_VOXEL_ORDER):
        data.path = path
        x = f.clone().requires_grad_(True)
        mx, arg = T.scatter_max(x, data)
        mx.backward(g)
        gmax = x.grad.clone()
        x.grad = None
        mean = T.scatter_mean(x, data)
        mean.backward(g)
        res[path] = (mx.detach(), arg, gmax, mean.detach(), x.grad.clone(), T.scatter_sum(f, data))
    a, b = res[scatter_ext.PATH_TABLE], res[scatter_ext.PATH_VOXEL_ORDER]
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])
    assert torch.equal(a[4], b[4])
    sabs = torch.zeros((w.U, w.C), device=DEV).index_add_(0, w.unq_inv.to(DEV), f.abs())
    assert bool(((a[5] - b[5]).abs() <= 2e-5 * sabs).all())
    assert bool(((a[3] - b[3]).abs() <= 2e-5 * sabs / data.unq_cnts).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("C", [1, 2, 3, 4, 6, 10, 16, 20, 24, 64])
def test_table_kernels_channel_widths_and_dtypes(C, dtype):
    from torchex_amd._native import scatter_ext
    g = torch.Generator().manual_seed(500 + C)
    N, U = 40_000, 37
    inv = torch.randint(0, U, (N,), generator=g)
    inv[inv == 5] = 6                       # an empty voxel
    inv[:3000] = 11                         # a crowded one
    feats = torch.randn((N, C), generator=g)
    feats[torch.rand((N, C), generator=g) < 0.1] = 0.5      # ties
    run_case(f"table C={C}", feats, inv, torch.bincount(inv, minlength=U), dtype=dtype,
             path=scatter_ext.PATH_TABLE)


def test_table_kernels_special_values_and_grouped_rows():
    from torchex_amd._native import scatter_ext
    g = torch.Generator().manual_seed(9)
    N, U, C = 30_000, 24, 8
    inv = torch.randint(0, U, (N,), generator=g)
    f = torch.randn((N, C), generator=g)
    f[torch.rand((N, C), generator=g) < 0.05] = float("nan")
    f[torch.rand((N, C), generator=g) < 0.05] = float("-inf")
    f[torch.rand((N, C), generator=g) < 0.02] = float("inf")
    f[torch.rand((N, C), generator=g) < 0.05] = -0.0
    f[torch.rand((N, C), generator=g) < 0.05] = 0.0
    f[inv == 0] = float("nan")
    f[inv == 1] = float("-inf")
    f[inv == 2] = -0.0
    rows3 = torch.nonzero(inv == 3).flatten()
    f[rows3] = -0.0
    f[rows3[len(rows3) // 2:]] = 0.0        # first maximal row holds -0.0: its bits are the result
    T = tx()
    cnts = torch.bincount(inv, minlength=U)
    for path in (scatter_ext.PATH_TABLE, scatter_ext.PATH_VOXEL_ORDER):
        data = T.ScatterData(inv.to(DEV), cnts.to(DEV))
        data.path = path
        mx, arg = T.scatter_max(f.to(DEV), data)
        wm, wa = orc.scatter_max_first(f.numpy(), inv.numpy().astype(np.int32), U)
        assert np.array_equal(arg.cpu().numpy(), wa), path
        assert bits_equal(mx.cpu().numpy(), wm), path
        assert np.signbit(mx.cpu().numpy()[2]).all() and np.signbit(mx.cpu().numpy()[3]).all()
        s = T.scatter_sum(f.to(DEV), data).cpu().numpy()
        ws = orc.scatter_sum_f64(f.numpy(), inv.numpy().astype(np.int32), U)
        assert np.array_equal(np.isnan(s), np.isnan(ws)) and np.array_equal(np.isinf(s), np.isinf(ws))
    # grouped rows (no permutation): the first-row rule through the table kernels; the
    # reference's tie rule needs voxel order and says so when the table kernels are forced
    order = torch.argsort(inv, stable=True)
    fin = torch.randint(-3, 4, (N, C), generator=g).float()
    run_case("table grouped", fin[order], inv[order], cnts, max_tie_rule="first", path=scatter_ext.PATH_TABLE)
    dref = T.ScatterData(inv[order].to(DEV), cnts.to(DEV))
    assert dref.max_tie_rule == "reference"
    dref.path = scatter_ext.PATH_TABLE
    with pytest.raises(RuntimeError, match="unsupported"):
        T.scatter_max(fin[order].to(DEV), dref)
    # many voxels: the table kernels do not apply
    w = workloads.lidar_sweep(N=50_000, C=16, seed=4)
    dl = T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV))
    dl.path = scatter_ext.PATH_TABLE
    with pytest.raises(RuntimeError, match="unsupported"):
        T.scatter_sum(w.feats.to(DEV), dl)


def test_plan_with_crowded_buckets_and_the_general_fallback():
    """Index preparation splits the ids into buckets of consecutive voxels.  A bucket with far
    more rows than the others is cut into slices of 2048 rows, one workgroup each; beyond 64
    slices the slices get longer; a bucket of more than 262,144 rows sends the whole plan to the
    general radix passes.  All give the same plan as the oracle."""
    g = torch.Generator().manual_seed(13)
    U, C = 5000, 8                      # 13 bits of id: buckets of 32 consecutive voxels
    for name, crowd in (("shared bucket", 100_000), ("long slices", 200_000), ("giant bucket", 300_000)):
        N = crowd + 120_000
        inv = torch.randint(0, U, (N,), generator=g)
        hot = torch.randperm(N, generator=g)[:crowd]
        inv[hot] = torch.randint(3, 9, (crowd,), generator=g)      # voxels 3..8 take `crowd` rows
        inv[:U] = torch.arange(U)
        feats = torch.randint(-4, 5, (N, C), generator=g).float()
        data = run_case(name, feats, inv, torch.bincount(inv, minlength=U))
        assert data.max_cnt > crowd // 7 and data.perm is not None


def test_element_offsets_beyond_2_to_31():
    """Maximum sizes: more than 2^31 elements in feats (N * C), in the input gradient and in
    out / arg (U * C), where the reference's 32-bit `feat_idx * num_dim + dim`
    (scatter_kernel.cu:115,147) wraps.  The first 16.9 M rows are singletons in shuffled voxel
    order, so their outputs are the rows themselves; the last 600 k rows, which lie past element
    2^31, fall into 100 k voxels of their own at the top of the id range and must come out as the
    same rows do when reduced alone, and that small problem is checked against the oracle."""
    T = tx()
    H, TAIL, UT, C = 16_900_000, 600_000, 100_000, 128
    N, U = H + TAIL, H + UT
    assert N * C > 2 ** 31 and U * C > 2 ** 31 and H * C > 2 ** 31
    say(f"[case] offsets beyond 2^31: N={N} U={U} C={C} fp16")
    g = torch.Generator(device=DEV).manual_seed(31)
    feats = torch.randn((N, C), generator=g, device=DEV, dtype=torch.float16)
    head_ids = torch.randperm(H, generator=g, device=DEV)
    gc = torch.Generator().manual_seed(32)
    tail_ids = torch.randint(0, UT, (TAIL,), generator=gc)
    inv = torch.cat([head_ids, tail_ids.to(DEV) + H])
    cnts = torch.cat([torch.ones(H, dtype=torch.int64), torch.bincount(tail_ids, minlength=UT)]).to(DEV)
    data = T.ScatterData(inv, cnts)
    assert data.num_unq == U and data.perm is not None and data.max_cnt == int(cnts.max())

    # the tail alone: a small problem of its own, checked against the oracle
    ft = feats[H:].contiguous()
    run_case("tail alone", ft.float().cpu(), tail_ids, torch.bincount(tail_ids, minlength=UT), dtype=torch.float16)
    dt = T.ScatterData(tail_ids.to(DEV), torch.bincount(tail_ids, minlength=UT).to(DEV))
    gt = torch.randn((U, C), generator=g, device=DEV, dtype=torch.float16)

    def same_bits(a, b):   # equal bit patterns (NaN included: the mean of an empty voxel)
        return torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16))

    fg = feats.requires_grad_(True)
    ftg = ft.requires_grad_(True)
    for name, op in (("sum", T.scatter_sum), ("mean", T.scatter_mean), ("max", T.scatter_max)):
        say(f"[case] offsets beyond 2^31: {name}")
        res, res_t = op(fg, data), op(ftg, dt)
        out, out_t = (res[0], res_t[0]) if name == "max" else (res, res_t)
        # singletons: the voxel's row itself (sum of one, mean over one, max of one)
        assert same_bits(out[:H].index_select(0, head_ids), feats[:H].detach()), f"{name}: singleton rows"
        if name == "max":
            assert same_bits(out[H:], out_t), f"{name}: voxels of the rows past element 2^31"
        else:
            # a voxel whose rows straddle two lane groups' chunks is summed as (earlier part) +
            # (later part), and where the chunk borders fall depends on the rows in front: the
            # fp32 sums of the two problems can differ in their last bit, which reaches the
            # fp16 output in a handful of the 12.8 M elements (by one unit in the last place)
            a, b = out[H:].detach().float(), out_t.detach().float()
            both_nan = torch.isnan(a) & torch.isnan(b)
            differs = (out[H:].contiguous().view(torch.int16) != out_t.contiguous().view(torch.int16)) & ~both_nan
            assert int(differs.sum()) <= 64, f"{name}: {int(differs.sum())} elements differ"
            assert torch.allclose(a, b, rtol=2.0 ** -10, atol=2.0 ** -24, equal_nan=True), f"{name}: rows past element 2^31"
        if name == "max":
            arg, arg_t = res[1], res_t[1]
            assert torch.equal(arg[:H].index_select(0, head_ids),
                               torch.arange(H, device=DEV, dtype=torch.int32)[:, None].expand(H, C))
            assert torch.equal(arg[H:], torch.where(arg_t >= 0, arg_t + H, arg_t))
        fg.grad = None
        ftg.grad = None
        out.backward(gt)
        out_t.backward(gt[H:])
        assert same_bits(fg.grad[H:], ftg.grad), f"{name} backward: rows past element 2^31"
        # a singleton's gradient row is its voxel's upstream row
        assert same_bits(fg.grad[:H], gt[:H].index_select(0, head_ids)), f"{name} backward: singleton rows"
        del res, res_t, out, out_t
    fg.grad = None


def test_python_function_classes_and_module_level_operators_agree():
    """`scatter_sum / scatter_mean / scatter_max` run an autograd node written in C++; the
    `Scatter*Function` classes with the reference's names (scatter_op.py:24-111) are Python
    `autograd.Function`s over the same launches.  Same outputs, same gradients, `arg` carries
    no gradient on either, a call under `no_grad` records nothing, and a gradient that reaches
    only `arg`'s partner of a tuple still flows."""
    T = tx()
    from torchex_amd import scatter_op as so
    w = workloads.lidar_sweep(N=60_000, C=48, seed=21)
    data = T.ScatterData(w.unq_inv.to(DEV), w.unq_cnts.to(DEV))
    g = workloads.upstream_grad(w.U, w.C, 5).to(DEV)
    for fast, cls in ((T.scatter_sum, so.ScatterSumFunction), (T.scatter_mean, so.ScatterMeanFunction),
                      (T.scatter_max, so.ScatterMaxFunction)):
        fa = w.feats.to(DEV).requires_grad_(True)
        fb = w.feats.to(DEV).requires_grad_(True)
        ra, rb = fast(fa, data), cls.apply(fb, data)
        if cls is so.ScatterMaxFunction:
            assert isinstance(ra, tuple) and len(ra) == 2
            assert torch.equal(ra[1], rb[1]) and ra[1].dtype == torch.int32
            assert not ra[1].requires_grad and not rb[1].requires_grad
            ra, rb = ra[0], rb[0]
        assert ra.requires_grad and ra.grad_fn is not None
        assert torch.equal(ra, rb)
        ra.backward(g)
        rb.backward(g)
        assert torch.equal(fa.grad, fb.grad)
        with torch.no_grad():
            rn = fast(fa, data)
        rn = rn[0] if isinstance(rn, tuple) else rn
        assert not rn.requires_grad and torch.equal(rn, ra)
    # part of a larger graph, twice through the same ScatterData
    f = w.feats.to(DEV).requires_grad_(True)
    mx, _ = T.scatter_max(f * 2.0, data)
    loss = (mx * g).sum() + (T.scatter_mean(f, data) * g).sum()
    loss.backward()
    f2 = w.feats.to(DEV).requires_grad_(True)
    mx2, _ = so.ScatterMaxFunction.apply(f2 * 2.0, data)
    ((mx2 * g).sum() + (so.ScatterMeanFunction.apply(f2, data) * g).sum()).backward()
    assert torch.equal(f.grad, f2.grad)
    # features that need no gradient: no node at all
    out = T.scatter_sum(w.feats.to(DEV), data)
    assert not out.requires_grad and out.grad_fn is None
