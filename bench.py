#!/usr/bin/env python3
"""Benchmark of the voxel scatter path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic points:
``scatter_mean`` forward+backward and ``scatter_max`` (+argmax) forward+backward,
through the public Python API (autograd included), with ``ScatterData`` built
beforehand (the reference's own timing also keeps ``ScatterData`` construction
outside the timed region, ``test/test_scatter.py:24,38-44``).  The headline workload is
the LiDAR-like sweep: N = 1,000,000 points, C = 128 fp32 features, 0.2 m voxels.
Inputs are resident in HBM before the timed region starts.

``value`` is points per second per operator pass: ``2 * N / t_step`` (each step
pushes the N points through two operators' forward+backward).  Per-kernel
durations are measured inside a second pass over the same steps, with a HIP event
between the four entry-point calls; per-operator times, GB/s and roofline fractions
derived from them are in ``per_kernel`` / ``per_op``.

``other_configs`` holds the same measurements (``--other-steps`` timed steps each, mean,
median and minimum per kernel) for the other configurations: the uniform box (with the
same step on the host cores next to it), the half-precision sweep (fp16, bf16), the Zipf
contention case, the four-sweep batch and the pillar binning of the sweep (the same
points in 0.2 m x 0.2 m columns: the heavy-tailed occupancy, two thirds of the points in
voxels that are split across wavefronts).  ``ms_per_step_graph`` is the step's four
entry-point calls replayed from a HIP graph (no host work per call).

Prints ONE JSON line on stdout.
"""
import argparse
import ctypes
import hashlib
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
TORCH_DTYPE = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
DTYPE_CODE = {"f32": 0, "f16": 1, "bf16": 2}
OP_CODE = {"sum": 0, "mean": 1, "max": 2, "max_reftie": 3}
WORKLOADS = ("lidar_sweep", "uniform_box", "zipf_contention", "multi_sweep", "reference_test_groups",
             "lidar_pillars")
# (workload, dtype) of the `other_configs` block, after the headline workload
OTHER_CONFIGS = (("uniform_box", "f32"), ("lidar_sweep", "f16"), ("lidar_sweep", "bf16"),
                 ("zipf_contention", "f32"), ("multi_sweep", "f32"), ("lidar_pillars", "f32"),
                 ("lidar_pillars", "f16"))
# HBM bytes per launch measured with rocprofv3 counters (FETCH_SIZE, WRITE_SIZE), per
# (workload, dtype, kernel), together with a digest of the kernel sources they were
# measured on: figures are reported only while the sources still match.
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_table.json")
KERNEL_SOURCES = ("torchex_amd/csrc/scatter_kernels.hip", "torchex_amd/csrc/table_kernels.hip",
                  "torchex_amd/csrc/txs_common.h")


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--kernel-iters", type=int, default=50, help="launches per per-kernel timing loop")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-frontend", action="store_true", help="skip the front-end timings")
    p.add_argument("--no-other-configs", action="store_true",
                   help="measure the selected workload only (profiles of one workload use this)")
    p.add_argument("--other-steps", type=int, default=50, help="timed steps per entry of other_configs")
    p.add_argument("--other-warmup", type=int, default=10, help="warm-up steps per entry of other_configs")
    p.add_argument("--sorted-input", action="store_true",
                   help="also time the step on the same points delivered grouped by voxel "
                        "(off by default so that a profile of the default command holds one "
                        "population of launches per kernel)")
    p.add_argument("--isolated", action="store_true",
                   help="also time each step kernel in a back-to-back loop of its own")
    p.add_argument("--points", type=int, default=1_000_000)
    p.add_argument("--channels", type=int, default=128)
    p.add_argument("--workload", default="lidar_sweep", choices=WORKLOADS,
                   help="lidar_sweep (default) is the workload the headline metric is quoted on; the "
                        "others run at their own fixed sizes and ignore --points/--channels")
    p.add_argument("--dtype", default="f32", choices=tuple(TORCH_DTYPE))
    return p.parse_args()


def event_ms(fn, iters, warm=5):
    """Average duration of ``fn`` over ``iters`` back-to-back calls, measured with
    HIP events recorded on the stream the kernels are launched on."""
    for _ in range(warm):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def cpu_baseline(w, g_mean, g_max, budget_s=12.0):
    """The same step with stock torch CPU ops (scatter_reduce / index_add / gather) on
    the host cores: a bounded sample of the same workload (about ``budget_s`` seconds of
    multi-threaded steps, then one step on one thread and one of the C oracle)."""
    from oracle import torch_oracle as tor
    threads = os.cpu_count() or 1
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    tor.step_mean_max(w.feats, w.unq_inv, w.unq_cnts, g_mean, g_max)   # warm-up
    iters, t0 = 0, time.perf_counter()
    while iters < 3 or (time.perf_counter() - t0 < budget_s and iters < 40):
        tor.step_mean_max(w.feats, w.unq_inv, w.unq_cnts, g_mean, g_max)
        iters += 1
    dt = (time.perf_counter() - t0) / iters
    used = torch.get_num_threads()
    torch.set_num_threads(1)          # one step on a single core, for scale
    t1 = time.perf_counter()
    tor.step_mean_max(w.feats, w.unq_inv, w.unq_cnts, g_mean, g_max)
    dt1 = time.perf_counter() - t1
    torch.set_num_threads(used)
    # the C restatement of the reference's algorithm (one core), one step for scale
    from oracle import c_oracle as orc
    import numpy as np
    f32, inv32 = w.feats.numpy(), w.unq_inv.numpy().astype(np.int32)
    cnt = w.unq_cnts.numpy()
    t2 = time.perf_counter()
    orc.mean_from_sum(orc.scatter_sum_f64(f32, inv32, w.U), cnt)
    orc.mean_backward(g_mean.numpy(), np.maximum(cnt, 1), inv32)
    _, arg = orc.scatter_max_first(f32, inv32, w.U)
    orc.max_backward(g_max.numpy(), arg, w.N)
    dt2 = time.perf_counter() - t2
    return {"value": 2 * w.N / dt, "unit": "points/s", "cores": used,
            "kind": "port", "ms_per_step": dt * 1e3, "single_thread_ms_per_step": dt1 * 1e3,
            "c_oracle_single_thread_ms_per_step": dt2 * 1e3,
            "sample": f"{iters} full steps (N={w.N}, C={w.C}) of torch.scatter_reduce/index_add/gather on CPU "
                      f"with {used} threads, then 1 step with 1 thread, then 1 step of the C oracle on 1 core"}


def instrumented_steps(scatter_ext, f, g_mean, g_max, plan, bplan, steps, warmup):
    """Duration (ms) of each of the step's four entry-point calls, issued in step order with
    a HIP event between them: (mean per call, {median, min} per call)."""
    names = ("mean_fwd", "mean_bwd", "max_fwd", "max_bwd")

    def raw_step(ev=None):
        rec = (lambda i: ev[i].record()) if ev is not None else (lambda i: None)
        rec(0)
        scatter_ext.forward(scatter_ext.MEAN, f, *plan)
        rec(1)
        scatter_ext.backward(scatter_ext.MEAN, g_mean, None, *bplan)
        rec(2)
        _, a2 = scatter_ext.forward(scatter_ext.MAX, f, *plan)
        rec(3)
        scatter_ext.backward(scatter_ext.MAX, g_max, a2, *bplan)
        rec(4)

    for _ in range(max(warmup, 1)):
        raw_step()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(steps)]
    torch.cuda.synchronize()
    for e in evs:
        raw_step(e)
    torch.cuda.synchronize()
    per = {n: sorted(e[i].elapsed_time(e[i + 1]) for e in evs) for i, n in enumerate(names)}
    mean = {n: sum(v) / len(v) for n, v in per.items()}
    spread = {n: {"median_ms": v[len(v) // 2], "min_ms": v[0]} for n, v in per.items()}
    return mean, spread


def graph_step_ms(scatter_ext, f, g_mean, g_max, plan, bplan, steps, warmup):
    """The step's four entry-point calls recorded once into a HIP graph and replayed: what
    the step costs when the host's per-call work (argument checks, output allocation,
    launches) is taken out.  The entry points only launch kernels, so they capture."""
    def raw_step():
        scatter_ext.forward(scatter_ext.MEAN, f, *plan)
        scatter_ext.backward(scatter_ext.MEAN, g_mean, None, *bplan)
        _, a2 = scatter_ext.forward(scatter_ext.MAX, f, *plan)
        scatter_ext.backward(scatter_ext.MAX, g_max, a2, *bplan)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        raw_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        raw_step()
    for _ in range(max(warmup, 1)):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    del graph
    return ms


def frontend_timings(T, workloads, dev, N):
    """Wall-clock timings of the callers either side of the scatter operators (voxel keys,
    unique + plan, points-in-boxes, coordinate hash) on LiDAR-like keys."""
    # keys -> (unique, inverse, counts) + plan.  torch.unique followed by ScatterData
    # sorts twice; ScatterData.from_keys sorts once.
    keys_cpu, key_bound = workloads._lidar_keys(N, torch.Generator().manual_seed(2))
    keys = keys_cpu.to(dev)

    def wall_ms(fn, iters=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / iters * 1e3

    def torch_unique_then_plan():
        _, i2, c2 = torch.unique(keys, return_inverse=True, return_counts=True)
        return T.ScatterData(i2, c2)

    frontend = {
        "torch_unique_plus_ScatterData_ms": wall_ms(torch_unique_then_plan),
        "ScatterData_from_keys_ms": wall_ms(lambda: T.ScatterData.from_keys(keys, key_bound)),
    }
    pts = (torch.rand((N, 4), generator=torch.Generator().manual_seed(5)) * 150.0 - 75.0).to(dev)
    pts[:, 2] = pts[:, 2] * (6.0 / 150.0) + 1.0
    vs_t = torch.tensor([0.2, 0.2, 0.2], device=dev)
    lo_t = torch.tensor([-75.0, -75.0, -2.0], device=dev)
    frontend["voxelize_ms"] = wall_ms(lambda: T.voxelize(pts, [0.2, 0.2, 0.2], [-75, -75, -2, 75, 75, 4]), 20)
    frontend["torch_div_floor_voxelize_ms"] = wall_ms(
        lambda: torch.div(pts[:, :3] - lo_t[None, :], vs_t[None, :], rounding_mode="floor").int(), 20)
    i2 = torch.unique(keys, return_inverse=True)[1]
    frontend["ingroup_inds_ms"] = wall_ms(lambda: T.ingroup_inds(i2))
    frontend["ScatterData_from_points_ms"] = wall_ms(
        lambda: T.ScatterData.from_points(pts, [0.2, 0.2, 0.2], [-75, -75, -2, 75, 75, 4]))

    # the other callers of the path: points-in-boxes producer and the coordinate hash
    gb = torch.Generator().manual_seed(11)
    nb = 200
    rois = torch.zeros((nb, 7))
    rois[:, 0:2] = torch.rand((nb, 2), generator=gb) * 140 - 70
    rois[:, 3:6] = torch.rand((nb, 3), generator=gb) * 4 + 1
    rois[:, 6] = torch.rand((nb,), generator=gb) * 6.283
    rois = rois.to(dev)
    p3 = pts[:200_000, :3].contiguous()
    frontend["dynamic_point_pool_200boxes_200kpts_ms"] = wall_ms(
        lambda: T.dynamic_point_pool(rois, p3, [0.5, 0.5, 0.2], 512, 200_000), 10)
    hk = torch.unique(keys).int()
    hv = torch.arange(hk.numel(), device=dev, dtype=torch.int32)
    table = T.grid_hash_build(hk, hv)
    k32 = keys.int()
    frontend["grid_hash_build_%dkeys_ms" % hk.numel()] = wall_ms(lambda: T.grid_hash_build(hk, hv), 20)
    frontend["grid_hash_probe_1M_ms"] = wall_ms(lambda: T.grid_hash_probe(k32, table), 20)
    # bytes each call has to move at least (inputs read once, outputs written once), and the
    # rate that makes at the wall-clock time above: these calls are short sequences of kernels
    # with one or two host reads, so the rates say how far launch and latency are from mattering
    # less than the bytes, not how well a kernel streams
    U = int(hk.numel())
    mb = {
        "voxelize": N * (16 + 12 + 4),                      # xyz(+1) in; coors and keys out
        "ScatterData_from_keys": N * (8 + 4 + 4 + 4) + U * (4 + 4 + 8 + 4),  # keys; inv, perm, seg; offsets, keys, counts, slots
        "ingroup_inds": N * (8 + 8),
        "grid_hash_build_%dkeys" % U: U * (4 + 4) + int(table.numel()) * 4,
        "grid_hash_probe_1M": N * (4 + 4 + 8),              # key in, value out, at least one table slot read
    }
    frontend["algorithmic_MB"] = {k: round(v / 1e6, 2) for k, v in mb.items()}
    frontend["GBps_at_wall_clock"] = {k: round(v / 1e6 / frontend[k + "_ms"], 1) for k, v in mb.items()}
    return frontend


def frontend_cpu(workloads, N):
    """The CPU side of the same front-end calls, once each on the host (one core unless the
    torch op threads itself): torch.unique and the floor division as the reference's callers
    run them, and the oracle's restatements of the other operators."""
    import numpy as np
    from oracle import c_oracle as orc
    keys_cpu, key_bound = workloads._lidar_keys(N, torch.Generator().manual_seed(2))

    def once_ms(fn):
        t = time.perf_counter()
        r = fn()
        return (time.perf_counter() - t) * 1e3, r

    out = {}
    out["torch_unique_inverse_counts_ms"], (unq, inv, _) = once_ms(
        lambda: torch.unique(keys_cpu, return_inverse=True, return_counts=True))
    pts = torch.rand((N, 4), generator=torch.Generator().manual_seed(5)) * 150.0 - 75.0
    pts[:, 2] = pts[:, 2] * (6.0 / 150.0) + 1.0
    lo_t, vs_t = torch.tensor([-75.0, -75.0, -2.0]), torch.tensor([0.2, 0.2, 0.2])
    out["torch_div_floor_voxelize_ms"], _ = once_ms(
        lambda: torch.div(pts[:, :3] - lo_t[None, :], vs_t[None, :], rounding_mode="floor").int())
    out["ingroup_inds_ms"], _ = once_ms(lambda: orc.ingroup_inds(inv.numpy()))
    gb = torch.Generator().manual_seed(11)
    nb = 200
    rois = torch.zeros((nb, 7))
    rois[:, 0:2] = torch.rand((nb, 2), generator=gb) * 140 - 70
    rois[:, 3:6] = torch.rand((nb, 3), generator=gb) * 4 + 1
    rois[:, 6] = torch.rand((nb,), generator=gb) * 6.283
    p3 = pts[:200_000, :3].contiguous().numpy()
    out["dynamic_point_pool_200boxes_200kpts_ms"], _ = once_ms(
        lambda: orc.dynamic_point_pool(rois.numpy(), p3, [0.5, 0.5, 0.2], 512, 200_000))
    hk = unq.numpy().astype(np.int32)
    hv = np.arange(hk.shape[0], dtype=np.int32)
    out["grid_hash_build_%dkeys_ms" % hk.shape[0]], table = once_ms(lambda: orc.grid_hash_build(hk, hv))
    out["grid_hash_probe_1M_ms"], _ = once_ms(lambda: orc.grid_hash_probe(keys_cpu.numpy().astype(np.int32), table))
    out["kind"] = "port"
    out["sample"] = "one call each on one host core (the torch ops: torch's own threading)"
    return out


class KernelNames:
    """Asks the library which kernel instantiation it launches for given extents."""

    def __init__(self):
        from torchex_amd import _native
        self.lib = _native.cabi()
        self.lib.txs_kernel_name.restype = ctypes.c_int

    def __call__(self, key, dtype, N, C, U):
        op, direction = key.rsplit("_", 1)
        buf = ctypes.create_string_buffer(64)
        rc = self.lib.txs_kernel_name(ctypes.c_int(direction == "bwd"), ctypes.c_int(OP_CODE[op]),
                                      ctypes.c_int(DTYPE_CODE[dtype]), ctypes.c_int64(N), ctypes.c_int64(C),
                                      ctypes.c_int64(U), ctypes.c_int64(16), ctypes.c_int(1), buf,
                                      ctypes.c_int64(64))
        return buf.value.decode() if rc == 0 else None


def load_traffic_table():
    """Measured HBM bytes per launch, or {} with a note when the kernel sources have changed
    since they were measured."""
    if not os.path.exists(TRAFFIC_TABLE):
        return {}, "no traffic table"
    with open(TRAFFIC_TABLE) as f:
        tab = json.load(f)
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    if h.hexdigest() != tab.get("kernel_sources_sha256"):
        return {}, "kernel sources changed since the counters were collected (%s)" % tab.get("collected_with", "?")
    return {(e["workload"], e["dtype"], e["kernel"]): e for e in tab["entries"]}, tab.get("collected_with")


def make_workload(workloads, name, points, channels):
    if name == "lidar_sweep":
        return workloads.lidar_sweep(N=points, C=channels, seed=2)
    return getattr(workloads, name)()


def measure(T, scatter_ext, workloads, names, w, dtype, steps, warmup, dev, extras=False, kernel_iters=50):
    """One workload at one dtype: the autograd step, then the step's four entry-point calls
    timed one by one in step order."""
    N, C, U = w.N, w.C, w.U
    tdt = TORCH_DTYPE[dtype]
    esz = 4 if dtype == "f32" else 2
    g_mean_cpu = workloads.upstream_grad(U, C, 102)
    g_max_cpu = workloads.upstream_grad(U, C, 103)
    feats = w.feats.to(dev).to(tdt).requires_grad_(True)
    inv, cnts = w.unq_inv.to(dev), w.unq_cnts.to(dev)
    g_mean, g_max = g_mean_cpu.to(dev).to(tdt), g_max_cpu.to(dev).to(tdt)

    for _ in range(3):                     # index preparation, timed separately
        data = T.ScatterData(inv, cnts)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        data = T.ScatterData(inv, cnts)
    torch.cuda.synchronize()
    prep_ms = (time.perf_counter() - t0) / 20 * 1e3

    def step():
        feats.grad = None
        T.scatter_mean(feats, data).backward(g_mean)
        feats.grad = None
        mx, _ = T.scatter_max(feats, data)
        mx.backward(g_max)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    feats.grad = None

    # per-kernel durations inside the step: the same four entry-point calls in the same
    # order as the timed region above, each bracketed by HIP events recorded on the
    # stream the kernels are launched on (so every launch sees the cache state it sees
    # in the step, not the one a back-to-back loop of one kernel leaves behind)
    f = feats.detach()
    plan = data.forward_args(C)
    bplan = data.backward_args()
    kt, kt_spread = instrumented_steps(scatter_ext, f, g_mean, g_max, plan, bplan, steps, warmup)
    kernel_sum_ms = sum(kt.values())
    graph_ms = graph_step_ms(scatter_ext, f, g_mean, g_max, plan, bplan, steps, warmup)
    res = {"N": N, "C": C, "U": U, "esz": esz, "data": data, "f": f, "g_mean": g_mean, "g_max": g_max,
           "g_mean_cpu": g_mean_cpu, "g_max_cpu": g_max_cpu, "inv": inv, "cnts": cnts, "plan": plan,
           "bplan": bplan, "prep_ms": prep_ms, "ms_per_step": ms_per_step, "kernel_sum_ms": kernel_sum_ms,
           "ms_per_step_graph": graph_ms}
    if extras:
        # not part of the step: back-to-back launches of scatter_sum's kernels and of the
        # forward under the reference's tie rule (what grouped input gets by default)
        it = kernel_iters
        kt["sum_fwd"] = event_ms(lambda: scatter_ext.forward(scatter_ext.SUM, f, *plan), it)
        kt["sum_bwd"] = event_ms(lambda: scatter_ext.backward(scatter_ext.SUM, g_mean, None, *bplan), it)
        kt["max_reftie_fwd"] = event_ms(lambda: scatter_ext.forward(scatter_ext.MAX_REFTIE, f, *plan), it)
    ab = {k: workloads.algorithmic_bytes(k.replace("max_reftie", "max"), N, C, U, esz) for k in kt}
    res["kt"] = kt
    res["ab"] = ab
    res["per_kernel"] = {k: {"kernel": names(k, dtype, N, C, U), "ms": kt[k], "GBps": ab[k] / kt[k] / 1e6,
                             "frac": ab[k] / kt[k] / 1e6 / HBM_PEAK_GBPS, **kt_spread.get(k, {})}
                         for k in kt}
    per_op = {}
    for op in ("mean", "max") + (("sum",) if extras else ()):
        t = kt[op + "_fwd"] + kt[op + "_bwd"]
        b = ab[op + "_fwd"] + ab[op + "_bwd"]
        per_op[op] = {"ms_fwd": kt[op + "_fwd"], "ms_bwd": kt[op + "_bwd"], "points_per_s": N / t * 1e3,
                      "GBps": b / t / 1e6, "frac_of_hbm_peak": b / t / 1e6 / HBM_PEAK_GBPS}
    res["per_op"] = per_op
    res["dominant"] = max(("max_fwd", "max_bwd", "mean_fwd", "mean_bwd"), key=lambda k: kt[k])
    return res


def workload_label(name, r, dtype):
    d = r["data"]
    return "%s N=%d C=%d %s, U=%d, max_cnt=%d, %s unq_inv%s" % (
        name, r["N"], r["C"], dtype, r["U"], d.max_cnt, "sorted" if d.is_sorted else "unsorted",
        ", voxel 0.2m" if name == "lidar_sweep" else ", pillar 0.2m x 0.2m" if name == "lidar_pillars" else "")


def compact(name, dtype, r):
    """The entry of one (workload, dtype) in other_configs."""
    dom = r["dominant"]
    step_bytes = sum(r["ab"][k] for k in ("mean_fwd", "mean_bwd", "max_fwd", "max_bwd"))
    return {
        "workload": workload_label(name, r, dtype), "dtype": dtype,
        "U": r["U"], "max_cnt": r["data"].max_cnt, "num_heavy": r["data"].num_heavy,
        "points_in_heavy_voxels": int(r["cnts"][r["cnts"] > r["data"].heavy_threshold].sum()),
        "ms_per_step": r["ms_per_step"], "kernel_sum_ms": r["kernel_sum_ms"],
        "ms_per_step_graph": r["ms_per_step_graph"],
        "points_per_s": 2 * r["N"] / r["ms_per_step"] * 1e3,
        "step_frac_of_hbm_peak": step_bytes / r["kernel_sum_ms"] / 1e6 / HBM_PEAK_GBPS,
        "per_op_frac": {op: v["frac_of_hbm_peak"] for op, v in r["per_op"].items()},
        "per_kernel": {k: {"ms": v["ms"], "frac": v["frac"], "median_ms": v.get("median_ms"),
                           "min_ms": v.get("min_ms")} for k, v in r["per_kernel"].items()},
        "dominant_kernel": r["per_kernel"][dom]["kernel"], "dominant_frac": r["per_kernel"][dom]["frac"],
        "index_prep_ms": r["prep_ms"],
    }


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    import __graft_entry__
    __graft_entry__._load_build().ensure_built()
    import torchex_amd as T
    from tests import workloads
    from torchex_amd._native import scatter_ext

    dev = torch.device("cuda:0")
    names = KernelNames()
    w = make_workload(workloads, a.workload, a.points, a.channels)
    r = measure(T, scatter_ext, workloads, names, w, a.dtype, a.steps, a.warmup, dev, extras=True,
                kernel_iters=a.kernel_iters)
    N, C, U, esz, data, f = r["N"], r["C"], r["U"], r["esz"], r["data"], r["f"]
    kt, ab, per_kernel = r["kt"], r["ab"], r["per_kernel"]
    scatter_fwd = scatter_ext.forward

    frontend = None
    if a.workload == "lidar_sweep" and not a.no_frontend:
        frontend = frontend_timings(T, workloads, dev, N)

    # the same points delivered grouped by voxel, which is the only order the reference's
    # kernels accept (its getPreSum needs sorted ids): no row permutation, sequential writes
    sorted_input = None
    if a.sorted_input and not data.is_sorted:
        order = torch.sort(r["inv"], stable=True)[1]
        f_s = f[order].contiguous()
        data_s = T.ScatterData(r["inv"][order].contiguous(), r["cnts"])
        plan_s = data_s.forward_args(C)
        kts, _ = instrumented_steps(scatter_ext, f_s, r["g_mean"], r["g_max"], plan_s,
                                    data_s.backward_args(), a.steps, a.warmup)
        sorted_input = {"per_kernel_ms": kts, "kernel_sum_ms": sum(kts.values()),
                        "points_per_s": 2 * N / sum(kts.values()) * 1e3,
                        "max_reftie_fwd_ms": event_ms(lambda: scatter_fwd(scatter_ext.MAX_REFTIE, f_s, *plan_s),
                                                      a.kernel_iters)}
        del f_s, data_s, plan_s, order

    isolated = None
    if a.isolated:
        # back-to-back launches of one entry point: upstream rows stay in the 256 MB
        # memory-side cache between launches, so the backward kernels read faster here
        it, plan, bplan = a.kernel_iters, r["plan"], r["bplan"]
        _, arg = scatter_fwd(scatter_ext.MAX, f, *plan)
        isolated = {
            "mean_fwd": event_ms(lambda: scatter_fwd(scatter_ext.MEAN, f, *plan), it),
            "mean_bwd": event_ms(lambda: scatter_ext.backward(scatter_ext.MEAN, r["g_mean"], None, *bplan), it),
            "max_fwd": event_ms(lambda: scatter_fwd(scatter_ext.MAX, f, *plan), it),
            "max_bwd": event_ms(lambda: scatter_ext.backward(scatter_ext.MAX, r["g_max"], arg, *bplan), it),
        }

    # a plain device copy of the feature matrix on the same box: the practical ceiling
    dst = torch.empty_like(f)
    copy_ms = event_ms(lambda: dst.copy_(f), 20)
    copy_gbps = 2 * f.numel() * esz / copy_ms / 1e6
    del dst

    dom = r["dominant"]
    traffic_table, traffic_source = load_traffic_table()
    entry = traffic_table.get((a.workload, a.dtype, per_kernel[dom]["kernel"]))
    if a.workload == "lidar_sweep" and (N, C) != (1_000_000, 128):
        entry = None    # the table holds the workloads at their default sizes
    roofline = {"bound": "hbm", "kernel": per_kernel[dom]["kernel"], "achieved": per_kernel[dom]["GBps"],
                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": per_kernel[dom]["frac"],
                "traffic": (entry["fetch_bytes"] + entry["write_bytes"]) if entry else None,
                "traffic_source": (entry or {}).get("profile", traffic_source),
                "algorithmic_bytes": ab[dom], "launch_ms": kt[dom]}

    out = {
        "metric": "scatter_mean+scatter_max(+argmax) fwd+bwd points/s (per operator pass), 1 GPU",
        "value": 2 * N / r["ms_per_step"] * 1e3,
        "unit": "points/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic",
        "config": {"workload": workload_label(a.workload, r, a.dtype),
                   "num_special_voxels": data.num_special, "num_heavy_voxels": data.num_heavy,
                   "heavy_threshold": data.heavy_threshold},
        "roofline": roofline,
        "per_op": r["per_op"],
        "per_kernel": per_kernel,
        "kernel_sum_ms": r["kernel_sum_ms"],
        "ms_per_step_graph": r["ms_per_step_graph"],
        "sorted_input": sorted_input,
        "device_copy_GBps": copy_gbps,
        "index_prep_ms": r["prep_ms"],
        "step_incl_index_prep_ms": r["ms_per_step"] + r["prep_ms"],
        "frontend": frontend,
    }
    if isolated is not None:
        out["per_kernel_isolated_ms"] = isolated
    g_mean_cpu, g_max_cpu = r["g_mean_cpu"], r["g_max_cpu"]
    del r, f, data
    torch.cuda.empty_cache()

    if not a.no_other_configs:
        others = []
        for name, dt in OTHER_CONFIGS:
            if (name, dt) == (a.workload, a.dtype):
                continue
            wo = w if name == a.workload else make_workload(workloads, name, 1_000_000, 128)
            ro = measure(T, scatter_ext, workloads, names, wo, dt, a.other_steps, a.other_warmup, dev)
            entry = compact(name, dt, ro)
            if name == "uniform_box" and dt == "f32" and not a.no_cpu_baseline:
                # the configuration quoted "on the CPU reference path": the same step on the host cores
                entry["cpu_baseline"] = cpu_baseline(wo, ro["g_mean_cpu"], ro["g_max_cpu"], budget_s=3.0)
            others.append(entry)
            del ro, wo
            torch.cuda.empty_cache()
        out["other_configs"] = others

    if not a.no_cpu_baseline and a.dtype == "f32":
        out["cpu_baseline"] = cpu_baseline(w, g_mean_cpu, g_max_cpu)
        if frontend is not None:
            out["frontend_cpu_baseline"] = frontend_cpu(workloads, N)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
