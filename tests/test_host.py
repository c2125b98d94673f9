"""CPU-side checks: the C ABI library loads and exports what the header declares,
host-only entry points behave, the package imports, workloads are deterministic."""
import ctypes
import io
import os
import re
from contextlib import redirect_stdout

import numpy as np
import torch

from tests.conftest import ROOT
from tests import workloads


def _lib():
    from torchex_amd import _native
    return _native.cabi()


def test_header_symbols_are_exported():
    with open(os.path.join(ROOT, "include", "torchex_scatter.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(txs_[a-z_0-9]+)\s*\(", text)))
    assert len(names) >= 14
    lib = _lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_header_is_plain_c_and_links(tmp_path):
    """The boundary is a C ABI: the header compiles as C11 with no extensions and a C
    program links against the library without any C++ or torch symbol in sight."""
    import shutil
    import subprocess
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        import pytest
        pytest.skip("no C compiler on this machine")
    src = tmp_path / "abi.c"
    src.write_text('#include "torchex_scatter.h"\n'
                   'int main(void) { return txs_abi_version() == 9 && txs_chunk_rows() > 0 ? 0 : 1; }\n')
    inc = os.path.join(ROOT, "include")
    pkg = os.path.join(ROOT, "torchex_amd")
    subprocess.check_call([cc, "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I" + inc,
                           "-fsyntax-only", str(src)])
    exe = tmp_path / "abi"
    subprocess.check_call([cc, "-std=c11", "-I" + inc, str(src), "-L" + pkg, "-ltorchex_scatter",
                           "-Wl,-rpath," + pkg, "-o", str(exe)])
    assert subprocess.call([str(exe)]) == 0


def test_host_only_entry_points():
    lib = _lib()
    assert lib.txs_abi_version() == 9
    lib.txs_status_string.restype = ctypes.c_char_p
    assert lib.txs_status_string(0) == b"ok"
    assert b"invalid" in lib.txs_status_string(1)
    assert b"unknown" in lib.txs_status_string(99)
    assert lib.txs_default_heavy_threshold() >= lib.txs_chunk_rows() > 0
    lib.txs_sort_workspace_len.restype = ctypes.c_int64
    n = 1_000_000
    assert lib.txs_sort_workspace_len(ctypes.c_int64(n), ctypes.c_int64(120000)) >= 2 * n


def test_argument_validation_needs_no_gpu():
    # these return before any launch
    lib = _lib()
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    def fwd(op, dtype, num_total, path=0):
        return lib.txs_scatter_forward(ci(op), ci(dtype), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), i64(0),
                                       i64(0), vp(0), i64(0), vp(0), vp(0), i64(num_total), i64(1), i64(1), i64(1),
                                       ci(path), vp(0))
    assert fwd(9, 0, 1) == 3
    assert fwd(0, 5, 1) == 3
    assert fwd(0, 0, 1, path=7) == 3
    assert fwd(0, 0, 1 << 40) == 1
    rc = lib.txs_scatter_backward(ci(2), ci(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), i64(5), i64(4),
                                  i64(2), ci(0), vp(0))
    assert rc == 1
    # scratch sizing and kernel naming are host-only too
    lib.txs_scatter_scratch_cells.restype = ctypes.c_int64
    assert lib.txs_scatter_scratch_cells(i64(1_000_000), i64(128), i64(300_000), i64(10)) == 1280
    assert lib.txs_scatter_scratch_cells(i64(-1), i64(128), i64(3), i64(0)) == -1
    buf = ctypes.create_string_buffer(64)
    assert lib.txs_kernel_name(ci(0), ci(2), ci(0), i64(1_000_000), i64(128), i64(300_000), i64(16), ci(1), buf,
                               i64(64)) == 0
    assert buf.value == b"scatter_fwd_kernel<F32,4,MAX>"
    assert lib.txs_kernel_name(ci(1), ci(1), ci(1), i64(1_000_000), i64(128), i64(300_000), i64(16), ci(1), buf,
                               i64(64)) == 0
    assert buf.value == b"scatter_bwd_kernel<F16,4,MEAN,8>"
    # long runs on average: the forward walks longer chunks
    assert lib.txs_kernel_name(ci(0), ci(0), ci(1), i64(1_000_000), i64(128), i64(89_260), i64(16), ci(1), buf,
                               i64(64)) == 0
    assert buf.value == b"scatter_fwd_kernel<F16,4,SUM>"
    rc = lib.txs_get_presum(vp(0), vp(0), i64(-1), i64(0), vp(0))
    assert rc == 1
    # the unique-by-occupancy-map and ranking entry points: sizes and null pointers are checked first
    lib.txs_unique_bitmap_workspace_len.restype = ctypes.c_int64
    words = (16_875_000 + 31) // 32
    assert lib.txs_unique_bitmap_workspace_len(i64(16_875_000)) >= 10 * words
    assert lib.txs_unique_bitmap_workspace_len(i64(0)) == -1
    assert lib.txs_unique_bitmap_workspace_len(i64((1 << 31) + 1)) == -1
    assert lib.txs_unique_bitmap_count(vp(0), ci(0), i64(5), i64(0), vp(0), vp(0), vp(0)) == 1
    assert lib.txs_unique_bitmap_count(vp(0), ci(0), i64(5), i64(100), vp(0), vp(8), vp(0)) == 1   # no keys
    assert lib.txs_unique_bitmap_assign(vp(0), ci(1), i64(1 << 40), i64(100), vp(0), vp(0), vp(0), vp(0)) == 1
    assert lib.txs_counts_from_presum(vp(0), i64(3), vp(0), vp(0)) == 1
    assert lib.txs_counts_from_presum(vp(0), i64(0), vp(0), vp(0)) == 0                             # nothing to do
    assert lib.txs_group_ranks(vp(0), i64(10), i64(10), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0), vp(0)) == 1
    lib.txs_plan_workspace_len.restype = ctypes.c_int64
    assert lib.txs_plan_workspace_len(i64(1_000_000), i64(326_859)) > 2 * 1_000_000
    lib.txs_dpp_workspace_len.restype = ctypes.c_int64
    # room for 2 result bits per (point, box): 25 groups of 8 boxes x 200k points x 16 bits
    assert lib.txs_dpp_workspace_len(i64(200_000), i64(200)) * 4 >= 25 * 200_000 * 2


def test_package_surface_matches_reference_exports():
    import torchex
    import torchex_amd
    for name in ["scatter_sum", "scatter_mean", "scatter_max", "ScatterData", "TorchTimer"]:
        assert hasattr(torchex, name) and getattr(torchex, name) is getattr(torchex_amd, name)
    import scatter_ext
    for name in ["sum", "max", "getPreSum"]:   # torchex/src/scatter/scatter.cpp:66-70
        assert callable(getattr(scatter_ext, name))
    # the modules the reference's other wrappers import by name, with their functions
    import dynamic_point_pool_ext   # src/dynamic_point_pool/dynamic_point_pool.cpp:166-169
    import grid_hash_ext            # src/grid_hash/grid_hash.cpp:115-118
    import ingroup_indices          # src/ingroup_inds/ingroup_inds.cpp:52-54
    assert callable(ingroup_indices.forward)
    assert callable(dynamic_point_pool_ext.forward) and callable(dynamic_point_pool_ext.dynamic_point_pool_mixed_gpu)
    assert callable(grid_hash_ext.build_table) and callable(grid_hash_ext.probe_table)


def test_reference_modules_reject_cpu_tensors():
    import pytest
    import dynamic_point_pool_ext
    import grid_hash_ext
    import ingroup_indices
    ids = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ingroup_indices.forward(ids, torch.zeros_like(ids))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        dynamic_point_pool_ext.forward(torch.zeros((1, 7)), torch.zeros((5, 3)), [0.0, 0.0, 0.0], 8,
                                       torch.zeros(9, dtype=torch.int64), torch.zeros(9, dtype=torch.int64),
                                       torch.zeros((9, 13)))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        grid_hash_ext.build_table(torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32))


def test_cpu_tensors_are_rejected_not_silently_computed():
    import pytest
    import scatter_ext
    f = torch.zeros((4, 4))
    pre = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        scatter_ext.sum(f, pre, torch.zeros((1, 4)), 4)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        scatter_ext.getPreSum(torch.zeros(4, dtype=torch.int32), pre)


def test_torch_timer_prints_running_mean():
    from torchex_amd import TorchTimer
    t = TorchTimer(2)
    buf = io.StringIO()
    with redirect_stdout(buf):
        for _ in range(4):
            with t.timing("x"):
                pass
        with t.timing("off", freq=-1):
            pass
    lines = buf.getvalue().strip().splitlines()
    assert len(lines) == 2 and all(l.startswith("Average time cost of x:") and l.endswith("ms") for l in lines)


def test_workloads_are_seeded_and_shaped():
    a = workloads.uniform_box(N=5000, C=4)
    b = workloads.uniform_box(N=5000, C=4)
    assert torch.equal(a.feats, b.feats) and torch.equal(a.unq_inv, b.unq_inv)
    assert a.unq_cnts.sum().item() == 5000 and a.unq_inv.max().item() == a.U - 1
    w = workloads.lidar_sweep(N=20000, C=4)
    assert w.unq_cnts.sum().item() == 20000
    z = workloads.zipf_contention(N=20000, C=2, num_ids=64)
    assert z.U <= 64 and z.unq_cnts.max().item() > 20000 / 64
    m = workloads.multi_sweep(N_per=2000, sweeps=3, C=2)
    assert m.N == 6000
    # keys of different sweeps never collide: every voxel's rows come from one sweep
    sweep = torch.arange(6000) // 2000
    lo = torch.full((m.U,), 99).scatter_reduce(0, m.unq_inv, sweep, "amin")
    hi = torch.full((m.U,), -1).scatter_reduce(0, m.unq_inv, sweep, "amax")
    assert torch.equal(lo, hi)


def test_algorithmic_bytes_formulae():
    N, C, U = 1_000_000, 128, 120_000
    assert workloads.algorithmic_bytes("max_fwd", N, C, U) == N * C * 4 + 4 * N + U * C * 4 + 4 * U * C
    fb = workloads.algorithmic_bytes("max_fwd", N, C, U) + workloads.algorithmic_bytes("max_bwd", N, C, U)
    assert abs(fb - 1.278e9) / 1.278e9 < 0.01
    fb = workloads.algorithmic_bytes("mean_fwd", N, C, U) + workloads.algorithmic_bytes("mean_bwd", N, C, U)
    assert abs(fb - 1.157e9) / 1.157e9 < 0.01
