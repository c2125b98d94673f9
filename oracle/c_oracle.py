"""ctypes binding of ``scatter_oracle.c`` over numpy arrays (test infrastructure).

Every function takes / returns C-contiguous numpy arrays: features ``float32
[N, C]``, ``unq_inv`` ``int32 [N]``, ``preSum`` ``int32 [U+1]``, counts ``int64
[U]``, ``arg`` ``int32 [U, C]``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile ``scatter_oracle.c`` with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_up_2n.restype = ctypes.c_int
        _lib.orc_up_2n.argtypes = [ctypes.c_int]
        _lib.orc_block_width.restype = ctypes.c_int
        _lib.orc_block_width.argtypes = [ctypes.c_int]
        _lib.orc_counts.restype = ctypes.c_int
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _ll(x):
    return ctypes.c_int64(int(x))


def up_2n(n):
    return lib().orc_up_2n(int(n))


def block_width(max_cnt):
    return lib().orc_block_width(int(max_cnt))


def get_presum_ref(unq_inv):
    """Reference getPreSum on a sorted ``unq_inv`` (length ``unq_inv[-1] + 2``)."""
    inv = _i32(unq_inv)
    n = inv.shape[0]
    pre = np.zeros(int(inv[-1]) + 2 if n else 1, dtype=np.int32)
    lib().orc_get_presum_ref(_p(inv), _ll(n), _p(pre))
    return pre


def counts(unq_inv, num_unq):
    inv = _i32(unq_inv)
    cnt = np.zeros(num_unq, dtype=np.int64)
    rc = lib().orc_counts(_p(inv), _ll(inv.shape[0]), _ll(num_unq), _p(cnt))
    if rc != 0:
        raise ValueError("unq_inv holds an id outside [0, num_unq)")
    return cnt


def presum(cnt):
    cnt = _i64(cnt)
    pre = np.zeros(cnt.shape[0] + 1, dtype=np.int32)
    lib().orc_presum(_p(cnt), _ll(cnt.shape[0]), _p(pre))
    return pre


def stable_perm(unq_inv, pre):
    inv = _i32(unq_inv)
    pre = _i32(pre)
    perm = np.empty(inv.shape[0], dtype=np.int32)
    lib().orc_stable_perm(_p(inv), _ll(inv.shape[0]), _ll(pre.shape[0] - 1), _p(pre), _p(perm))
    return perm


def scatter_sum_ref(feats_sorted, pre, max_cnt):
    f = _f32(feats_sorted)
    pre = _i32(pre)
    U, C = pre.shape[0] - 1, f.shape[1]
    out = np.zeros((U, C), dtype=np.float32)
    lib().orc_scatter_sum_ref(_p(f), _p(pre), _p(out), _ll(C), _ll(U), ctypes.c_int(int(max_cnt)))
    return out


def scatter_max_ref(feats_sorted, pre, max_cnt):
    f = _f32(feats_sorted)
    pre = _i32(pre)
    U, C = pre.shape[0] - 1, f.shape[1]
    out = np.zeros((U, C), dtype=np.float32)
    arg = np.zeros((U, C), dtype=np.int32)
    lib().orc_scatter_max_ref(_p(f), _p(pre), _p(out), _p(arg), _ll(C), _ll(U),
                              ctypes.c_int(int(max_cnt)))
    return out, arg


def scatter_sum_f64(feats, unq_inv, num_unq):
    f = _f32(feats)
    inv = _i32(unq_inv)
    out = np.zeros((num_unq, f.shape[1]), dtype=np.float64)
    lib().orc_scatter_sum_f64(_p(f), _p(inv), _ll(f.shape[0]), _ll(f.shape[1]), _ll(num_unq), _p(out))
    return out


def scatter_max_first(feats, unq_inv, num_unq):
    f = _f32(feats)
    inv = _i32(unq_inv)
    out = np.zeros((num_unq, f.shape[1]), dtype=np.float32)
    arg = np.zeros((num_unq, f.shape[1]), dtype=np.int32)
    lib().orc_scatter_max_first(_p(f), _p(inv), _ll(f.shape[0]), _ll(f.shape[1]), _ll(num_unq),
                                _p(out), _p(arg))
    return out, arg


def mean_from_sum(sums, cnt):
    s = _f32(sums)
    cnt = _i64(cnt).reshape(-1)
    out = np.empty_like(s)
    lib().orc_mean_from_sum(_p(s), _p(cnt), _ll(s.shape[1]), _ll(s.shape[0]), _p(out))
    return out


def sum_backward(g, unq_inv):
    g = _f32(g)
    inv = _i32(unq_inv)
    gin = np.empty((inv.shape[0], g.shape[1]), dtype=np.float32)
    lib().orc_sum_backward(_p(g), _p(inv), _ll(inv.shape[0]), _ll(g.shape[1]), _p(gin))
    return gin


def mean_backward(g, cnt, unq_inv):
    g = _f32(g)
    inv = _i32(unq_inv)
    cnt = _i64(cnt).reshape(-1)
    gin = np.empty((inv.shape[0], g.shape[1]), dtype=np.float32)
    lib().orc_mean_backward(_p(g), _p(cnt), _p(inv), _ll(inv.shape[0]), _ll(g.shape[1]), _p(gin))
    return gin


def max_backward(g, arg, n):
    g = _f32(g)
    arg = _i32(arg)
    gin = np.empty((n, g.shape[1]), dtype=np.float32)
    lib().orc_max_backward(_p(g), _p(arg), _ll(n), _ll(g.shape[1]), _ll(g.shape[0]), _p(gin))
    return gin


def sorted_view(feats, unq_inv, num_unq):
    """Group rows by voxel with a stable sort, as the reference requires its
    callers to do: returns ``(feats_sorted, perm, preSum, counts)``."""
    cnt = counts(unq_inv, num_unq)
    pre = presum(cnt)
    perm = stable_perm(unq_inv, pre)
    return _f32(feats)[perm], perm, pre, cnt


def scatter_sum_reforder(feats, unq_inv, num_unq):
    """scatter_sum of unsorted input in the reference's fp32 rounding order."""
    fs, _, pre, cnt = sorted_view(feats, unq_inv, num_unq)
    return scatter_sum_ref(fs, pre, int(cnt.max()) if cnt.size else 1)


def scatter_max_reforder(feats, unq_inv, num_unq):
    """scatter_max of unsorted input with the reference's lane tie rule; the
    arg indices are mapped back to original row numbers."""
    fs, perm, pre, cnt = sorted_view(feats, unq_inv, num_unq)
    out, arg = scatter_max_ref(fs, pre, int(cnt.max()) if cnt.size else 1)
    arg_rows = np.where(arg >= 0, perm[np.clip(arg, 0, None)] if perm.size else arg, -1).astype(np.int32)
    return out, arg_rows


def ingroup_inds(group_ids):
    g = _i64(group_ids)
    out = np.empty_like(g)
    if g.size:
        lib().orc_ingroup_inds(_p(g), _ll(g.shape[0]), _ll(int(g.max())), _p(out))
    return out


def voxelize(points, voxel_size, range_lo, dims):
    pts = _f32(points)
    lo = _f32(range_lo)
    vs = _f32(voxel_size)
    dm = _i32(dims)
    n = pts.shape[0]
    coors = np.empty((n, 3), dtype=np.int32)
    keys = np.empty(n, dtype=np.int32)
    lib().orc_voxelize(_p(pts), _ll(n), _ll(pts.shape[1]), _p(lo), _p(vs), _p(dm), _p(coors), _p(keys))
    return coors, keys


def dynamic_point_pool(rois, pts, extra_wlh, max_pts, max_all, rois_batch=None, pts_batch=None):
    r = _f32(rois)
    p = _f32(pts)
    e = _f32(extra_wlh)
    idx = np.full(max_all, -1, dtype=np.int64)
    roi = np.full(max_all, -1, dtype=np.int64)
    feats = np.zeros((max_all, 13), dtype=np.float32)
    rb = _i32(rois_batch) if rois_batch is not None else None
    pb = _i32(pts_batch) if pts_batch is not None else None
    assert (rb is None) == (pb is None)
    lib().orc_dynamic_point_pool_mixed.restype = ctypes.c_int64
    m = lib().orc_dynamic_point_pool_mixed(_p(r), _p(rb) if rb is not None else None, _ll(r.shape[0]), _p(p),
                                           _p(pb) if pb is not None else None, _ll(p.shape[0]), _p(e),
                                           ctypes.c_int(int(max_pts)), _ll(max_all), _p(idx), _p(roi), _p(feats))
    return idx[:m], roi[:m], feats[:m]


def grid_hash_build(keys, values):
    k = _i32(keys)
    v = _i32(values)
    size = 1
    while size < max(k.shape[0], 1):
        size <<= 1
    table = np.full((size, 2), -1, dtype=np.int32)
    rc = lib().orc_grid_hash_build(_p(k), _p(v), _ll(k.shape[0]), _p(table), ctypes.c_int(size))
    if rc != 0:
        raise RuntimeError("hash table full")
    return table


def grid_hash_probe(keys, table):
    k = _i32(keys)
    t = _i32(table)
    out = np.empty(k.shape[0], dtype=np.int32)
    lib().orc_grid_hash_probe(_p(k), _ll(k.shape[0]), _p(t), ctypes.c_int(t.shape[0]), _p(out))
    return out
