"""ctypes front end of the CPU oracle (oracle/svox_oracle.cpp).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this module; the
product package never does.  Everything here works on host memory (numpy arrays or CPU torch
tensors) and mirrors the operator names of `svox_amd.csrc`.
"""
import ctypes
import os
import subprocess

import numpy as np

from svox_amd.csrc import _abi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsvox_oracle.so")

_lib = None
P = ctypes.POINTER
c_void_p, c_int32, c_int64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64


def build(verbose=False):
    """(Re)compile the oracle with the Makefile next to this file."""
    proc = subprocess.run(["make", "-B", "-C", HERE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
    if proc.returncode != 0:
        raise RuntimeError("building the oracle failed")
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        T, R, C, O, S = (P(_abi.TreeSpecC), P(_abi.RaysSpecC), P(_abi.CameraSpecC),
                         P(_abi.RenderOptionsC), P(_abi.MarchStatsC))
        sigs = {
            "oracle_out_data_dim": (ctypes.c_int, [c_int32, c_int32, c_int32]),
            "oracle_expf": (ctypes.c_float, [ctypes.c_float]),
            "oracle_sigmoid": (ctypes.c_float, [ctypes.c_float]),
            "oracle_max_threads": (ctypes.c_int, []),
            "oracle_basis": (ctypes.c_int, [c_int32, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_int32]),
            "oracle_query_vertical": (ctypes.c_int, [T, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
            "oracle_query_vertical_backward": (ctypes.c_int, [T, c_void_p, c_int64, c_void_p, c_int32, c_void_p, c_int32]),
            "oracle_assign_vertical": (ctypes.c_int, [T, c_void_p, c_int64, c_void_p, c_int32]),
            "oracle_calc_corners": (ctypes.c_int, [T, c_void_p, c_int64, c_void_p]),
            "oracle_volume_render": (ctypes.c_int, [T, R, O, c_void_p, S, c_int32]),
            "oracle_volume_render_image": (ctypes.c_int, [T, C, O, c_void_p, S, c_int32]),
            "oracle_volume_render_backward": (ctypes.c_int, [T, R, O, c_void_p, c_void_p, c_int32, S, c_int32, c_int32,
                                                             c_void_p]),
            "oracle_volume_render_image_backward": (ctypes.c_int, [T, C, O, c_void_p, c_void_p, c_int32, S, c_int32,
                                                                   c_int32, c_void_p]),
            "oracle_se_grad": (ctypes.c_int, [T, R, O, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p,
                                              c_void_p]),
            "oracle_se_grad_image": (ctypes.c_int, [T, C, O, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                                    c_void_p, c_void_p]),
            "oracle_grid_weight_render": (ctypes.c_int, [c_void_p, c_int32, c_int32, C, O, c_void_p, c_void_p, c_void_p,
                                                         c_void_p]),
            "oracle_image_rays": (ctypes.c_int, [T, C, O, c_void_p, c_void_p, c_void_p]),
            "oracle_trace_visits": (c_int64, [T, R, c_int64, O, c_void_p, c_void_p, c_void_p, c_void_p, c_int64]),
        }
        for name, (res, args) in sigs.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _np(x, dtype=None):
    """numpy view of a numpy array or CPU torch tensor, C-contiguous."""
    if x is None:
        return None
    if hasattr(x, "detach"):
        x = x.detach().cpu().numpy()
    x = np.ascontiguousarray(x)
    if dtype is not None and x.dtype != dtype:
        x = x.astype(dtype)
    return x


def _ptr(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


class Tree:
    """Host copy of a tree: numpy arrays with the layout of N3Tree's tensors."""

    def __init__(self, data, child, parent_depth, offset=None, scaling=None, extra_data=None,
                 weight_accum=None, weight_accum_max=False):
        self.data = _np(data)
        assert self.data.dtype in (np.float32, np.float64) and self.data.ndim == 5
        dt = self.data.dtype
        self.child = _np(child, np.int32)
        self.parent_depth = _np(parent_depth, np.int32)
        self.offset = _np(offset, dt)
        self.scaling = _np(scaling, dt)
        self.extra_data = _np(extra_data, dt) if extra_data is not None and np.size(_np(extra_data)) else None
        self.weight_accum = weight_accum
        self.weight_accum_max = weight_accum_max

    @classmethod
    def from_n3tree(cls, tree, world=True):
        return cls(tree.data, tree.child, tree.parent_depth,
                   tree.offset if world else None, tree.invradius if world else None, tree.extra_data)

    @property
    def dtype(self):
        return self.data.dtype

    def spec(self):
        s = _abi.TreeSpecC()
        s.data = _ptr(self.data)
        s.child = _ptr(self.child)
        s.parent_depth = _ptr(self.parent_depth)
        s.extra_data = _ptr(self.extra_data)
        s.extra_rows, s.extra_cols = (self.extra_data.shape if self.extra_data is not None else (0, 0))
        s.offset = _ptr(self.offset)
        s.scaling = _ptr(self.scaling)
        s.weight_accum = _ptr(self.weight_accum)
        s.weight_accum_max = int(self.weight_accum_max)
        s.capacity = self.child.shape[0]
        s.N = self.child.shape[1]
        s.data_dim = self.data.shape[4]
        s.dtype = _abi.SVOX_F32 if self.data.dtype == np.float32 else _abi.SVOX_F64
        return s


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with status {rc}")


def _opt(opt):
    return opt._pack() if hasattr(opt, "_pack") else opt


def out_data_dim(opt, data_dim):
    return lib().oracle_out_data_dim(int(opt.format), int(opt.basis_dim), int(data_dim))


def expf(x):
    x = np.asarray(x, dtype=np.float32)
    f = lib().oracle_expf
    return np.array([f(float(v)) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def basis(fmt, basis_dim, dirs, extra=None):
    """(B, basis_dim) basis values for directions (B, 3)."""
    dirs = _np(dirs)
    dt = dirs.dtype
    extra = _np(extra, dt)
    out = np.zeros((dirs.shape[0], basis_dim), dtype=dt)
    code = _abi.SVOX_F32 if dt == np.float32 else _abi.SVOX_F64
    for i in range(dirs.shape[0]):
        _check(lib().oracle_basis(fmt, basis_dim, _ptr(extra), 0 if extra is None else extra.shape[1],
                                  dirs[i].ctypes.data_as(c_void_p), out[i].ctypes.data_as(c_void_p), code),
               "basis")
    return out


def query_vertical(tree, points, want_levels=False):
    pts = _np(points, tree.dtype)
    Q = pts.shape[0]
    values = np.empty((Q, tree.data.shape[4]), dtype=tree.dtype)
    ids = np.empty((Q,), dtype=np.int64)
    levels = np.empty((Q,), dtype=np.int32)
    s = tree.spec()
    _check(lib().oracle_query_vertical(ctypes.byref(s), _ptr(pts), Q, _ptr(values), _ptr(ids), _ptr(levels)),
           "query_vertical")
    return (values, ids, levels) if want_levels else (values, ids)


def query_vertical_backward(tree, points, grad_output):
    pts = _np(points, tree.dtype)
    go = _np(grad_output, tree.dtype)
    M, N = tree.child.shape[0], tree.child.shape[1]
    grad = np.empty((M, N, N, N, go.shape[1]), dtype=tree.dtype)
    s = tree.spec()
    _check(lib().oracle_query_vertical_backward(ctypes.byref(s), _ptr(pts), pts.shape[0], _ptr(go),
                                                go.shape[1], _ptr(grad), 0), "query_vertical_backward")
    return grad


def assign_vertical(tree, points, values):
    """In place on tree.data."""
    pts = _np(points, tree.dtype)
    v = _np(values, tree.dtype)
    s = tree.spec()
    _check(lib().oracle_assign_vertical(ctypes.byref(s), _ptr(pts), pts.shape[0], _ptr(v), v.shape[1]),
           "assign_vertical")


def calc_corners(tree, indexer):
    idx = _np(indexer, np.int64)
    out = np.empty((idx.shape[0], 3), dtype=tree.dtype)
    s = tree.spec()
    _check(lib().oracle_calc_corners(ctypes.byref(s), _ptr(idx), idx.shape[0], _ptr(out)), "calc_corners")
    return out


def _rays(tree, origins, dirs, vdirs):
    o, d, v = _np(origins, tree.dtype), _np(dirs, tree.dtype), _np(vdirs, tree.dtype)
    return (o, d, v), _abi.RaysSpecC(_ptr(o), _ptr(d), _ptr(v), o.shape[0])


def _cam(tree, c2w, fx, fy, width, height):
    c = _np(c2w, tree.dtype)
    assert c.shape[1] == 4 and c.shape[0] >= 3
    return c, _abi.CameraSpecC(_ptr(c), float(fx), float(fy), int(width), int(height))


def volume_render(tree, origins, dirs, vdirs, opt, want_stats=False, n_threads=1):
    keep, r = _rays(tree, origins, dirs, vdirs)
    o = _opt(opt)
    od = lib().oracle_out_data_dim(o.format, o.basis_dim, tree.data.shape[4])
    out = np.empty((r.n_rays, od), dtype=tree.dtype)
    st = _abi.MarchStatsC()
    s = tree.spec()
    _check(lib().oracle_volume_render(ctypes.byref(s), ctypes.byref(r), ctypes.byref(o), _ptr(out),
                                      ctypes.byref(st), n_threads), "volume_render")
    return (out, st.as_dict()) if want_stats else out


def volume_render_image(tree, c2w, fx, fy, width, height, opt, want_stats=False, n_threads=1):
    keep, c = _cam(tree, c2w, fx, fy, width, height)
    o = _opt(opt)
    od = lib().oracle_out_data_dim(o.format, o.basis_dim, tree.data.shape[4])
    out = np.empty((height, width, od), dtype=tree.dtype)
    st = _abi.MarchStatsC()
    s = tree.spec()
    _check(lib().oracle_volume_render_image(ctypes.byref(s), ctypes.byref(c), ctypes.byref(o), _ptr(out),
                                            ctypes.byref(st), n_threads), "volume_render_image")
    return (out, st.as_dict()) if want_stats else out


def volume_render_backward(tree, origins, dirs, vdirs, opt, grad_output, want_stats=False, n_threads=1,
                           exact_sum=True, want_slack=False):
    """d(data) of the reference's backward kernel.  exact_sum (the default of every gradient function
    here): the terms (formed in the tree's scalar type, as the reference forms them) are added in
    float64 and rounded once -- the sum every floating-point order of the reference's atomics
    approximates, independent of ray order and thread count.  exact_sum=False adds them in the
    tree's scalar type in ray order (thread-dependent with n_threads > 1).
    want_slack (with exact_sum): also returns, shaped like the gradient, how far a sum of an element's
    n terms in the tree's scalar type may stray from the exact sum in any order:
    sqrt(n) * unit roundoff * sum |term| (what "up to the order of the atomics" amounts to)."""
    keep, r = _rays(tree, origins, dirs, vdirs)
    o = _opt(opt)
    go = _np(grad_output, tree.dtype)
    grad = np.empty_like(tree.data)
    slack = np.zeros_like(tree.data) if want_slack and exact_sum else None
    st = _abi.MarchStatsC()
    s = tree.spec()
    _check(lib().oracle_volume_render_backward(ctypes.byref(s), ctypes.byref(r), ctypes.byref(o), _ptr(go),
                                               _ptr(grad), 0, ctypes.byref(st), n_threads, int(exact_sum),
                                               _ptr(slack) if slack is not None else None),
           "volume_render_backward")
    res = (grad, slack) if want_slack else grad
    return (res, st.as_dict()) if want_stats else res


def volume_render_image_backward(tree, c2w, fx, fy, width, height, opt, grad_output, want_stats=False,
                                 n_threads=1, exact_sum=True, want_slack=False):
    keep, c = _cam(tree, c2w, fx, fy, width, height)
    o = _opt(opt)
    go = _np(grad_output, tree.dtype)
    grad = np.empty_like(tree.data)
    slack = np.zeros_like(tree.data) if want_slack and exact_sum else None
    st = _abi.MarchStatsC()
    s = tree.spec()
    _check(lib().oracle_volume_render_image_backward(ctypes.byref(s), ctypes.byref(c), ctypes.byref(o),
                                                     _ptr(go), _ptr(grad), 0, ctypes.byref(st), n_threads,
                                                     int(exact_sum), _ptr(slack) if slack is not None else None),
           "volume_render_image_backward")
    res = (grad, slack) if want_slack else grad
    return (res, st.as_dict()) if want_stats else res


def se_grad(tree, origins, dirs, vdirs, colors, opt, n_threads=1, exact_sum=True, want_slack=False):
    """(colour (B, C), grad, hessdiag) of 0.5 * |render - colors|^2; grad and hessdiag shaped like tree.data.
    want_slack: two more arrays, the order slack of grad and of hessdiag (see volume_render_backward)."""
    keep, r = _rays(tree, origins, dirs, vdirs)
    o = _opt(opt)
    od = lib().oracle_out_data_dim(o.format, o.basis_dim, tree.data.shape[4])
    ref = _np(colors, tree.dtype)
    assert ref.shape == (r.n_rays, od)
    out = np.empty((r.n_rays, od), dtype=tree.dtype)
    grad, hess = np.empty_like(tree.data), np.empty_like(tree.data)
    slack = (np.zeros_like(tree.data), np.zeros_like(tree.data)) if want_slack and exact_sum else (None, None)
    s = tree.spec()
    _check(lib().oracle_se_grad(ctypes.byref(s), ctypes.byref(r), ctypes.byref(o), _ptr(ref), _ptr(out), _ptr(grad),
                                _ptr(hess), n_threads, int(exact_sum), *[_ptr(x) if x is not None else None for x in slack]),
           "se_grad")
    return (out, grad, hess) + (slack if want_slack else ())


def se_grad_image(tree, c2w, fx, fy, width, height, colors, opt, n_threads=1, exact_sum=True, want_slack=False):
    keep, c = _cam(tree, c2w, fx, fy, width, height)
    o = _opt(opt)
    od = lib().oracle_out_data_dim(o.format, o.basis_dim, tree.data.shape[4])
    ref = _np(colors, tree.dtype)
    assert ref.shape == (height, width, od)
    out = np.empty((height, width, od), dtype=tree.dtype)
    grad, hess = np.empty_like(tree.data), np.empty_like(tree.data)
    slack = (np.zeros_like(tree.data), np.zeros_like(tree.data)) if want_slack and exact_sum else (None, None)
    s = tree.spec()
    _check(lib().oracle_se_grad_image(ctypes.byref(s), ctypes.byref(c), ctypes.byref(o), _ptr(ref), _ptr(out),
                                      _ptr(grad), _ptr(hess), n_threads, int(exact_sum),
                                      *[_ptr(x) if x is not None else None for x in slack]), "se_grad_image")
    return (out, grad, hess) + (slack if want_slack else ())


def grid_weight_render(data, c2w, fx, fy, width, height, opt, offset, scaling):
    """(grid_weight, grid_hit) of a dense (reso, reso, reso) density grid seen from one camera."""
    d = _np(data)
    assert d.ndim == 3 and d.shape[0] == d.shape[1] == d.shape[2]
    c = _np(c2w, d.dtype)
    cam = _abi.CameraSpecC(_ptr(c), float(fx), float(fy), int(width), int(height))
    off, sc = _np(offset, d.dtype), _np(scaling, d.dtype)
    o = _opt(opt)
    weight, hit = np.empty_like(d), np.empty_like(d)
    _check(lib().oracle_grid_weight_render(_ptr(d), d.shape[0], 0 if d.dtype == np.float32 else 1, ctypes.byref(cam),
                                           ctypes.byref(o), _ptr(off), _ptr(sc), _ptr(weight), _ptr(hit)),
           "grid_weight_render")
    return weight, hit


def image_rays(tree, c2w, fx, fy, width, height, opt):
    """(origins, dirs, vdirs), each (H*W, 3): the rays the image kernels trace (tree coordinates)."""
    keep, c = _cam(tree, c2w, fx, fy, width, height)
    o = _opt(opt)
    n = width * height
    outs = [np.empty((n, 3), dtype=tree.dtype) for _ in range(3)]
    s = tree.spec()
    _check(lib().oracle_image_rays(ctypes.byref(s), ctypes.byref(c), ctypes.byref(o), *[_ptr(a) for a in outs]),
           "image_rays")
    return tuple(outs)


def trace_visits(tree, origins, dirs, vdirs, ray_index, opt, max_visits=100000):
    """Leaf sequence of one ray: dict of arrays leaf (int64), t, delta_t, sigma (float64)."""
    keep, r = _rays(tree, origins, dirs, vdirs)
    o = _opt(opt)
    leaf = np.empty(max_visits, dtype=np.int64)
    t, dt, sg = (np.empty(max_visits, dtype=np.float64) for _ in range(3))
    s = tree.spec()
    n = lib().oracle_trace_visits(ctypes.byref(s), ctypes.byref(r), ray_index, ctypes.byref(o), _ptr(leaf),
                                  _ptr(t), _ptr(dt), _ptr(sg), max_visits)
    if n < 0:
        raise RuntimeError(f"oracle trace_visits failed with status {n}")
    n = min(n, max_visits)
    return {"leaf": leaf[:n], "t": t[:n], "delta_t": dt[:n], "sigma": sg[:n]}


def max_threads():
    return lib().oracle_max_threads()
