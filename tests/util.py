"""Helpers shared by the tests."""
import copy
import os

import numpy as np
import torch

import svox_amd as svox
from svox_amd import csrc as C


def options(tree, **kw):
    """RenderOptions for `tree` as VolumeRenderer would build them; kw: VolumeRenderer arguments plus
    fast / sigma_thresh / stop_thresh."""
    fast = kw.pop("fast", False)
    sigma_thresh = kw.pop("sigma_thresh", None)
    stop_thresh = kw.pop("stop_thresh", None)
    r = svox.VolumeRenderer(tree, **kw)
    if sigma_thresh is not None:
        r.sigma_thresh = sigma_thresh
    if stop_thresh is not None:
        r.stop_thresh = stop_thresh
    return r._get_options(fast)


def rays_spec(rays, device=None):
    s = C.RaysSpec()
    s.origins = rays.origins if device is None else rays.origins.to(device)
    s.dirs = rays.dirs if device is None else rays.dirs.to(device)
    s.vdirs = rays.viewdirs if device is None else rays.viewdirs.to(device)
    return s


def cam_spec(c2w, width, height, fx, fy=None, device=None, dtype=torch.float32):
    s = C.CameraSpec()
    s.c2w = c2w.to(device=device, dtype=dtype).contiguous()
    s.width, s.height, s.fx, s.fy = width, height, fx, fx if fy is None else fy
    return s


def rel_err(a, b):
    """max |a - b| / max |b| (relative to the largest reference magnitude)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    denom = np.abs(b).max()
    return float(np.abs(a - b).max() / (denom if denom > 0 else 1.0))


def grad_close(got, ref, rel=1e-4):
    """Element-wise gradient comparison that tolerates atomic summation order: every element must be
    within rel of the reference relative to the reference's own magnitude or to a floor tied to the
    largest gradient (sums of many terms of mixed sign cancel)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    floor = np.abs(ref).max() * 1e-3
    err = np.abs(got - ref) / np.maximum(np.abs(ref), floor if floor > 0 else 1.0)
    if os.environ.get("SVOX_TEST_VERBOSE"):
        print(f"[grad_close] worst relative error {float(err.max()):.3e} (limit {rel:.0e})", flush=True)
    return float(err.max()), err.max() <= rel


def on_gpu(tree, device):
    """A copy of `tree` on `device`; the original stays on the CPU (nn.Module.to moves in place)."""
    return copy.deepcopy(tree).to(device)
