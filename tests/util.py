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


ORDER_SLACK_FACTOR = 2.0


# Worst error of every grad_close call of the session, by label: tests/conftest.py prints them after the run, so that
# the log shows how close to the gate the kernels run and not only that they passed.
GATE_LOG = []


def _caller_label():
    test = os.environ.get("PYTEST_CURRENT_TEST", "")
    return test.split(" ")[0].split("::", 1)[-1] if test else "?"


def grad_close(got, ref, rel=1e-4, slack=None, what=None):
    """Element-wise gradient comparison against the oracle's exact sum: every element must be within
    `rel` of the reference, relative to the reference's own magnitude or, for elements below it, to a
    floor of 1e-3 of the largest gradient.

    slack (the oracle's want_slack output): what fp32 additions of an element's terms in an arbitrary
    order can differ from the exact sum by, sqrt(n) * 2^-24 * sum |term|.  Sequential fp32 sums of the
    same terms in shuffled orders -- what the reference's own atomics produce -- reach 0.5 to 1.05 of
    it on the many-rays-per-leaf cases of these tests, which is 2e-5 to 1.6e-4 in the relative measure
    above; ORDER_SLACK_FACTOR times the slack is taken off the difference before it is measured.  One
    term missing from a leaf that 4000 rays share is still 30 times that allowance."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    floor = np.abs(ref).max() * 1e-3
    diff = np.abs(got - ref)
    if slack is not None:
        diff = np.maximum(diff - ORDER_SLACK_FACTOR * np.asarray(slack, dtype=np.float64), 0.0)
    err = diff / np.maximum(np.abs(ref), floor if floor > 0 else 1.0)
    worst = float(err.max()) if err.size else 0.0
    GATE_LOG.append((_caller_label() + (f" [{what}]" if what else ""), worst, rel, slack is not None))
    if os.environ.get("SVOX_TEST_VERBOSE"):
        print(f"[grad_close] worst relative error {worst:.3e} (limit {rel:.0e})", flush=True)
    return worst, worst <= rel


def on_gpu(tree, device):
    """A copy of `tree` on `device`; the original stays on the CPU (nn.Module.to moves in place)."""
    return copy.deepcopy(tree).to(device)
