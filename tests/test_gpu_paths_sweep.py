"""Seeded sweep over random small trees and options: every GPU path of the renderer against the oracle.

Per case: shell / dense / deep-chain tree, 100-5000 sphere rays, random step size, fast or exact
thresholds, random background.  Paths: forward, marching backward with and without a workspace, noted
forward + replayed backward, se_grad with and without a workspace -- each with the rays handled as a
small batch and as a large one (debug flag 2), on the plain tree and with the empty leaves marked; the
forward pass, the noted forward pass and se_grad also on either of the small-launch kernels (debug
flags 4 and 8).  With marks made with the case's own sigma_thresh (svox_mark_leaves_below: the forward kernels
then shade every leaf the marks let through and read its density with its coefficients) the forward pass runs on
all four kernel choices, and the backward and noted passes once each (they leave such marks aside when the
threshold is not 0).

Bars: pictures equal to the oracle's bit for bit; gradients within 1e-4 relative of the oracle's exact
sum (fp32 terms added in float64) beyond the order slack of fp32 additions, elements below 1e-3 of the
largest gradient measured against that floor (util.grad_close).  Cases 2, 7 and 17 put thousands of
rays into a few dozen leaves: there the fp32 additions of the terms in an arbitrary order -- the
reference's atomics as much as this library's -- are themselves up to 1.6e-4 from the exact sum.
"""
import itertools

import numpy as np
import pytest
import torch

from svox_amd import csrc as C
from svox_amd import synth
from util import grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu

FORMATS = ["RGBA", "SH1", "SH4", "SH9", "SH16", "SH25"]
N_CASES = 36
CASES = list(range(N_CASES))


def case_parameters():
    """The parameters of all N_CASES cases, drawn in order from one seeded generator."""
    rng = np.random.default_rng(0)
    out = []
    for it in range(N_CASES):
        p = {"fmt": FORMATS[it % 6], "seed": int(rng.integers(1 << 30)), "kind": it % 3}
        if p["kind"] == 0:
            p["tree"] = dict(depth=int(rng.integers(4, 8)), n_spheres=int(rng.integers(2, 8)),
                             sigma_range=(float(rng.uniform(0.5, 20)), float(rng.uniform(20, 300))))
        elif p["kind"] == 1:
            p["tree"] = dict(levels=int(rng.integers(2, 4)), zero_fraction=float(rng.uniform(0, 0.7)))
        else:
            p["tree"] = dict(levels=int(rng.integers(8, 16)))
            if p["fmt"] not in ("SH4", "RGBA"):
                p["fmt"] = "SH4"
        p["n_rays"] = int(rng.integers(100, 5000))
        p["step"] = float(10 ** rng.uniform(-3.5, -2))
        p["fast"] = bool(rng.integers(2))
        p["background"] = float(rng.uniform(0, 1))
        out.append(p)
    return out


PARAMETERS = case_parameters()


def build_tree(p):
    if p["kind"] == 0:
        return synth.shell_tree(data_format=p["fmt"], seed=p["seed"], **p["tree"])
    if p["kind"] == 1:
        return synth.dense_tree(p["tree"]["levels"], p["fmt"], seed=p["seed"], sigma="lognormal", coeff_std=0.5,
                                zero_fraction=p["tree"]["zero_fraction"])
    return synth.deep_tree(p["tree"]["levels"], data_format=p["fmt"], seed=p["seed"])[0]


@pytest.mark.parametrize("case", CASES)
def test_every_render_path_against_the_exact_sum_oracle(gpu, oracle_mod, case):
    p = PARAMETERS[case]
    tree = build_tree(p)
    n, seed = p["n_rays"], p["seed"]
    rays = synth.sphere_rays(n, seed=seed % 1000)
    opt = options(tree, step_size=p["step"], fast=p["fast"], background_brightness=p["background"])
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(seed % 77)) * 1e-2
    want_g, slack_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go,
                                                        n_threads=8, want_slack=True)
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(seed % 55))
    want_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=8, want_slack=True)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    plain = dev._spec()
    marked = dev._spec()
    marked.child_marks = C.mark_empty_leaves(plain)
    decided = dev._spec()
    decided.child_marks = C.mark_empty_leaves(plain, opt.sigma_thresh)
    decided.child_marks_thresh = opt.sigma_thresh
    failures = []
    paths = ("fwd", "bwd", "bwd_nows", "noted", "se", "se_nows")
    combos = list(itertools.product((0, 2), ((plain, "plain"), (marked, "marked")), paths))
    # the forward pass, the noted forward pass and se_grad's noting march once more on each of the two
    # small-launch kernels (one wavefront per 64 rays that walks and shades; two wavefronts, one for
    # each), whatever the launch size would choose
    combos += list(itertools.product((4, 8), ((plain, "plain"), (marked, "marked")), ("fwd", "noted", "se")))
    combos += list(itertools.product((0, 2, 4, 8), ((decided, "decided"),), ("fwd",)))
    combos += list(itertools.product((0,), ((decided, "decided"),), ("bwd", "noted", "se")))
    # the one-ray-per-lane kernels (what fp64 trees, partial component ranges and the other record shapes run on),
    # forced onto the same fp32 cases: forward, the gradient kernel and se_grad, whose wavefronts add the records
    # of a step together
    combos += list(itertools.product((1,), ((plain, "plain"),), ("fwd", "bwd_nows", "se_nows")))
    for flags, (spec, spec_name), name in combos:
        tag = f"{name}/flags{flags}/{spec_name}"
        C.set_debug_flags(flags)
        try:
            if name == "fwd":
                if not np.array_equal(C.volume_render(spec, rs, opt).cpu().numpy(), want):
                    failures.append(f"{tag}: picture differs")
            elif name in ("bwd", "bwd_nows"):
                g = C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=name == "bwd").cpu().numpy()
                err, ok = grad_close(g, want_g, slack=slack_g)
                if not ok:
                    failures.append(f"{tag}: gradient {err:.3e}")
            elif name == "noted":
                out, notes = C.volume_render_noted(spec, rs, opt)
                if not np.array_equal(out.cpu().numpy(), want):
                    failures.append(f"{tag}: picture differs")
                g = C.volume_render_backward_noted(spec, rs, opt, go.to(gpu), notes).cpu().numpy()
                err, ok = grad_close(g, want_g, slack=slack_g)
                if not ok:
                    failures.append(f"{tag}: gradient {err:.3e}")
            else:
                got = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=name == "se")
                if not np.array_equal(got[0].cpu().numpy(), want_se[0]):
                    failures.append(f"{tag}: colour differs")
                for what, x, w, sl in zip(("gradient", "hessian"), got[1:], want_se[1:3], want_se[3:]):
                    err, ok = grad_close(x.cpu().numpy(), w, slack=sl)
                    if not ok:
                        failures.append(f"{tag}: {what} {err:.3e}")
        finally:
            C.set_debug_flags(0)
    assert not failures, f"case {case} {p}: " + "; ".join(failures)
