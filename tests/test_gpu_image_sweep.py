"""Seeded sweep over small images: every image path of the renderer against the oracle.

Per case: shell or dense tree in one of the six record formats, 1-3 poses of a random small picture
(sizes that are no multiples of the 8x8 tile), random step size, fast or exact thresholds, random
background.  Paths: forward, marching backward with and without a workspace, noted forward + replayed
backward, se_grad_persp with and without a workspace -- on the plain tree and with the empty leaves
marked, and with the launches forced onto one wavefront per tile (debug flag 4) and onto two (flag 8)
as well as left to the library's choice.

Bars: pictures and se_grad colours equal to the oracle's bit for bit; gradients within 1e-4 relative
(util.grad_close)."""
import numpy as np
import pytest
import torch

from svox_amd import csrc as C
from svox_amd import synth
from util import cam_spec, grad_close, on_gpu, options

pytestmark = pytest.mark.gpu

FORMATS = ["RGBA", "SH4", "SH9", "SH16", "SH25", "SH1"]
N_CASES = 12


def case_parameters():
    rng = np.random.default_rng(2)
    out = []
    for it in range(N_CASES):
        p = {"fmt": FORMATS[it % 6], "seed": int(rng.integers(1 << 30)), "dense": it % 2 == 1}
        if p["dense"]:
            p["tree"] = dict(levels=int(rng.integers(2, 4)), zero_fraction=float(rng.uniform(0, 0.7)))
        else:
            p["tree"] = dict(depth=int(rng.integers(4, 7)), n_spheres=int(rng.integers(2, 8)),
                             sigma_range=(float(rng.uniform(0.5, 20)), float(rng.uniform(20, 300))))
        p["W"], p["H"] = int(rng.integers(20, 90)), int(rng.integers(20, 70))
        p["fx"] = float(rng.uniform(0.6, 1.5) * p["W"])
        p["n"] = int(rng.integers(1, 4))
        p["radius"] = float(rng.uniform(1.5, 4))
        p["step"] = float(10 ** rng.uniform(-3.3, -2))
        p["fast"] = bool(rng.integers(2))
        p["background"] = float(rng.uniform(0, 1))
        out.append(p)
    return out


PARAMETERS = case_parameters()


@pytest.mark.parametrize("case", range(N_CASES))
def test_every_image_path_against_the_oracle(gpu, oracle_mod, case):
    p = PARAMETERS[case]
    if p["dense"]:
        tree = synth.dense_tree(p["tree"]["levels"], p["fmt"], seed=p["seed"], sigma="lognormal", coeff_std=0.5,
                                zero_fraction=p["tree"]["zero_fraction"])
    else:
        tree = synth.shell_tree(data_format=p["fmt"], seed=p["seed"], **p["tree"])
    W, H, fx, n = p["W"], p["H"], p["fx"], p["n"]
    poses = synth.orbit_poses(n, seed=p["seed"] % 999, radius=p["radius"])
    opt = options(tree, step_size=p["step"], fast=p["fast"], background_brightness=p["background"])
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = np.stack([oracle_mod.volume_render_image(ot, c2w, fx, fx, W, H, opt, n_threads=8) for c2w in poses])
    go = torch.randn(n, H, W, 3, generator=torch.Generator().manual_seed(p["seed"] % 77)) * 1e-2
    want_g = sum(oracle_mod.volume_render_image_backward(ot, c2w, fx, fx, W, H, opt, go[i])
                 for i, c2w in enumerate(poses))
    ref = torch.rand(H, W, 3, generator=torch.Generator().manual_seed(p["seed"] % 55))
    want_se = oracle_mod.se_grad_image(ot, poses[0], fx, fx, W, H, ref, opt, n_threads=8)
    dev = on_gpu(tree, gpu)
    cam = cam_spec(torch.stack(poses).to(gpu), W, H, fx)
    cam1 = cam_spec(poses[0].to(gpu), W, H, fx)
    plain = dev._spec()
    marked = dev._spec()
    marked.child_marks = C.mark_empty_leaves(plain)
    # marks made with the case's own sigma_thresh: the forward kernels shade every leaf they let through
    decided = dev._spec()
    decided.child_marks = C.mark_empty_leaves(plain, opt.sigma_thresh)
    decided.child_marks_thresh = opt.sigma_thresh
    failures = []

    def check_grad(tag, got, ref_grad):
        err, ok = grad_close(got.cpu().numpy(), ref_grad)
        if not ok:
            failures.append(f"{tag}: {err:.3e}")

    for flags in (0, 4, 8):
        for spec, name in ((plain, "plain"), (marked, "marked"), (decided, "decided")):
            tag = f"flags{flags}/{name}"
            C.set_debug_flags(flags)
            try:
                if not np.array_equal(C.volume_render_images(spec, cam, opt).cpu().numpy(), want):
                    failures.append(f"{tag}: picture differs")
                if name == "decided" and flags != 0:
                    continue     # (the other paths leave such marks aside or use them as plain marks: once is enough)
                out, notes = C.volume_render_images_noted(spec, cam, opt)
                if not np.array_equal(out.cpu().numpy(), want):
                    failures.append(f"{tag}: noted picture differs")
                check_grad(f"{tag}: gradient from notes",
                           C.volume_render_images_backward_noted(spec, cam, opt, go.to(gpu), notes), want_g)
                got = C.se_grad_persp(spec, cam1, opt, ref.to(gpu), workspace=True)
                if not np.array_equal(got[0].cpu().numpy(), want_se[0]):
                    failures.append(f"{tag}: se_grad colour differs")
                check_grad(f"{tag}: se_grad gradient", got[1], want_se[1])
                check_grad(f"{tag}: se_grad hessian", got[2], want_se[2])
                if flags == 0:   # the marching kernels do not depend on the flags
                    for workspace in (True, False):
                        check_grad(f"{tag}: marching gradient (workspace {workspace})",
                                   C.volume_render_images_backward(spec, cam, opt, go.to(gpu), workspace=workspace),
                                   want_g)
                    got = C.se_grad_persp(spec, cam1, opt, ref.to(gpu), workspace=False)
                    if not np.array_equal(got[0].cpu().numpy(), want_se[0]):
                        failures.append(f"{tag}: marching se_grad colour differs")
                    check_grad(f"{tag}: marching se_grad gradient", got[1], want_se[1])
                    check_grad(f"{tag}: marching se_grad hessian", got[2], want_se[2])
            finally:
                C.set_debug_flags(0)
    # the one-ray-per-lane kernels on the same pictures (debug flag 1): forward, gradient and se_grad
    C.set_debug_flags(1)
    try:
        if not np.array_equal(C.volume_render_images(plain, cam, opt).cpu().numpy(), want):
            failures.append("generic: picture differs")
        check_grad("generic: gradient", C.volume_render_images_backward(plain, cam, opt, go.to(gpu), workspace=False), want_g)
        got = C.se_grad_persp(plain, cam1, opt, ref.to(gpu), workspace=False)
        if not np.array_equal(got[0].cpu().numpy(), want_se[0]):
            failures.append("generic: se_grad colour differs")
        check_grad("generic: se_grad gradient", got[1], want_se[1])
        check_grad("generic: se_grad hessian", got[2], want_se[2])
    finally:
        C.set_debug_flags(0)
    assert not failures, f"case {case} {p}: " + "; ".join(failures)


# Picture shapes whose grid of 16x16 blocks is a single block, a row, a column, or has an odd number
# of rings: the blocks of an image are counted ring by ring from the middle, and every pixel must be
# rendered exactly once whatever the shape.
SHAPES = [(1, 1), (16, 16), (17, 16), (200, 5), (5, 200), (33, 17), (48, 80), (81, 49), (130, 100)]


@pytest.mark.parametrize("shape", SHAPES, ids=[f"{w}x{h}" for w, h in SHAPES])
def test_every_pixel_of_odd_shaped_pictures(gpu, oracle_mod, shape):
    W, H = shape
    tree = synth.shell_tree(depth=5, n_spheres=5, data_format="SH4", seed=11, sigma_range=(5.0, 60.0))
    fx = 0.9 * max(W, H)
    poses = synth.orbit_poses(2, seed=5, radius=2.5)
    opt = options(tree, step_size=2e-3, fast=True, background_brightness=0.25)
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = np.stack([oracle_mod.volume_render_image(ot, c2w, fx, fx, W, H, opt, n_threads=8) for c2w in poses])
    go = torch.randn(2, H, W, 3, generator=torch.Generator().manual_seed(3)) * 1e-2
    want_g = sum(oracle_mod.volume_render_image_backward(ot, c2w, fx, fx, W, H, opt, go[i])
                 for i, c2w in enumerate(poses))
    dev = on_gpu(tree, gpu)
    spec = dev._spec()
    cam = cam_spec(torch.stack(poses).to(gpu), W, H, fx)
    assert np.array_equal(C.volume_render_images(spec, cam, opt).cpu().numpy(), want)
    one = C.volume_render_image(spec, cam_spec(poses[1].to(gpu), W, H, fx), opt)
    assert np.array_equal(one.cpu().numpy(), want[1])
    for workspace in (True, False):
        got = C.volume_render_images_backward(spec, cam, opt, go.to(gpu), workspace=workspace)
        err, ok = grad_close(got.cpu().numpy(), want_g)
        assert ok, f"{W}x{H} workspace {workspace}: {err:.3e}"
