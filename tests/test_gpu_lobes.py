"""Trees of lobes -- spherical gaussians (data_format SGn) and anisotropic ones (ASGn), svox/helpers.py:384-437;
bases rt_kernel.cu:120-139 -- on the wavefront-per-tile octree kernels: every render path against the oracle,
for the basis sizes those kernels are built for, and the hand-over to the one-ray-per-lane kernels for the
sizes they are not.

Bars: pictures bit for bit, gradients within 1e-4 relative (util.grad_close)."""
import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import cam_spec, grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu


def lobe_tree(n_lobes, seed, depth=6, kind="SG"):
    """A sparse shell tree whose records are read as n_lobes spherical gaussians ([lambda, mu] each) or
    anisotropic ones ([lambda_x, lambda_y, an orthonormal frame])."""
    tree = synth.shell_tree(depth=depth, n_spheres=5, data_format=f"{kind}{n_lobes}", seed=seed, sigma_range=(5.0, 80.0))
    g = torch.Generator().manual_seed(seed + 17)
    if kind == "SG":
        lobes = torch.cat([torch.rand(n_lobes, 1, generator=g) * 4, synth.unit_vectors(n_lobes, g)], dim=1)
    else:
        frames = torch.linalg.qr(torch.randn(n_lobes, 3, 3, generator=g))[0].reshape(n_lobes, 9)
        lobes = torch.cat([torch.rand(n_lobes, 2, generator=g) * 3, frames], dim=1)
    del tree.extra_data
    tree.register_buffer("extra_data", lobes)
    return tree


@pytest.mark.parametrize("kind, n_lobes", [("SG", 1), ("SG", 4), ("SG", 9), ("SG", 16), ("SG", 25),
                                           ("ASG", 4), ("ASG", 9), ("ASG", 25)])
def test_lobes_on_the_octree_kernels(gpu, oracle_mod, kind, n_lobes):
    tree = lobe_tree(n_lobes, seed=3 + n_lobes, kind=kind)
    n = 3000
    rays = synth.sphere_rays(n, seed=4)
    W, H, fx = 70, 50, 60.0
    poses = synth.orbit_poses(2, seed=6, radius=2.5)
    ot = oracle_mod.Tree.from_n3tree(tree)
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(5)) * 1e-2
    gi = torch.randn(2, H, W, 3, generator=torch.Generator().manual_seed(6)) * 1e-2
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(7))
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    cam = cam_spec(torch.stack(poses).to(gpu), W, H, fx)
    for fast in (True, False):
        opt = options(tree, step_size=2e-3, fast=fast)
        assert C.octree_kernels_serve(dev._spec(), opt)
        want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
        want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
        want_img = np.stack([oracle_mod.volume_render_image(ot, c2w, fx, fx, W, H, opt, n_threads=8) for c2w in poses])
        want_gi = sum(oracle_mod.volume_render_image_backward(ot, c2w, fx, fx, W, H, opt, gi[i])
                      for i, c2w in enumerate(poses))
        want_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=8)
        plain = dev._spec()
        marked = dev._spec()
        marked.child_marks = C.mark_empty_leaves(plain)
        for flags in (0, 2, 4, 8, 1):     # the library's choice; batches run like large ones; one / two wavefronts per tile; generic
            for spec in (plain, marked):
                C.set_debug_flags(flags)
                try:
                    tag = (kind, n_lobes, fast, flags, spec is marked)
                    assert np.array_equal(C.volume_render(spec, rs, opt).cpu().numpy(), want), tag
                    assert np.array_equal(C.volume_render_images(spec, cam, opt).cpu().numpy(), want_img), tag
                    out, notes = C.volume_render_noted(spec, rs, opt)
                    assert np.array_equal(out.cpu().numpy(), want), tag
                    for got in (C.volume_render_backward_noted(spec, rs, opt, go.to(gpu), notes),
                                C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=True),
                                C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=False)):
                        err, ok = grad_close(got.cpu().numpy(), want_g)
                        assert ok, (tag, err)
                    for workspace in (True, False):
                        got = C.volume_render_images_backward(spec, cam, opt, gi.to(gpu), workspace=workspace)
                        err, ok = grad_close(got.cpu().numpy(), want_gi)
                        assert ok, (tag, "image", workspace, err)
                        se = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=workspace)
                        assert np.array_equal(se[0].cpu().numpy(), want_se[0]), (tag, "se colour", workspace)
                        for k in (1, 2):
                            err, ok = grad_close(se[k].cpu().numpy(), want_se[k])
                            assert ok, (tag, "se", k, workspace, err)
                finally:
                    C.set_debug_flags(0)


def test_which_kernels_serve_which_trees(gpu):
    """The wavefront-per-tile kernels take fp32 trees with RGBA, SH, SG or ASG records of 1, 4, 9, 16 or 25 basis
    functions, for any range of components; everything else goes to the one-ray-per-lane kernels."""
    def serve(tree, **kw):
        dev = on_gpu(tree, gpu)
        return C.octree_kernels_serve(dev._spec(), options(tree, **kw))
    assert serve(synth.dense_tree(2, "RGBA", seed=1))
    assert serve(synth.dense_tree(2, "SH9", seed=1))
    assert serve(synth.dense_tree(2, "SH9", seed=1), density_softplus=True)
    assert serve(synth.dense_tree(2, "SH9", seed=1), min_comp=1, max_comp=3)
    assert serve(synth.dense_tree(2, "SH9", seed=1), min_comp=2, max_comp=1)         # the empty range: mid grey
    assert not serve(synth.dense_tree(2, "SH4", seed=1, dtype=torch.float64))
    assert serve(lobe_tree(9, seed=2, depth=4))
    assert not serve(lobe_tree(5, seed=2, depth=4))                       # no kernel built for five lobes
    assert serve(lobe_tree(4, seed=2, depth=4, kind="ASG"))
    assert not serve(lobe_tree(6, seed=2, depth=4, kind="ASG"))
    assert serve(svox.N3Tree(N=3, data_format="SH4", init_refine=1))          # other branching factors: same kernels, float walk
    assert not serve(svox.N3Tree(N=3, data_format="SH4", init_refine=1, dtype=torch.float64))


@pytest.mark.parametrize("op", ["sum", "max"])
def test_weight_accumulation_on_a_spherical_gaussian_tree(gpu, oracle_mod, op):
    """accumulate_weights (svox/svox.py:1136-1158, rt_kernel.cu:298-304) through the octree forward kernel
    of the spherical-gaussian policy, and the Python renderer end to end (autograd included)."""
    tree = lobe_tree(9, seed=21)
    rays = synth.sphere_rays(2000, seed=8)
    opt = options(tree, step_size=2e-3, fast=True)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ot.weight_accum = np.zeros(tree.child.shape, dtype=np.float32)
    ot.weight_accum_max = op == "max"
    want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    assert ot.weight_accum.max() > 0
    dev = on_gpu(tree, gpu)
    dev.data.requires_grad_(True)
    renderer = svox.VolumeRenderer(dev, step_size=2e-3)
    dev_rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.viewdirs.to(gpu))
    with torch.no_grad():
        with dev.accumulate_weights(op=op) as accum:
            out = renderer(dev_rays, fast=True)
            got = accum.value.cpu().numpy()
    assert np.array_equal(out.cpu().numpy(), want)
    if op == "max":
        assert np.array_equal(got, ot.weight_accum)
    else:
        assert np.abs(got - ot.weight_accum).max() <= 1e-5 * max(1.0, np.abs(ot.weight_accum).max())
    # the gradient through autograd (notes taken by the forward pass)
    go = torch.randn(2000, 3, generator=torch.Generator().manual_seed(4)) * 1e-2
    ot.weight_accum = None
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    renderer(dev_rays, fast=True).backward(go.to(gpu))
    err, ok = grad_close(dev.data.grad.cpu().numpy(), want_g)
    assert ok, err
