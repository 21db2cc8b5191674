"""GPU parity of the rendering operators against the CPU oracle.

Bars: rendered colours within 1e-5 absolute (fp32) -- in fact the kernels and the oracle share every
rounding step, so the fp32 comparisons below demand exact equality; gradients within 1e-4 relative
(atomic summation order differs); visit counters exact.
"""
import json
import os

import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import cam_spec, grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def render_both(gpu, oracle_mod, tree, rays, opt, generic=0):
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref, ref_stats = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt, want_stats=True)
    dev = on_gpu(tree, gpu)
    C.set_debug_flags(generic)
    try:
        out = C.volume_render(dev._spec(), rays_spec(rays, gpu), opt)
        stats = C.volume_render_stats(dev._spec(), rays_spec(rays, gpu), opt)
    finally:
        C.set_debug_flags(0)
    return out.cpu().numpy(), ref, stats, ref_stats, dev, ot


@pytest.mark.parametrize("generic", [0, 1])
def test_config1_rgba_forward_backward(gpu, oracle_mod, generic):
    """The smallest benchmark configuration: dense 16^3 RGBA tree, 4096 sphere rays, step 1e-3, white background."""
    tree = synth.dense_tree(3, "RGBA", seed=0)
    rays = synth.sphere_rays(4096, seed=0)
    opt = options(tree, step_size=1e-3, background_brightness=1.0)
    out, ref, stats, ref_stats, dev, ot = render_both(gpu, oracle_mod, tree, rays, opt, generic)
    assert np.array_equal(out, ref)
    for k in ("rays", "rays_hit", "samples", "samples_shaded", "levels"):
        assert stats[k] == ref_stats[k], k
    go = torch.randn(4096, 3, generator=torch.Generator().manual_seed(1))
    ref_grad, bstats = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go,
                                                         want_stats=True)
    assert stats["samples_bwd"] == bstats["samples_bwd"] and stats["samples_bwd_pos"] == bstats["samples_bwd_pos"]
    C.set_debug_flags(generic)
    try:
        grad = C.volume_render_backward(dev._spec(), rays_spec(rays, gpu), opt, go.to(gpu))
    finally:
        C.set_debug_flags(0)
    err, ok = grad_close(grad.cpu().numpy(), ref_grad)
    assert ok, err


@pytest.mark.parametrize("fmt", ["SH1", "SH4", "SH9", "SH16", "SH25", "RGBA"])
@pytest.mark.parametrize("fast", [False, True])
def test_sparse_tree_batch_all_formats(gpu, oracle_mod, fmt, fast):
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format=fmt, seed=21, sigma_range=(20.0, 200.0))
    rays = synth.sphere_rays(3000, seed=5)
    # a few rays that miss the cube, start inside it, or run along an axis
    o = rays.origins.clone()
    d = rays.dirs.clone()
    o[:50] += 3.0
    o[50:100] = torch.rand(50, 3, generator=torch.Generator().manual_seed(2))
    d[100:110] = torch.tensor([0.0, 0.0, 1.0])
    o[100:110] = torch.tensor([0.3, 0.6, -0.5])
    rays = svox.Rays(o.contiguous(), d.contiguous(), d.clone())
    opt = options(tree, step_size=5e-4, fast=fast)
    out, ref, stats, ref_stats, dev, ot = render_both(gpu, oracle_mod, tree, rays, opt)
    assert np.array_equal(out, ref)
    assert stats["samples"] == ref_stats["samples"] and stats["samples_shaded"] == ref_stats["samples_shaded"]
    C.set_debug_flags(1)
    try:
        out_generic = C.volume_render(dev._spec(), rays_spec(rays, gpu), opt).cpu().numpy()
    finally:
        C.set_debug_flags(0)
    assert np.array_equal(out_generic, ref)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(8)) * 1e-2
    ref_grad = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    grad = C.volume_render_backward(dev._spec(), rays_spec(rays, gpu), opt, go.to(gpu))
    err, ok = grad_close(grad.cpu().numpy(), ref_grad)
    assert ok, err


@pytest.mark.parametrize("ndc", [False, True])
def test_image_render_and_backward(gpu, oracle_mod, ndc):
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format="SH9", seed=33,
                            geometry="noise" if ndc else "spheres")
    W, H, fx = 75, 53, 60.0     # not multiples of the 16x16 tile
    if ndc:
        c2w = torch.tensor([[1.0, 0, 0, 0.1], [0, 1, 0, -0.05], [0, 0, 1, 0.3]])
        kw = dict(ndc=svox.NDCConfig(W, H, fx))
        tree.invradius.data[:] = 0.5
        tree.offset.data[:] = 0.5      # NDC cube [-1,1]^3 -> [0,1]^3
    else:
        c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0]
        kw = {}
    opt = options(tree, step_size=1e-3, **kw)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref, ref_stats = oracle_mod.volume_render_image(ot, c2w, fx, fx, W, H, opt, want_stats=True)
    dev = on_gpu(tree, gpu)
    cam = cam_spec(c2w, W, H, fx, device=gpu)
    out = C.volume_render_image(dev._spec(), cam, opt)
    assert out.shape == (H, W, 3)
    assert np.array_equal(out.cpu().numpy(), ref)
    for flags in (4, 8):     # either forward kernel for launches of this size, whatever the choice would be
        C.set_debug_flags(flags)
        try:
            assert torch.equal(C.volume_render_image(dev._spec(), cam, opt), out), flags
        finally:
            C.set_debug_flags(0)
    assert ref_stats["rays_hit"] > 0.2 * W * H
    stats = C.volume_render_stats(dev._spec(), cam, opt)
    assert stats["samples"] == ref_stats["samples"] and stats["rays"] == W * H
    go = torch.randn(H, W, 3, generator=torch.Generator().manual_seed(3))
    ref_grad = oracle_mod.volume_render_image_backward(ot, c2w, fx, fx, W, H, opt, go)
    grad = C.volume_render_image_backward(dev._spec(), cam, opt, go.to(gpu))
    err, ok = grad_close(grad.cpu().numpy(), ref_grad)
    assert ok, err
    # the same without a workspace (the second march walks the tree again)
    grad = C.volume_render_image_backward(dev._spec(), cam, opt, go.to(gpu), workspace=False)
    err, ok = grad_close(grad.cpu().numpy(), ref_grad)
    assert ok, err
    # and from the notes of a forward pass that keeps them
    noted, notes = C.volume_render_images_noted(dev._spec(), cam, opt)
    assert notes is not None and torch.equal(noted, out)
    grad = C.volume_render_images_backward_noted(dev._spec(), cam, opt, go.to(gpu), notes)
    err, ok = grad_close(grad.cpu().numpy(), ref_grad)
    assert ok, err
    # the batch kernels on the oracle's pixel rays give the same picture
    ro, rd, rv = oracle_mod.image_rays(oracle_mod.Tree.from_n3tree(tree), c2w, fx, fx, W, H, opt)
    assert np.isfinite(rd).all()


def test_generic_options_double_and_lobes(gpu, oracle_mod):
    """fp64, SG / ASG lobes, component ranges, softplus, padding, N = 3: the generic kernels."""
    g = torch.Generator().manual_seed(6)
    rays = synth.sphere_rays(1500, seed=9)
    cases = []
    t = synth.dense_tree(2, "SH9", seed=3, sigma="lognormal", coeff_std=0.5)
    cases.append(("sh9_comp_range", t, dict(min_comp=1, max_comp=3), torch.float32))
    cases.append(("sh9_grey", t, dict(min_comp=2, max_comp=1), torch.float32))
    cases.append(("sh9_softplus_pad", t, dict(density_softplus=True, rgb_padding=0.001), torch.float32))
    lobes = torch.cat([torch.rand(5, 1, generator=g) * 4, synth.unit_vectors(5, g)], dim=1)
    t = svox.N3Tree(data_format="SG5", init_refine=2, extra_data=lobes)
    t.data.data.normal_(generator=g)
    t.data.data[..., -1] = t.data.data[..., -1].abs() * 5
    cases.append(("sg5", t, {}, torch.float32))
    frames = torch.linalg.qr(torch.randn(4, 3, 3, generator=g))[0].reshape(4, 9)
    t = svox.N3Tree(data_format="ASG4", init_refine=2, extra_data=torch.cat([torch.rand(4, 2, generator=g) * 3, frames], 1))
    t.data.data.normal_(generator=g)
    t.data.data[..., -1] = t.data.data[..., -1].abs() * 5
    cases.append(("asg4", t, {}, torch.float32))
    t = svox.N3Tree(N=3, data_format="SH4", init_refine=2)
    t.data.data.normal_(generator=g)
    t.data.data[..., -1] = t.data.data[..., -1].abs() * 8
    cases.append(("n3_sh4", t, {}, torch.float32))
    t = synth.dense_tree(2, "SH4", seed=8, sigma="lognormal", dtype=torch.float64)
    cases.append(("sh4_double", t, {}, torch.float64))
    for name, tree, kw, dt in cases:
        r = svox.Rays(rays.origins.to(dt), rays.dirs.to(dt), rays.viewdirs.to(dt))
        opt = options(tree, step_size=2e-3, **kw)
        for generic in (0, 1):       # the kernels the library picks, then the one-ray-per-lane kernels for every case
            out, ref, stats, ref_stats, dev, ot = render_both(gpu, oracle_mod, tree, r, opt, generic)
            if "softplus" in name:
                assert np.abs(out - ref).max() <= 1e-5, name    # logf comes from two math libraries
            else:
                assert np.array_equal(out, ref), (name, generic)
            go = torch.randn(out.shape, generator=torch.Generator().manual_seed(1), dtype=dt)
            ref_grad = oracle_mod.volume_render_backward(ot, r.origins, r.dirs, r.viewdirs, opt, go)
            C.set_debug_flags(generic)
            try:
                grad = C.volume_render_backward(dev._spec(), rays_spec(r, gpu), opt, go.to(gpu))
            finally:
                C.set_debug_flags(0)
            err, ok = grad_close(grad.cpu().numpy(), ref_grad, what=f"{name} generic {generic}")
            assert ok, (name, generic, err)


@pytest.mark.parametrize("fmt,lo,hi", [("SH9", 1, 3), ("SH9", 2, 1), ("SH16", 4, 15), ("SH4", 0, 0), ("SG9", 2, 6),
                                       ("ASG4", 1, 2)])
def test_component_ranges_on_the_wavefront_kernels(gpu, oracle_mod, fmt, lo, hi):
    """A range of basis components (rt_kernel.cu:286-288; min_comp > max_comp renders mid grey) on the wavefront-per-tile
    kernels: every call -- forward on one and two wavefronts per tile, noted forward and replay, marching backward with
    and without a workspace, se_grad from notes and marching, an image and its gradient -- against the oracle."""
    g = torch.Generator().manual_seed(21)
    if fmt.startswith("SH"):
        tree = synth.shell_tree(depth=5, n_spheres=4, data_format=fmt, seed=4, sigma_range=(5.0, 80.0))
    else:
        n = int(fmt[-1])
        if fmt.startswith("SG"):
            extra = torch.cat([torch.rand(n, 1, generator=g) * 4 + 0.5, synth.unit_vectors(n, g)], dim=1)
        else:
            frames = torch.linalg.qr(torch.randn(n, 3, 3, generator=g))[0].reshape(n, 9)
            extra = torch.cat([torch.rand(n, 2, generator=g) * 3, frames], 1)
        tree = svox.N3Tree(data_format=fmt, init_refine=3, extra_data=extra)
        tree.data.data.normal_(0, 0.7, generator=g)
        tree.data.data[..., -1] = tree.data.data[..., -1].abs() * 6 * (torch.rand(tree.child.shape, generator=g) < 0.6)
    rays = synth.sphere_rays(1200, seed=13)
    opt = options(tree, step_size=2e-3, min_comp=lo, max_comp=hi)
    ot = oracle_mod.Tree.from_n3tree(tree)
    dev = on_gpu(tree, gpu)
    assert C.octree_kernels_serve(dev._spec(), opt) == 1
    rs = rays_spec(rays, gpu)
    want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    go = torch.randn(1200, 3, generator=g) * 1e-2
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    ref = torch.rand(1200, 3, generator=g)
    want_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=8)
    for flags in (0, 2, 4, 8):
        C.set_debug_flags(flags)
        try:
            assert np.array_equal(C.volume_render(dev._spec(), rs, opt).cpu().numpy(), want), flags
            out, notes = C.volume_render_noted(dev._spec(), rs, opt)
            assert notes is not None and np.array_equal(out.cpu().numpy(), want), flags
            err, ok = grad_close(C.volume_render_backward_noted(dev._spec(), rs, opt, go.to(gpu), notes).cpu().numpy(),
                                 want_g, what=f"range notes flags {flags}")
            assert ok, (flags, err)
            for workspace in (True, False):
                err, ok = grad_close(C.volume_render_backward(dev._spec(), rs, opt, go.to(gpu),
                                                              workspace=workspace).cpu().numpy(), want_g,
                                     what=f"range backward flags {flags} workspace {workspace}")
                assert ok, (flags, workspace, err)
                got = C.se_grad(dev._spec(), rs, ref.to(gpu), opt, workspace=workspace)
                assert np.array_equal(got[0].cpu().numpy(), want_se[0]), (flags, workspace)
                for what, x, w in zip(("gradient", "hessian"), got[1:], want_se[1:3]):
                    err, ok = grad_close(x.cpu().numpy(), w, what=f"range se_grad {what} flags {flags}")
                    assert ok, (flags, workspace, what, err)
        finally:
            C.set_debug_flags(0)
    # one picture and its gradient through the image kernels
    W, H, fx = 48, 40, 60.0
    c2w = synth.orbit_poses(1, seed=3, radius=2.5)[0]
    want_img = oracle_mod.volume_render_image(ot, c2w, fx, fx, W, H, opt)
    cam = cam_spec(c2w.to(gpu), W, H, fx)
    assert np.array_equal(C.volume_render_image(dev._spec(), cam, opt).cpu().numpy(), want_img)
    go_img = torch.randn(H, W, 3, generator=g) * 1e-2
    want_gi = oracle_mod.volume_render_image_backward(ot, c2w, fx, fx, W, H, opt, go_img)
    err, ok = grad_close(C.volume_render_image_backward(dev._spec(), cam, opt, go_img.to(gpu)).cpu().numpy(), want_gi,
                         what="range image gradient")
    assert ok, err


def irregular_tree(N, fmt, seed, rounds=3):
    """A tree of branching factor N refined at random (a few thousand leaves of several sizes), about half of them
    with density."""
    g = torch.Generator().manual_seed(seed)
    tree = svox.N3Tree(N=N, data_format=fmt, init_refine=1, depth_limit=6)
    for _ in range(rounds):
        leaves = tree._all_leaves()
        keep = min(0.5, 40.0 / leaves.shape[0] * (1 + _))          # (a round adds some 40 to 120 nodes of N^3 cells)
        pick = torch.rand(leaves.shape[0], generator=g) < keep
        if pick.any():
            tree.refine(sel=tuple(leaves[pick].T))
    tree.data.data.normal_(0, 0.5, generator=g)
    sigma = tree.data.data[..., -1]
    sigma.copy_(torch.exp(torch.randn(sigma.shape, generator=g)) * 8 * (torch.rand(sigma.shape, generator=g) < 0.5))
    return tree


@pytest.mark.parametrize("N,fmt", [(3, "SH4"), (3, "RGBA"), (4, "SH9"), (5, "SH1")])
def test_other_branching_factors_on_the_wavefront_kernels(gpu, oracle_mod, N, fmt):
    """fp32 trees with N != 2 (common.cuh:52-90 with N as a scalar; AT_DISPATCH over the same kernels, rt_kernel.cu:1029)
    run on the wavefront-per-tile kernels: the walk is the reference's floating-point walk from the root (no integer
    formulation is exact there), everything else -- rounds, shade list, record lists, notes, replays -- is shared with
    the octrees.  Forward pictures equal the oracle's bit for bit on every forward kernel; gradients, se_grad and the
    image paths meet the plain gate."""
    tree = irregular_tree(N, fmt, seed=40 + N)
    assert tree.n_leaves > 300
    n = 2500
    rays = synth.sphere_rays(n, seed=N)
    opt = options(tree, step_size=2e-3, fast=True, background_brightness=0.25)
    ot = oracle_mod.Tree.from_n3tree(tree)
    want, want_stats = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt, want_stats=True)
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(2)) * 1e-2
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go, n_threads=8)
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(7))
    want_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=8)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    spec = dev._spec()
    assert C.octree_kernels_serve(spec, opt)
    marked = dev._spec()
    marked.child_marks = C.mark_empty_leaves(spec)
    stats = C.volume_render_stats(spec, rs, opt)
    for k in ("rays", "rays_hit", "samples", "samples_shaded", "levels", "samples_tail"):
        assert stats[k] == want_stats[k], k
    assert stats["samples_shaded"] > 1000

    def close(got, ref_, what):
        err, ok = grad_close(got.cpu().numpy(), ref_, what=what)
        assert ok, (what, err)

    for flags in (0, 2, 4, 8):
        C.set_debug_flags(flags)
        try:
            for sp in (spec, marked):
                assert np.array_equal(C.volume_render(sp, rs, opt).cpu().numpy(), want), flags
            out, notes = C.volume_render_noted(spec, rs, opt)
            assert notes is not None and np.array_equal(out.cpu().numpy(), want)
            close(C.volume_render_backward_noted(spec, rs, opt, go.to(gpu), notes), want_g, f"N={N} replay flags {flags}")
            if flags in (0, 2):
                for workspace in (True, False):
                    close(C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=workspace), want_g,
                          f"N={N} backward flags {flags} workspace {workspace}")
                    got = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=workspace)
                    assert np.array_equal(got[0].cpu().numpy(), want_se[0])
                    close(got[1], want_se[1], f"N={N} se_grad gradient flags {flags} workspace {workspace}")
                    close(got[2], want_se[2], f"N={N} se_grad hessian flags {flags} workspace {workspace}")
        finally:
            C.set_debug_flags(0)
    # the one-ray-per-lane kernels agree bit for bit on the picture
    C.set_debug_flags(1)
    try:
        assert np.array_equal(C.volume_render(spec, rs, opt).cpu().numpy(), want)
    finally:
        C.set_debug_flags(0)
    # images, through the renderer
    c2w = synth.orbit_poses(2, seed=4, radius=2.5)
    W, H, fx = 90, 70, 80.0
    want_img = np.stack([oracle_mod.volume_render_image(ot, p, fx, fx, W, H, opt) for p in c2w])
    r = svox.VolumeRenderer(dev, step_size=2e-3, background_brightness=0.25)
    with torch.no_grad():
        assert np.array_equal(r.render_persp(torch.stack(c2w).to(gpu), width=W, height=H, fx=fx, fast=True).cpu().numpy(), want_img)
    igo = torch.randn(H, W, 3, generator=torch.Generator().manual_seed(3)) * 1e-2
    want_ig = oracle_mod.volume_render_image_backward(ot, c2w[0], fx, fx, W, H, opt, igo)
    dev.data.grad = None
    r.render_persp(c2w[0].to(gpu), width=W, height=H, fx=fx, fast=True).backward(igo.to(gpu))
    close(dev.data.grad, want_ig, f"N={N} image autograd")
    dev.data.grad = None


@pytest.mark.parametrize("generic", [0, 1])
def test_weight_accumulation(gpu, oracle_mod, generic):
    """accumulate_weights (sum / max) through the renderer, batch and image, thresholds and early stop
    included: the octree kernels and the generic ones against the oracle."""
    cases = [(synth.dense_tree(2, "RGBA", seed=14), synth.sphere_rays(500, seed=2), False),
             (synth.shell_tree(depth=6, n_spheres=6, data_format="SH9", seed=4), synth.sphere_rays(4000, seed=3), True)]
    c2w = synth.orbit_poses(1, seed=6, radius=2.5)[0]
    W, H, fx = 70, 50, 60.0
    for tree, rays, fast in cases:
        opt = options(tree, fast=fast)
        for op in ("sum", "max"):
            ot = oracle_mod.Tree.from_n3tree(tree)
            ot.weight_accum = np.zeros(tree.child.shape, dtype=np.float32)
            ot.weight_accum_max = op == "max"
            oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
            oracle_mod.volume_render_image(ot, c2w, fx, fx, W, H, opt)
            assert ot.weight_accum.max() > 0
            dev = on_gpu(tree, gpu)
            renderer = svox.VolumeRenderer(dev)
            C.set_debug_flags(generic)
            try:
                with dev.accumulate_weights(op=op) as accum:
                    renderer(svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.viewdirs.to(gpu)), fast=fast)
                    renderer.render_persp(c2w.to(gpu), width=W, height=H, fx=fx, fast=fast)
                    got = accum.value.cpu().numpy()
            finally:
                C.set_debug_flags(0)
            if op == "max":
                assert np.array_equal(got, ot.weight_accum)
            else:
                assert np.abs(got - ot.weight_accum).max() <= 1e-5 * max(1.0, np.abs(ot.weight_accum).max())


def test_toy_example_through_python_api(gpu):
    """The reference's documentation example (docs/source/ex_opt_toy.py) run through this package
    on the GPU reproduces its recorded output (docs/source/ex_opt_toy.rst:20-44)."""
    gold = json.load(open(os.path.join(HERE, "golden", "ex_opt_toy.json")))
    lr = gold["setup"]["lr"]
    t = svox.N3Tree(device=gpu, data_format="SH1")
    t[0, 0, 0, :-1] = 0.0
    t[0, 0, 0, -1:] = 0.5
    r = svox.VolumeRenderer(t)
    target = torch.tensor([gold["setup"]["target"]], device=gpu)
    ray_ori = torch.tensor([gold["setup"]["ray_origin"]], device=gpu)
    ray_dir = torch.tensor([gold["setup"]["ray_dir"]], device=gpu)
    ray = svox.Rays(origins=ray_ori, dirs=ray_dir, viewdirs=ray_dir)

    def phase():
        printed = []
        for i in range(20):
            rend = r(ray, cuda=True)
            if i % 2 == 0:
                printed.append(rend.detach()[0].cpu().numpy())
            ((rend - target) ** 2).sum().backward()
            t.data.data -= lr * t.data.grad
            t.zero_grad()
        return np.array(printed)

    p1 = phase()
    t.expand("SH4")
    assert repr(r.data_format) == "SH4"
    p2 = phase()
    assert np.abs(p1 - np.array(gold["phase1"])).max() < 2e-7
    assert np.abs(p2 - np.array(gold["phase2"])).max() < 2e-7


def test_render_persp_autograd_and_empty(gpu, oracle_mod):
    tree = on_gpu(synth.dense_tree(2, "SH4", seed=2, sigma="lognormal"), gpu)
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    c2w = synth.orbit_poses(1, seed=1, radius=3.0)[0].to(gpu)
    img = r.render_persp(c2w, width=40, height=30, fx=50.0, fast=True)
    assert img.shape == (30, 40, 3) and img.requires_grad
    img.sum().backward()
    assert tree.data.grad is not None and tree.data.grad.shape == tree.data.shape
    assert torch.isfinite(tree.data.grad).all() and tree.data.grad.abs().sum() > 0
    rays = svox.Rays(torch.zeros(0, 3, device=gpu), torch.zeros(0, 3, device=gpu), torch.zeros(0, 3, device=gpu))
    assert r(rays).shape == (0, 3)
    # permuting rays permutes the output
    rr = synth.sphere_rays(256, seed=3)
    perm = torch.randperm(256, generator=torch.Generator().manual_seed(0))
    a = r(svox.Rays(rr.origins.to(gpu), rr.dirs.to(gpu), rr.viewdirs.to(gpu))).detach()
    b = r(svox.Rays(rr.origins[perm].to(gpu), rr.dirs[perm].to(gpu), rr.viewdirs[perm].to(gpu))).detach()
    assert torch.equal(a[perm.to(gpu)], b)


def test_several_poses_in_one_launch_equal_separate_calls(gpu, oracle_mod):
    tree = on_gpu(synth.shell_tree(depth=6, n_spheres=5, data_format="SH16", seed=41), gpu)
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    poses = torch.stack(synth.orbit_poses(3, seed=2, radius=2.2)).to(gpu)          # (3, 3, 4)
    W, H, fx = 61, 44, 70.0
    batch = r.render_persp(poses, width=W, height=H, fx=fx, fast=True)
    assert batch.shape == (3, H, W, 3)
    singles = [r.render_persp(p, width=W, height=H, fx=fx, fast=True) for p in poses]
    for i in range(3):
        assert torch.equal(batch[i], singles[i])
    # homogeneous (n, 4, 4) poses give the same pictures
    hom = torch.cat([poses, torch.tensor([0.0, 0, 0, 1], device=gpu).expand(3, 1, 4)], dim=1).contiguous()
    assert torch.equal(r.render_persp(hom, width=W, height=H, fx=fx, fast=True), batch)
    go = torch.randn(3, H, W, 3, generator=torch.Generator().manual_seed(0)).to(gpu)
    batch.backward(go)
    g_batch = tree.data.grad.clone()
    tree.data.grad = None
    for i in range(3):
        singles[i].backward(go[i])
    err, ok = grad_close(g_batch.cpu().numpy(), tree.data.grad.cpu().numpy())
    assert ok, err


def pathological_rays():
    nan, inf = float("nan"), float("inf")
    o = [[0.5, 0.5, -1.0], [0.5, 0.5, -1.0], [nan, 0.5, 0.5], [0.5, 0.5, -1.0], [1e8, 1e8, 1e8], [0.0, 0.0, 0.0],
         [1.0, 1.0, 1.0], [0.5, 0.5, 0.5], [0.25, 0.5, -3.0], [-inf, 0.5, 0.5], [0.5, 0.5, -1.0], [0.5, 0.5, 1e30],
         [0.3, 0.3, -1e-30], [2.0, 0.5, 0.5]]
    d = [[0.0, 0.0, 0.0], [0.0, 0.0, nan], [0.0, 0.0, 1.0], [0.0, 0.0, inf], [-1.0, -1.0, -1.0], [1.0, 1.0, 1.0],
         [-1.0, -1.0, -1.0], [1e-30, 0.0, 0.0], [0.0, 0.0, 1.0], [1.0, 0.0, 0.0], [0.0, 0.0, 1e-20], [0.0, 0.0, -1.0],
         [0.0, 0.0, 1.0], [-1.0, 0.0, 0.0]]
    o = torch.tensor(o, dtype=torch.float32)
    d = torch.tensor(d, dtype=torch.float32)
    return svox.Rays(o, d, d.clone())


@pytest.mark.parametrize("fmt", ["SH4", "RGBA"])
def test_pathological_rays_end_and_match_the_oracle(gpu, oracle_mod, fmt):
    """Zero / NaN / infinite directions and origins, rays on faces and corners, origins so far away
    that t cannot advance: every ray ends, and ends the same way as in the oracle."""
    tree = synth.shell_tree(depth=5, n_spheres=4, data_format=fmt, seed=17)
    rays = pathological_rays()
    for kw in (dict(step_size=1e-3), dict(step_size=1e-9, fast=True)):
        opt = options(tree, **kw)
        out, ref, stats, ref_stats, dev, ot = render_both(gpu, oracle_mod, tree, rays, opt)
        assert np.array_equal(out, ref, equal_nan=True)
        assert stats["samples"] == ref_stats["samples"]
        for flags in (1, 2, 4, 8):     # generic kernel; refilling kernel; one wavefront per 64 rays; two
            C.set_debug_flags(flags)
            try:
                other = C.volume_render(dev._spec(), rays_spec(rays, gpu), opt).cpu().numpy()
            finally:
                C.set_debug_flags(0)
            assert np.array_equal(other, ref, equal_nan=True), flags
        go = torch.ones(rays.origins.shape[0], 3)
        ref_grad = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
        grad = C.volume_render_backward(dev._spec(), rays_spec(rays, gpu), opt, go.to(gpu)).cpu().numpy()
        finite = np.isfinite(ref_grad)
        assert np.array_equal(np.isfinite(grad), finite)
        err, ok = grad_close(np.where(finite, grad, 0.0), np.where(finite, ref_grad, 0.0))
        assert ok, err


@pytest.mark.parametrize("fmt", ["SH9", "RGBA"])
def test_backward_workspace_sizes(gpu, oracle_mod, fmt, monkeypatch):
    """The backward with a workspace (march 2 replayed from notes of march 1) for shares of the
    workspace that hold none, some and all of the rays' leaves, and without a workspace: the same
    gradient as the oracle's every time."""
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format=fmt, seed=9, sigma_range=(2.0, 20.0))
    rays = synth.sphere_rays(6000, seed=4)
    opt = options(tree, step_size=1e-3)
    ot = oracle_mod.Tree.from_n3tree(tree)
    go = torch.randn(6000, 3, generator=torch.Generator().manual_seed(5))
    want, stats = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go, want_stats=True)
    assert stats["samples_bwd_pos"] > 8 * 6000          # many rays have more than 4 and 8 such leaves
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    monkeypatch.setattr(C, "SMALL_BATCH_ROOM", 1)     # (the sizes below are meant as they stand)
    for per_ray in (0, 15, 30, 90):      # no workspace; first chunks only; some / plenty of shared chunks
        monkeypatch.setattr(C, "BACKWARD_RECORDS_PER_RAY", per_ray)
        got = C.volume_render_backward(dev._spec(), rs, opt, go.to(gpu), workspace=per_ray > 0).cpu().numpy()
        err, ok = grad_close(got, want)
        assert ok, (per_ray, err)


def test_backward_workspace_argument_handling(gpu, oracle_mod):
    """The C entry point with workspaces it cannot use (misaligned, too small for one chunk per ray)
    gives the plain backward's result; a negative size is an error."""
    import ctypes
    from svox_amd.csrc import _abi
    tree = synth.shell_tree(depth=5, n_spheres=4, data_format="SH4", seed=2, sigma_range=(2.0, 20.0))
    rays = synth.sphere_rays(1000, seed=1)
    opt = options(tree, step_size=1e-3)
    go = torch.randn(1000, 3, generator=torch.Generator().manual_seed(5))
    want = oracle_mod.volume_render_backward(oracle_mod.Tree.from_n3tree(tree), rays.origins, rays.dirs, rays.viewdirs,
                                             opt, go)
    dev = on_gpu(tree, gpu)
    lib = _abi.load_library()
    spec = C._pack_tree(dev._spec())
    rs_obj = rays_spec(rays, gpu)
    rs = C._pack_rays(rs_obj, torch.float32)
    copt = opt._pack()
    go_d = go.to(gpu)
    # 1000 chunks, 16 words of a bitmap (one bit per ray), 256 bytes of bookkeeping
    enough = 1000 * 384 + 128 + 256
    buf = torch.empty(enough + 64, dtype=torch.uint8, device=gpu)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cases = [(buf.data_ptr() + 4, enough), (buf.data_ptr(), enough - 1), (buf.data_ptr(), enough), (None, 0)]
    for ptr, nbytes in cases:
        grad = torch.full_like(dev.data.data, 7.0)
        rc = lib.svox_volume_render_backward_ws(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), go_d.data_ptr(),
                                                grad.data_ptr(), 0, ptr, nbytes, stream)
        assert rc == 0, lib.svox_last_error()
        err, ok = grad_close(grad.cpu().numpy(), want)
        assert ok, (nbytes, err)
    grad = torch.empty_like(dev.data.data)
    rc = lib.svox_volume_render_backward_ws(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), go_d.data_ptr(),
                                            grad.data_ptr(), 0, buf.data_ptr(), -1, stream)
    assert rc < 0 and b"workspace" in lib.svox_last_error()
    assert lib.svox_volume_render_backward_workspace_bytes(1000, 30) == 1000 * 2 * 384 + 128 + 256
    assert lib.svox_volume_render_backward_workspace_bytes(0, 30) == 0


@pytest.mark.parametrize("order", ["random", "image"])
@pytest.mark.parametrize("fmt", ["SH9", "RGBA"])
def test_persistent_batch_kernels_on_a_small_batch(gpu, oracle_mod, fmt, order):
    """The kernels large batches run in (several 64-ray chunks per wavefront, dealt out over the
    wavefronts, idle lanes refilled) on a batch small enough for the oracle: unrelated rays, and the
    rays of an image row by row with a ragged end."""
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format=fmt, seed=23, sigma_range=(20.0, 200.0))
    if order == "random":
        rays = synth.sphere_rays(5000 + 37, seed=9)
    else:
        c2w = synth.orbit_poses(1, seed=6, radius=2.4)[0]
        rays = svox.VolumeRenderer.persp_rays(c2w, 83, 61, 75.0)    # 5063 rays, not a multiple of 64
    rays = svox.Rays(rays.origins.contiguous(), rays.dirs.contiguous(), rays.dirs.clone())
    opt = options(tree, step_size=1e-3, fast=True)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    go = torch.randn(ref.shape, generator=torch.Generator().manual_seed(8)) * 1e-2
    ref_grad = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    colors = torch.rand(ref.shape, generator=torch.Generator().manual_seed(4))
    ref_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, colors, opt)
    dev = on_gpu(tree, gpu)
    C.set_debug_flags(2)
    try:
        out = C.volume_render(dev._spec(), rays_spec(rays, gpu), opt)
        grads = [C.volume_render_backward(dev._spec(), rays_spec(rays, gpu), opt, go.to(gpu), workspace=w)
                 for w in (True, False)]
        se = C.se_grad(dev._spec(), rays_spec(rays, gpu), colors.to(gpu), opt)
    finally:
        C.set_debug_flags(0)
    assert np.array_equal(out.cpu().numpy(), ref)
    for grad in grads:
        err, ok = grad_close(grad.cpu().numpy(), ref_grad)
        assert ok, err
    assert np.array_equal(se[0].cpu().numpy(), ref_se[0])
    for got, want in zip(se[1:], ref_se[1:]):
        err, ok = grad_close(got.cpu().numpy(), want)
        assert ok, err


@pytest.mark.parametrize("persistent", [False, True])
@pytest.mark.parametrize("fmt,fast", [("SH9", True), ("SH16", False), ("SH25", True), ("RGBA", True)])
def test_noted_forward_and_backward_from_notes(gpu, oracle_mod, fmt, fast, persistent, monkeypatch):
    """volume_render_noted gives volume_render's picture; volume_render_backward_noted gives the
    gradient from its notes alone: with room for every ray's notes, with room for some (the others are
    marched again), and with a workspace that carries another call's stamp."""
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format=fmt, seed=29, sigma_range=(20.0, 200.0))
    rays = synth.sphere_rays(4000 + 21, seed=12)
    o = rays.origins.clone()
    o[:60] += 3.0                                   # these miss the cube
    rays = svox.Rays(o.contiguous(), rays.dirs.contiguous(), rays.dirs.clone())
    opt = options(tree, step_size=1e-3, fast=fast)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    go = torch.randn(ref.shape, generator=torch.Generator().manual_seed(8)) * 1e-2
    ref_grad = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    C.set_debug_flags(2 if persistent else 0)
    try:
        monkeypatch.setattr(C, "SMALL_BATCH_ROOM", 1)     # (the sizes below are meant as they stand)
        for per_ray in (30, 15):
            monkeypatch.setattr(C, "BACKWARD_RECORDS_PER_RAY", per_ray)
            out, notes = C.volume_render_noted(dev._spec(), rs, opt)
            assert notes is not None
            assert np.array_equal(out.cpu().numpy(), ref)
            grad = C.volume_render_backward_noted(dev._spec(), rs, opt, go.to(gpu), notes)
            err, ok = grad_close(grad.cpu().numpy(), ref_grad)
            assert ok, (per_ray, err)
        # notes of other rays (another origins tensor): the stamp does not match, every ray is marched
        other = svox.Rays(rays.origins.clone(), rays.dirs, rays.viewdirs)
        grad = C.volume_render_backward_noted(dev._spec(), rays_spec(other, gpu), opt, go.to(gpu), notes)
        err, ok = grad_close(grad.cpu().numpy(), ref_grad)
        assert ok, err
    finally:
        C.set_debug_flags(0)


def test_notes_budget_follows_the_scene(gpu, oracle_mod, monkeypatch):
    """Rays through a dense tree meet more leaves with density than the starting room for notes holds:
    the first training step loses notes (those rays are marched: same gradient), the renderer gives
    the next steps more room until nothing is lost, and takes it back for rays that need none."""
    monkeypatch.setattr(C, "SMALL_BATCH_ROOM", 1)     # (without the extra room a batch this small starts with)
    tree = synth.dense_tree(5, "SH4", seed=3, sigma="lognormal", coeff_std=0.5, zero_fraction=0.0)
    rays = synth.sphere_rays(3000, seed=5)
    opt = options(tree, step_size=1e-3)
    ot = oracle_mod.Tree.from_n3tree(tree)
    go = torch.randn(3000, 3, generator=torch.Generator().manual_seed(2)) * 1e-2
    want, slack = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go,
                                                    n_threads=8, want_slack=True)
    dev = on_gpu(tree, gpu)
    dev.data.requires_grad_(True)
    r = svox.VolumeRenderer(dev, step_size=1e-3)
    dev_rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.viewdirs.to(gpu))
    factors, asked = [], []
    for _ in range(5):
        dev.data.grad = None
        factors.append(r.notes_budget.factor)
        r(dev_rays).backward(go.to(gpu))
        torch.cuda.synchronize()
        err, ok = grad_close(dev.data.grad.cpu().numpy(), want, slack=slack)
        assert ok, (factors, err)
    factors.append(r.notes_budget.records_per_ray() // C.BACKWARD_RECORDS_PER_RAY)
    assert factors[0] == 1 and factors[-1] > 1, factors
    assert factors[-1] == factors[-2], factors            # it settles
    # with the room it settled on nothing is lost any more
    out, notes = C.volume_render_noted(dev._spec(), rays_spec(rays, gpu), opt, r.notes_budget.records_per_ray())
    counter, pool = C.notes_pool_use(notes, 3000)
    assert 0 < int(counter.cpu()[0]) < pool
    # rays that miss the tree need no room: the budget goes back to where it started
    away = svox.Rays(dev_rays.origins + 5.0, dev_rays.dirs, dev_rays.viewdirs)
    for _ in range(6):
        dev.data.grad = None
        r(away).backward(go.to(gpu))
        torch.cuda.synchronize()
    assert r.notes_budget.records_per_ray() == C.BACKWARD_RECORDS_PER_RAY


def test_autograd_uses_notes_and_marches_again_after_a_write(gpu, oracle_mod):
    """renderer(rays).backward(): the gradient from the forward pass's notes equals the oracle's; if
    tree.data is written to between the two passes, the backward pass sees the tree as it then is
    (svox/renderer.py:61-63 keeps no copy either)."""
    tree = on_gpu(synth.shell_tree(depth=6, n_spheres=6, data_format="SH4", seed=31, sigma_range=(20.0, 200.0)), gpu)
    rays = synth.sphere_rays(3000, seed=3)
    rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.dirs.clone().to(gpu))
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    go = (torch.randn(3000, 3, generator=torch.Generator().manual_seed(1)) * 1e-2).to(gpu)
    opt = r._get_options(True)

    def oracle_grad():
        ot = oracle_mod.Tree.from_n3tree(tree)      # copies the tensors to the host
        return oracle_mod.volume_render_backward(ot, rays.origins.cpu(), rays.dirs.cpu(), rays.viewdirs.cpu(), opt,
                                                 go.cpu())

    out = r(rays, fast=True)
    out.backward(go, retain_graph=True)
    err, ok = grad_close(tree.data.grad.cpu().numpy(), oracle_grad())
    assert ok, err
    tree.data.grad = None
    out.backward(go)                       # a second backward pass finds the notes used up and marches
    err, ok = grad_close(tree.data.grad.cpu().numpy(), oracle_grad())
    assert ok, err
    tree.data.grad = None
    out = r(rays, fast=True)
    with torch.no_grad():
        tree.data[..., -1] *= 0.5          # the densities change after the forward pass
    out.backward(go)
    err, ok = grad_close(tree.data.grad.cpu().numpy(), oracle_grad())
    assert ok, err


def test_no_notes_are_kept_where_no_gradient_is_recorded(gpu, monkeypatch):
    """Inside torch.no_grad(), or for a tree whose data does not require a gradient, the renderer
    calls the plain forward operators (which stop rays early); with a gradient on, the noted ones.
    The images are the same either way."""
    from svox_amd import renderer as rmod
    tree = on_gpu(synth.shell_tree(depth=5, n_spheres=4, data_format="SH4", seed=5, sigma_range=(20.0, 200.0)), gpu)
    rays = synth.sphere_rays(900, seed=2)
    rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.dirs.clone().to(gpu))
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0].to(gpu)
    calls = []
    for name in ("volume_render", "volume_render_noted", "volume_render_image", "volume_render_images",
                 "volume_render_images_noted"):
        def counted(*a, _f=getattr(rmod._C, name), _n=name, **kw):
            calls.append(_n)
            return _f(*a, **kw)
        monkeypatch.setattr(rmod._C, name, counted)
    assert tree.data.requires_grad
    with torch.no_grad():
        plain = r(rays, fast=True)
        plain_img = r.render_persp(c2w, width=96, height=64, fx=80.0, fast=True)
    assert calls == ["volume_render", "volume_render_image"], calls
    calls.clear()
    noted = r(rays, fast=True)
    noted_img = r.render_persp(c2w, width=96, height=64, fx=80.0, fast=True)
    assert calls == ["volume_render_noted", "volume_render_images_noted"], calls
    assert noted.grad_fn is not None and plain.grad_fn is None
    assert torch.equal(plain, noted) and torch.equal(plain_img, noted_img)
    calls.clear()
    tree.data.requires_grad_(False)
    r(rays, fast=True)
    assert calls == ["volume_render"], calls


def test_noted_entry_points_argument_handling(gpu, oracle_mod):
    """svox_volume_render_noted / _backward_noted through the C ABI: without a usable workspace they are
    the plain operators; a negative size and missing buffers are errors."""
    import ctypes
    from svox_amd.csrc import _abi
    tree = synth.shell_tree(depth=5, n_spheres=4, data_format="SH4", seed=2, sigma_range=(2.0, 20.0))
    rays = synth.sphere_rays(700, seed=1)
    opt = options(tree, step_size=1e-3, fast=True)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    go = torch.randn(700, 3, generator=torch.Generator().manual_seed(5))
    want = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    dev = on_gpu(tree, gpu)
    lib = _abi.load_library()
    spec = C._pack_tree(dev._spec())
    rs_obj = rays_spec(rays, gpu)
    rs = C._pack_rays(rs_obj, torch.float32)
    copt = opt._pack()
    go_d = go.to(gpu)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    enough = int(lib.svox_volume_render_backward_workspace_bytes(700, 30))
    buf = torch.zeros(enough + 64, dtype=torch.uint8, device=gpu)
    for ptr, nbytes in [(None, 0), (buf.data_ptr() + 4, enough), (buf.data_ptr(), 700 * 384), (buf.data_ptr(), enough)]:
        out = torch.full((700, 3), 7.0, device=gpu)
        rc = lib.svox_volume_render_noted(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), out.data_ptr(),
                                          ptr, nbytes, stream)
        assert rc == 0, lib.svox_last_error()
        assert np.array_equal(out.cpu().numpy(), ref)
        grad = torch.full_like(dev.data.data, 7.0)
        rc = lib.svox_volume_render_backward_noted(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt),
                                                   go_d.data_ptr(), grad.data_ptr(), 0, ptr, nbytes, stream)
        assert rc == 0, lib.svox_last_error()
        err, ok = grad_close(grad.cpu().numpy(), want)
        assert ok, (nbytes, err)
    out = torch.empty(700, 3, device=gpu)
    rc = lib.svox_volume_render_noted(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), out.data_ptr(),
                                      buf.data_ptr(), -1, stream)
    assert rc < 0 and b"workspace" in lib.svox_last_error()
    rc = lib.svox_volume_render_noted(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), None,
                                      buf.data_ptr(), enough, stream)
    assert rc < 0 and b"out" in lib.svox_last_error()
    rc = lib.svox_volume_render_backward_noted(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt),
                                               go_d.data_ptr(), None, 0, buf.data_ptr(), enough, stream)
    assert rc < 0 and b"grad_data_out" in lib.svox_last_error()


def test_training_step_in_a_hip_graph(gpu):
    """The entry points allocate nothing and clear with a kernel, so a caller may capture them: a noted
    forward + backward recorded once and replayed, with eager work in between, gives the eager result
    every time (the tree's data changes between the replays)."""
    tree = on_gpu(synth.shell_tree(depth=6, n_spheres=6, data_format="SH9", seed=37, sigma_range=(20.0, 200.0)), gpu)
    rays = synth.sphere_rays(5000, seed=4)
    rs = rays_spec(rays, gpu)
    opt = options(tree, step_size=1e-3, fast=True)
    go = (torch.randn(5000, 3, generator=torch.Generator().manual_seed(2)) * 1e-2).to(gpu)
    spec = tree._spec()

    def eager():
        out, notes = C.volume_render_noted(spec, rs, opt)
        return out, C.volume_render_backward_noted(spec, rs, opt, go, notes)

    eager()                                  # loads the library and its kernels outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_notes = C.volume_render_noted(spec, rs, opt)
        g_grad = C.volume_render_backward_noted(spec, rs, opt, go, g_notes)
    for step in range(3):
        with torch.no_grad():
            tree.data[..., -1] *= 0.9        # eager work between the replays: the densities change
        want_out, want_grad = eager()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, want_out), step
        err, ok = grad_close(g_grad.cpu().numpy(), want_grad.cpu().numpy())
        assert ok, (step, err)


def test_writes_past_the_version_counters_between_forward_and_backward(gpu, oracle_mod):
    """Writes torch's version counters do not see (svox's own idiom, docs/source/ex_opt_toy.py:26, and the
    views' `set`) between forward and backward: through a view or followed by tree.touch() the backward
    pass drops the forward pass's notes -- and marks of empty leaves kept on the tree -- and marches
    through the tree as it then is, which is what the reference's backward pass sees
    (svox/renderer.py:57-72 keeps nothing of the forward pass)."""
    tree = on_gpu(synth.shell_tree(depth=6, n_spheres=6, data_format="SH4", seed=31, sigma_range=(20.0, 200.0)), gpu)
    rays = synth.sphere_rays(3000, seed=3)
    rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.dirs.clone().to(gpu))
    c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0].to(gpu)
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    go = (torch.randn(3000, 3, generator=torch.Generator().manual_seed(1)) * 1e-2).to(gpu)
    gi = (torch.randn(48, 64, 3, generator=torch.Generator().manual_seed(2)) * 1e-2).to(gpu)
    opt = r._get_options(True)
    pts = torch.rand(4000, 3, generator=torch.Generator().manual_seed(1)).to(gpu)

    def oracle_grads():
        ot = oracle_mod.Tree.from_n3tree(tree)      # the tree as it is now
        a = oracle_mod.volume_render_backward(ot, rays.origins.cpu(), rays.dirs.cpu(), rays.viewdirs.cpu(), opt, go.cpu())
        b = oracle_mod.volume_render_image_backward(ot, c2w.cpu(), 50.0, 50.0, 64, 48, opt, gi.cpu())
        return a, b

    def check(write):
        tree.data.grad = None
        out = r(rays, fast=True)
        img = r.render_persp(c2w, width=64, height=48, fx=50.0, fast=True)
        versions = (tree.data._version, tree.child._version)
        write()
        assert (tree.data._version, tree.child._version) == versions    # torch has not seen the write
        want_batch, want_image = oracle_grads()
        out.backward(go)
        err, ok = grad_close(tree.data.grad.cpu().numpy(), want_batch)
        assert ok, err
        tree.data.grad = None
        img.backward(gi)
        err, ok = grad_close(tree.data.grad.cpu().numpy(), want_image)
        assert ok, err

    def view_write():
        tree[pts, -1:] = 150.0           # N3TreeView.set: empty leaves become dense

    def raw_write_then_touch():
        tree.data.data[..., -1] *= 0.25
        tree.touch()

    def kernel_write():
        tree.set(pts[:500], torch.full((500, tree.data_dim), 0.3, device=gpu))

    for marked in (False, True):
        for write in (view_write, raw_write_then_touch, kernel_write):
            if marked:
                tree.mark_empty_leaves()
                assert tree._spec().child_marks is not None
            check(write)
            assert tree._spec().child_marks is None      # every such write also drops kept marks

    # kept marks + a view write: the next picture is the one an unmarked tree gives
    tree.mark_empty_leaves()
    tree[pts[:100], -1:] = 0.0
    tree[pts[100:200], -1:] = 90.0
    with torch.no_grad():
        after = r.render_persp(c2w, width=64, height=48, fx=50.0, fast=True)
    ot = oracle_mod.Tree.from_n3tree(tree)
    assert np.array_equal(after.cpu().numpy(), oracle_mod.volume_render_image(ot, c2w.cpu(), 50.0, 50.0, 64, 48, opt))


def test_notes_are_not_replayed_for_other_directions_or_another_structure(gpu, oracle_mod):
    """The stamp of the notes in a workspace names the ray directions and the child table as well:
    svox_volume_render_backward_noted called with other directions (same origins), or with another
    child table (same data), marches instead of replaying notes that do not belong to the call."""
    tree = on_gpu(synth.shell_tree(depth=5, n_spheres=5, data_format="SH4", seed=8, sigma_range=(20.0, 200.0)), gpu)
    ot = oracle_mod.Tree.from_n3tree(tree)
    n = 2000
    rays = synth.sphere_rays(n, seed=6)
    other = synth.sphere_rays(n, seed=7)
    opt = options(tree, step_size=1e-3)
    go = (torch.randn(n, 3, generator=torch.Generator().manual_seed(3)) * 1e-2).to(gpu)
    spec = tree._spec()
    rs = rays_spec(rays, gpu)
    out, notes = C.volume_render_noted(spec, rs, opt)
    assert notes is not None
    # same origins tensor, other directions
    rs2 = C.RaysSpec()
    rs2.origins = rs.origins
    rs2.dirs = other.dirs.to(gpu)
    # (aim the new directions from the old origins at the cube again)
    tgt = torch.rand(n, 3, generator=torch.Generator().manual_seed(9)).to(gpu)
    d = tgt - rs.origins
    rs2.dirs = (d / d.norm(dim=1, keepdim=True)).contiguous()
    rs2.vdirs = rs2.dirs.clone()
    got = C.volume_render_backward_noted(spec, rs2, opt, go, notes)
    want = oracle_mod.volume_render_backward(ot, rs2.origins.cpu(), rs2.dirs.cpu(), rs2.vdirs.cpu(), opt, go.cpu())
    err, ok = grad_close(got.cpu().numpy(), want)
    assert ok, err
    # same data tensor, another child table (every leaf of the first node's children merged away is
    # not needed: a table of the same shape in which the root's cells are leaves is enough)
    out, notes = C.volume_render_noted(spec, rs, opt)
    flat = tree._spec()
    flat.child = torch.zeros_like(tree.child)
    got = C.volume_render_backward_noted(flat, rs, opt, go, notes)
    flat_tree = oracle_mod.Tree(tree.data.detach().cpu().numpy(), flat.child.cpu().numpy(), tree.parent_depth.cpu().numpy(),
                                tree.offset.cpu().numpy(), tree.invradius.cpu().numpy())
    want = oracle_mod.volume_render_backward(flat_tree, rays.origins, rays.dirs, rays.viewdirs, opt, go.cpu())
    err, ok = grad_close(got.cpu().numpy(), want)
    assert ok, err


def test_workspace_and_marking_thresholds_from_both_sides(gpu, monkeypatch):
    """The two size heuristics of the shim: the backward workspace (notes) shrinks to what the byte
    limit and the free device memory allow and is left out below 15 leaves per ray; a multi-pose call
    marks the empty leaves from AUTO_MARK_RAYS_PER_CELL rays per cell on.  Results do not depend on
    either."""
    tree = on_gpu(synth.shell_tree(depth=5, n_spheres=4, data_format="SH4", seed=5, sigma_range=(20.0, 200.0)), gpu)
    n = 4096
    size_of = C._abi.load_library().svox_volume_render_backward_workspace_bytes
    assert C._backward_workspace(tree, n)[1] == size_of(n, 120)        # (a small batch: four times the room)
    assert C._backward_workspace(tree, 1 << 19)[1] == size_of(1 << 19, 60)
    assert C._backward_workspace(tree, (1 << 19) + 1)[1] == size_of((1 << 19) + 1, 30)
    monkeypatch.setattr(C, "SMALL_BATCH_ROOM", 1)
    assert C._backward_workspace(tree, n)[1] == size_of(n, 30)
    monkeypatch.setattr(C, "BACKWARD_WORKSPACE_LIMIT", size_of(n, 30) - 1)
    assert C._backward_workspace(tree, n)[1] == size_of(n, 15)
    monkeypatch.setattr(C, "BACKWARD_WORKSPACE_LIMIT", size_of(n, 15))
    assert C._backward_workspace(tree, n)[1] == size_of(n, 15)
    monkeypatch.setattr(C, "BACKWARD_WORKSPACE_LIMIT", size_of(n, 15) - 1)
    assert C._backward_workspace(tree, n) == (None, 0)
    # no room: the differentiable forward pass runs without notes, the gradient is the same
    rays = synth.sphere_rays(n, seed=2)
    rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.dirs.clone().to(gpu))
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    go = torch.randn(n, 3, device=gpu)
    r(rays).backward(go)
    without_notes = tree.data.grad.clone()
    tree.data.grad = None
    monkeypatch.setattr(C, "BACKWARD_WORKSPACE_LIMIT", 4 << 30)
    r(rays).backward(go)
    err, ok = grad_close(tree.data.grad.cpu().numpy(), without_notes.cpu().numpy())
    assert ok, err
    # the share of the free memory: a large request is cut down to it
    monkeypatch.setattr(C, "_ASK_DEVICE_ABOVE", 0)
    monkeypatch.setattr(C, "BACKWARD_WORKSPACE_FREE_FRACTION", 1e-9)
    assert C._backward_workspace(tree, n) == (None, 0)
    monkeypatch.setattr(C, "BACKWARD_WORKSPACE_FREE_FRACTION", 0.25)
    assert C._backward_workspace(tree, n)[1] == size_of(n, 30)
    # marking: exactly at the threshold the call marks, one ray below it does not
    cells = tree.child.numel()
    opt = options(tree, step_size=1e-3, fast=True)
    monkeypatch.setattr(C, "AUTO_MARK_RAYS_PER_CELL", 1000 / cells)
    assert C._marks_for_this_call(tree._spec(), opt, 1000) is None        # (below the floor on the rays)
    monkeypatch.setattr(C, "AUTO_MARK_MIN_RAYS", 0)
    assert C._marks_for_this_call(tree._spec(), opt, 1000) is not None
    assert C._marks_for_this_call(tree._spec(), opt, 999) is None
    monkeypatch.setattr(C, "AUTO_MARK_MIN_RAYS", 2000)
    assert C._marks_for_this_call(tree._spec(), opt, 1999) is None
    assert C._marks_for_this_call(tree._spec(), opt, 2000) is not None


def test_render_of_a_saved_and_loaded_tree(gpu, oracle_mod, tmp_path):
    """save -> load -> render (svox/svox.py:835-865, 899-938): the file stores float16 records, so the
    picture of the loaded tree is, bit for bit, the picture of the original tree with its records
    rounded to float16 -- on the GPU and in the oracle.  (Interoperability with a file written by the
    reference itself cannot be pinned: the reference ships none.)"""
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format="SH9", seed=12, sigma_range=(20.0, 200.0))
    path = str(tmp_path / "scene.npz")
    tree.save(path)
    loaded = svox.N3Tree.load(path, device=gpu)
    assert loaded.data.is_cuda and loaded.child.is_cuda and repr(loaded.data_format) == "SH9"
    rounded = on_gpu(tree, gpu)
    with torch.no_grad():
        rounded.data.copy_(rounded.data.half().float())
    c2w = synth.orbit_poses(1, seed=2, radius=2.5)[0]
    kw = dict(width=120, height=90, fx=100.0, fast=True)
    with torch.no_grad():
        a = svox.VolumeRenderer(loaded, step_size=1e-3).render_persp(c2w.to(gpu), **kw)
        b = svox.VolumeRenderer(rounded, step_size=1e-3).render_persp(c2w.to(gpu), **kw)
        c = svox.VolumeRenderer(on_gpu(tree, gpu), step_size=1e-3).render_persp(c2w.to(gpu), **kw)
    assert torch.equal(a, b) and not torch.equal(a, c)
    ot = oracle_mod.Tree.from_n3tree(loaded)
    ref = oracle_mod.volume_render_image(ot, c2w, 100.0, 100.0, 120, 90, options(loaded, step_size=1e-3, fast=True))
    assert np.array_equal(a.cpu().numpy(), ref)
    pts = torch.rand(5000, 3, generator=torch.Generator().manual_seed(1)).to(gpu)
    va, ia = loaded(pts, want_node_ids=True)
    vb, ib = rounded(pts, want_node_ids=True)
    assert torch.equal(ia, ib) and torch.equal(va, vb)


@pytest.mark.parametrize("fmt", ["SH9", "RGBA"])
def test_density_softplus_on_the_octree_forward_kernel(gpu, oracle_mod, fmt):
    """density_softplus (rt_kernel.cu:276-277) in the specialised forward kernels: bit for bit what the
    generic kernel gives (one softplus routine on the device), 1e-5 from the oracle (another logf),
    for a ray batch handled both ways and for an image; marks made without the option play no part (the
    softplus of any stored density is > 0), marks made with it and the render's threshold decide the shading."""
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format=fmt, seed=17, sigma_range=(0.5, 30.0))
    with torch.no_grad():
        sigma = tree.data[..., -1]
        sigma -= 3.0                              # stored densities of both signs
        sigma[sigma == -3.0] = -8.0               # (the softplus of the empty leaves lies below the fast threshold)
    rays = synth.sphere_rays(3000, seed=4)
    opt = options(tree, step_size=1e-3, density_softplus=True, fast=True, rgb_padding=0.001)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    marked = dev._spec()
    marked.child_marks = C.mark_empty_leaves(dev._spec())
    decided = dev._spec()
    decided.child_marks = C.mark_empty_leaves(dev._spec(), opt.sigma_thresh, True)
    decided.child_marks_thresh, decided.child_marks_softplus = opt.sigma_thresh, True
    assert (decided.child_marks == -2).any()
    C.set_debug_flags(1)
    try:
        generic = C.volume_render(dev._spec(), rs, opt)
    finally:
        C.set_debug_flags(0)
    assert np.abs(generic.cpu().numpy() - ref).max() <= 1e-5
    assert C.octree_kernels_serve(dev._spec(), opt)
    for flags in (0, 2, 4, 8):
        C.set_debug_flags(flags)
        try:
            assert torch.equal(C.volume_render(dev._spec(), rs, opt), generic), flags
            assert torch.equal(C.volume_render(marked, rs, opt), generic), flags
            assert torch.equal(C.volume_render(decided, rs, opt), generic), flags
        finally:
            C.set_debug_flags(0)
    c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0]
    cam = cam_spec(c2w, 75, 53, 60.0, device=gpu)
    img = C.volume_render_image(dev._spec(), cam, opt)
    want = oracle_mod.volume_render_image(ot, c2w, 60.0, 60.0, 75, 53, opt)
    assert np.abs(img.cpu().numpy() - want).max() <= 1e-5
    assert torch.equal(C.volume_render_image(decided, cam, opt), img)
    C.set_debug_flags(1)
    try:
        assert torch.equal(C.volume_render_image(dev._spec(), cam, opt), img)
    finally:
        C.set_debug_flags(0)


# (logf of two libraries, the device's and the host's, meet in the softplus: measured 2e-5 to 5e-5)
SOFTPLUS_GATE = 1e-4


@pytest.mark.parametrize("fmt", ["SH9", "RGBA", "SH16"])
def test_density_softplus_gradients_on_the_octree_kernels(gpu, oracle_mod, fmt):
    """density_softplus in the backward pass and in se_grad (rt_kernel.cu:376, 440, 471-474, 518-710) on the octree
    kernels: marching backward with and without a workspace, notes taken by either forward kernel and replayed,
    autograd through the renderer, se_grad marching and from notes, ray batches handled as small and as large ones,
    and an image -- against the oracle, and against the one-ray-per-lane kernels that served this option before."""
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format=fmt, seed=17, sigma_range=(0.5, 30.0))
    with torch.no_grad():
        tree.data[..., -1] -= 3.0
    n = 3000
    rays = synth.sphere_rays(n, seed=4)
    opt = options(tree, step_size=1e-3, density_softplus=True, fast=True, rgb_padding=0.001)
    ot = oracle_mod.Tree.from_n3tree(tree)
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(2)) * 1e-2
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go, n_threads=8)
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(7))
    want_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=8)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    spec = dev._spec()
    assert C.octree_kernels_serve(spec, opt)
    plain_out = C.volume_render(spec, rs, opt)

    def close(got, want, what):
        err, ok = grad_close(got.cpu().numpy(), want, rel=SOFTPLUS_GATE, what=what)
        assert ok, (what, err)

    for flags in (0, 2, 4, 8):
        C.set_debug_flags(flags)
        try:
            if flags in (0, 2):
                for workspace in (True, False):
                    close(C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=workspace), want_g,
                          f"softplus backward flags {flags} workspace {workspace}")
                got = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=False)
                assert np.abs(got[0].cpu().numpy() - want_se[0]).max() <= 1e-5
                close(got[1], want_se[1], f"softplus se_grad gradient flags {flags}")
                close(got[2], want_se[2], f"softplus se_grad hessian flags {flags}")
            out, notes = C.volume_render_noted(spec, rs, opt)
            assert notes is not None and torch.equal(out, plain_out)
            close(C.volume_render_backward_noted(spec, rs, opt, go.to(gpu), notes), want_g, f"softplus notes flags {flags}")
            got = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=True)
            assert np.abs(got[0].cpu().numpy() - want_se[0]).max() <= 1e-5
            close(got[1], want_se[1], f"softplus se_grad from notes, gradient, flags {flags}")
            close(got[2], want_se[2], f"softplus se_grad from notes, hessian, flags {flags}")
        finally:
            C.set_debug_flags(0)
    # the one-ray-per-lane kernels on the same device: the same softplus routine, so only the order of the sums differs
    C.set_debug_flags(1)
    try:
        generic_g = C.volume_render_backward(spec, rs, opt, go.to(gpu))
        generic_se = C.se_grad(spec, rs, ref.to(gpu), opt)
    finally:
        C.set_debug_flags(0)
    err, ok = grad_close(C.volume_render_backward(spec, rs, opt, go.to(gpu)).cpu().numpy(), generic_g.cpu().numpy(),
                         what="softplus backward, octree against generic kernels")
    assert ok, err
    got = C.se_grad(spec, rs, ref.to(gpu), opt)
    assert torch.equal(got[0], generic_se[0])
    for a, b, what in zip(got[1:], generic_se[1:], ("gradient", "hessian")):
        err, ok = grad_close(a.cpu().numpy(), b.cpu().numpy(), what=f"softplus se_grad {what}, octree against generic kernels")
        assert ok, (what, err)
    # through the renderer (notes kept between the passes), rays and an image
    r = svox.VolumeRenderer(dev, step_size=1e-3, density_softplus=True, rgb_padding=0.001)
    dev.data.grad = None
    out = r(svox.Rays(rs.origins, rs.dirs, rs.vdirs), fast=True)
    assert torch.equal(out.detach(), plain_out)
    out.backward(go.to(gpu))
    close(dev.data.grad, want_g, "softplus autograd")
    c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0]
    igo = torch.randn(53, 75, 3, generator=torch.Generator().manual_seed(3)) * 1e-2
    want_ig = oracle_mod.volume_render_image_backward(ot, c2w, 60.0, 60.0, 75, 53, opt, igo)
    dev.data.grad = None
    r.render_persp(c2w.to(gpu), width=75, height=53, fx=60.0, fast=True).backward(igo.to(gpu))
    close(dev.data.grad, want_ig, "softplus autograd image")
    iref = torch.rand(53, 75, 3, generator=torch.Generator().manual_seed(9))
    want_ise = oracle_mod.se_grad_image(ot, c2w, 60.0, 60.0, 75, 53, iref, opt)
    got = r.se_grad_persp(c2w.to(gpu), iref.to(gpu), width=75, height=53, fx=60.0)
    assert np.abs(got[0].cpu().numpy() - want_ise[0]).max() <= 1e-5
    close(got[1], want_ise[1], "softplus se_grad_persp gradient")
    close(got[2], want_ise[2], "softplus se_grad_persp hessian")
    dev.data.grad = None


@pytest.mark.parametrize("fmt", ["RGBA", "SH4", "SH16", "SH25"])
def test_gradient_gate_without_order_slack(gpu, oracle_mod, fmt):
    """The plain gate -- 1e-4 relative to the oracle's exact sum, no allowance for the order of the additions -- on a
    scene where few rays meet in a leaf (a 128^3 shell tree, 3 000 rays): every family of kernels that forms
    gradients (marching backward, replay of notes taken by either forward kernel, se_grad marching and from notes,
    for ray batches handled as small and as large ones and for an image)."""
    tree = synth.shell_tree(depth=7, n_spheres=6, data_format=fmt, seed=23, sigma_range=(5.0, 120.0))
    n = 3000
    rays = synth.sphere_rays(n, seed=12)
    opt = options(tree, step_size=1e-3, fast=True, background_brightness=0.5)
    ot = oracle_mod.Tree.from_n3tree(tree)
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(2)) * 1e-2
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go, n_threads=8)
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(7))
    want_se = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=8)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    spec = dev._spec()

    def close(got, want, what):
        err, ok = grad_close(got.cpu().numpy(), want, what=what)
        assert ok, (what, err)

    for flags in (0, 2, 4, 8):
        C.set_debug_flags(flags)
        try:
            if flags in (0, 2):
                close(C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=False), want_g, f"marching, flags {flags}")
                got = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=False)
                close(got[1], want_se[1], f"se_grad marching, gradient, flags {flags}")
                close(got[2], want_se[2], f"se_grad marching, hessian, flags {flags}")
            close(C.volume_render_backward(spec, rs, opt, go.to(gpu), workspace=True), want_g, f"noting march + replay, flags {flags}")
            out, notes = C.volume_render_noted(spec, rs, opt)
            close(C.volume_render_backward_noted(spec, rs, opt, go.to(gpu), notes), want_g, f"replay, flags {flags}")
            got = C.se_grad(spec, rs, ref.to(gpu), opt, workspace=True)
            close(got[1], want_se[1], f"se_grad replay, gradient, flags {flags}")
            close(got[2], want_se[2], f"se_grad replay, hessian, flags {flags}")
        finally:
            C.set_debug_flags(0)
    c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0]
    W, H, fx = 96, 80, 90.0
    igo = torch.randn(H, W, 3, generator=torch.Generator().manual_seed(3)) * 1e-2
    want_ig = oracle_mod.volume_render_image_backward(ot, c2w, fx, fx, W, H, opt, igo, n_threads=8)
    cam = cam_spec(c2w, W, H, fx, device=gpu)
    for workspace in (True, False):
        close(C.volume_render_image_backward(spec, cam, opt, igo.to(gpu), workspace=workspace), want_ig,
              f"image, workspace {workspace}")
    out, notes = C.volume_render_images_noted(spec, cam, opt)
    close(C.volume_render_images_backward_noted(spec, cam, opt, igo.to(gpu), notes), want_ig, "image replay")


def test_notes_are_kept_only_where_they_are_taken(gpu):
    """A renderer whose tree or options the noting kernels do not serve (fp64 records, a negative sigma_thresh) runs
    the plain forward pass: no workspace is allocated, the autograd context keeps nothing, and
    the notes budget never looks at a counter nobody wrote."""
    from svox_amd import renderer as R
    rays = synth.sphere_rays(500, seed=1)
    kept = []
    orig = R._C.volume_render_noted

    def spy(*a, **k):
        out, notes = orig(*a, **k)
        kept.append(notes)
        return out, notes

    R._C.volume_render_noted = spy
    try:
        cases = []
        t3 = svox.N3Tree(N=3, data_format="SH4", init_refine=1, device=gpu)
        t3.data.data.normal_()
        t3.data.data[..., -1].abs_()
        cases.append((svox.VolumeRenderer(t3, step_size=1e-2), True))         # (N = 3 runs on the same kernels)
        cases.append((svox.VolumeRenderer(t3, step_size=1e-2, max_comp=2), True))     # (and so does a range of components)
        t64 = on_gpu(synth.dense_tree(2, "SH4", seed=1, sigma="lognormal", dtype=torch.float64), gpu)
        cases.append((svox.VolumeRenderer(t64, step_size=1e-2), False))
        t2 = on_gpu(synth.dense_tree(3, "SH4", seed=0, sigma="lognormal"), gpu)
        neg = svox.VolumeRenderer(t2, step_size=1e-2)
        neg.sigma_thresh = -1.0
        cases.append((neg, False))
        cases.append((svox.VolumeRenderer(t2, step_size=1e-2, density_softplus=True), True))
        cases.append((svox.VolumeRenderer(t2, step_size=1e-2), True))
        for r, takes in cases:
            kept.clear()
            dt = r.tree.data.dtype
            grays = svox.Rays(rays.origins.to(gpu, dt), rays.dirs.to(gpu, dt), rays.viewdirs.to(gpu, dt))
            for _ in range(3):
                r.tree.data.grad = None
                r(grays).sum().backward()
                torch.cuda.synchronize()
            assert len(kept) == 3 and all((k is not None) == takes for k in kept), (takes, kept)
            assert r.notes_budget.factor == 1
            if not takes:
                assert r.notes_budget._pending is None
    finally:
        R._C.volume_render_noted = orig


def test_what_a_give_up_of_the_two_wavefront_kernel_leaves_behind(gpu, oracle_mod):
    """The waits between the walking and the shading wavefront are bounded.  With the bound at one look (debug flag
    16: the shading gives up as soon as it finds nothing new, the walk once its ring is full) every kernel still ends;
    the pixels of the rays given up on are NaN, never a plausible colour; their notes say "march me", so the gradient
    that follows is the right one; and the library's counter tells the host."""
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format="SH9", seed=3)
    rays = synth.sphere_rays(4000, seed=6)
    opt = options(tree, step_size=1e-3, fast=True)
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    go = torch.randn(4000, 3, generator=torch.Generator().manual_seed(2)) * 1e-2
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    before = C.give_up_count()
    C.set_debug_flags(8 | 16)
    try:
        out = C.volume_render(dev._spec(), rs, opt).cpu().numpy()
        noted, notes = C.volume_render_noted(dev._spec(), rs, opt)
    finally:
        C.set_debug_flags(0)
    gave_up = np.isnan(out).any(axis=1)
    assert gave_up.any() and C.give_up_count() > before
    assert np.array_equal(out[~gave_up], want[~gave_up])           # the others are untouched
    noted = noted.cpu().numpy()
    bad = np.isnan(noted).any(axis=1)
    assert np.array_equal(noted[~bad], want[~bad])
    g = C.volume_render_backward_noted(dev._spec(), rs, opt, go.to(gpu), notes)
    err, ok = grad_close(g.cpu().numpy(), want_g, what="gradient after a give-up")
    assert ok, err
    # the stateless backward operator takes its notes with grad_out at hand (the sum of the first march rides along)
    C.set_debug_flags(8 | 16)
    try:
        g = C.volume_render_backward(dev._spec(), rs, opt, go.to(gpu))
    finally:
        C.set_debug_flags(0)
    err, ok = grad_close(g.cpu().numpy(), want_g, what="stateless gradient after a give-up")
    assert ok, err
    # and a healthy run gives up nowhere
    now = C.give_up_count()
    C.set_debug_flags(8)
    try:
        assert np.array_equal(C.volume_render(dev._spec(), rs, opt).cpu().numpy(), want)
    finally:
        C.set_debug_flags(0)
    assert C.give_up_count() == now


def test_a_training_step_replays_from_a_hip_graph(gpu):
    """forward + backward + SGD update captured with torch.cuda.graph: every launch of the library goes
    to torch's current stream, its zero-fills are kernels and all its buffers come from torch's allocator,
    so the step can be captured.  Every replay -- with unrelated eager work and a synchronisation between
    them -- must give what the eager step gives (up to the order of the atomic additions)."""
    tree = on_gpu(synth.dense_tree(3, "SH4", seed=0, sigma="lognormal", coeff_std=0.5), gpu)
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    n = 4096
    rays = synth.sphere_rays(n, seed=1)
    rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.dirs.clone().to(gpu))
    target = torch.rand(n, 3, device=gpu, generator=torch.Generator(device=gpu).manual_seed(3))
    start = tree.data.detach().clone()

    def step():
        out = r(rays)
        loss = ((out - target) ** 2).sum()
        loss.backward()
        with torch.no_grad():
            tree.data.data -= 0.1 * tree.data.grad
        tree.data.grad = None
        return loss.detach()

    eager_losses, eager_data = [], []
    for _ in range(4):
        eager_losses.append(float(step()))
        eager_data.append(tree.data.detach().clone())
    assert eager_losses[3] < eager_losses[0]

    tree.data.data.copy_(start)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # (torch asks for a warm-up on a side stream)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured_loss = step()
    tree.data.data.copy_(start)
    for i in range(4):
        graph.replay()
        torch.cuda.synchronize()
        assert abs(float(captured_loss) - eager_losses[i]) <= 1e-5 * abs(eager_losses[i]), (i, float(captured_loss))
        err, ok = grad_close(tree.data.detach().cpu().numpy(), eager_data[i].cpu().numpy(), rel=1e-5)
        assert ok, (i, err)
        assert float((torch.rand(1000, device=gpu) * 2).sum()) > 0          # eager work between the replays
