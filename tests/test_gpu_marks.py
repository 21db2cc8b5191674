"""Marks of the empty leaves (svox_mark_empty_leaves, SvoxTreeSpec.child_marks; no reference counterpart):
with the marks the render operators give the same results as without, to the last bit where the plain
results are bit-exact, and the marks never outlive a change of the tree that the package can see."""
import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import cam_spec, grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu


def sparse_tree(fmt, gpu, seed=21, depth=6):
    """shell tree whose empty leaves hold 0, a few of them negative densities and a few NaN"""
    tree = synth.shell_tree(depth=depth, n_spheres=6, data_format=fmt, seed=seed, sigma_range=(20.0, 200.0))
    g = torch.Generator().manual_seed(seed)
    sigma = tree.data.data[..., -1]
    empty = (sigma == 0) & (tree.child == 0)
    pick = empty & (torch.rand(sigma.shape, generator=g) < 0.05)
    sigma[pick] = -3.0
    pick = empty & (torch.rand(sigma.shape, generator=g) < 0.01)
    sigma[pick] = float("nan")
    return on_gpu(tree, gpu)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_marks_are_the_child_table_with_the_empty_leaves_marked(gpu, dtype):
    tree = synth.dense_tree(3, "SH4", seed=2, zero_fraction=0.4, dtype=dtype)
    tree.data.data[0, 0, 0, 1, -1] = float("nan")
    tree.data.data[1, 1, 0, 1, -1] = -1.0
    tree = tree.to(gpu)
    marks = C.mark_empty_leaves(tree._spec())
    sigma = tree.data.data[..., -1]
    want = torch.where(tree.child != 0, tree.child,
                       torch.where(sigma > 0, torch.zeros_like(tree.child), torch.full_like(tree.child, -2)))
    assert marks.dtype == torch.int32 and torch.equal(marks, want)
    assert (marks == -2).any() and (marks == 0).any() and (marks > 0).any()


@pytest.mark.parametrize("flags", [0, 2])
@pytest.mark.parametrize("fmt", ["RGBA", "SH4", "SH16", "SH25"])
def test_renders_with_marks_equal_renders_without(gpu, oracle_mod, fmt, flags):
    tree = sparse_tree(fmt, gpu)
    rays = synth.sphere_rays(3000, seed=5)
    rs = rays_spec(rays, gpu)
    go = (torch.randn(3000, 3, generator=torch.Generator().manual_seed(1)) * 1e-2).to(gpu)
    ref = torch.rand(3000, 3, generator=torch.Generator().manual_seed(7)).to(gpu)
    c2w = synth.orbit_poses(2, seed=4, radius=2.5)
    cam = cam_spec(torch.stack(c2w).to(gpu), 75, 53, 60.0)
    plain = tree._spec()
    marked = tree._spec()
    marked.child_marks = C.mark_empty_leaves(plain)
    C.set_debug_flags(flags)
    try:
        for opt in (options(tree, step_size=1e-3), options(tree, step_size=1e-3, fast=True)):
            a, b = C.volume_render(plain, rs, opt), C.volume_render(marked, rs, opt)
            assert torch.equal(a, b)
            assert torch.equal(C.volume_render_images(plain, cam, opt), C.volume_render_images(marked, cam, opt))
            ga = C.volume_render_backward(plain, rs, opt, go)
            gb = C.volume_render_backward(marked, rs, opt, go)
            err, ok = grad_close(gb.cpu().numpy(), ga.cpu().numpy())
            assert ok, err
            out, notes = C.volume_render_noted(marked, rs, opt)
            assert torch.equal(out, a)
            gn = C.volume_render_backward_noted(marked, rs, opt, go, notes)
            err, ok = grad_close(gn.cpu().numpy(), ga.cpu().numpy())
            assert ok, err
        opt = options(tree, step_size=1e-3)
        sa, sb = C.se_grad(plain, rs, ref, opt), C.se_grad(marked, rs, ref, opt)
        assert torch.equal(sa[0], sb[0])
        for x, y in zip(sa[1:], sb[1:]):
            err, ok = grad_close(y.cpu().numpy(), x.cpu().numpy())
            assert ok, err
    finally:
        C.set_debug_flags(0)
    # and the oracle, which knows nothing of marks, agrees with the marked render
    opt = options(tree, step_size=1e-3, fast=True)
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    assert np.array_equal(C.volume_render(marked, rs, opt).cpu().numpy(), want)


def test_marks_are_ignored_where_an_empty_leaf_could_contribute(gpu, oracle_mod):
    """A negative sigma_thresh lets leaves with sigma in (thresh, 0] take part (rt_kernel.cu:278): the
    marks are then left aside.  Weight accumulation, fp64 and softplus renders are unaffected as well."""
    tree = sparse_tree("SH4", gpu, seed=5)
    rays = synth.sphere_rays(2000, seed=3)
    rs = rays_spec(rays, gpu)
    plain, marked = tree._spec(), tree._spec()
    marked.child_marks = C.mark_empty_leaves(plain)
    opt = options(tree, step_size=1e-3, sigma_thresh=-5.0)
    a, b = C.volume_render(plain, rs, opt), C.volume_render(marked, rs, opt)
    both_nan = torch.isnan(a) & torch.isnan(b)
    assert torch.equal(torch.where(both_nan, torch.zeros_like(a), a), torch.where(both_nan, torch.zeros_like(b), b))
    want = oracle_mod.volume_render(oracle_mod.Tree.from_n3tree(tree), rays.origins, rays.dirs, rays.viewdirs, opt)
    assert np.array_equal(b.cpu().numpy(), want, equal_nan=True)
    # (the render above differs from the one with threshold 0: the negative densities take part)
    c = C.volume_render(plain, rs, options(tree, step_size=1e-3))
    assert not torch.equal(torch.nan_to_num(a), torch.nan_to_num(c))
    opt = options(tree, step_size=1e-3, density_softplus=True)
    assert torch.equal(C.volume_render(plain, rs, opt), C.volume_render(marked, rs, opt))
    for acc_op in ("sum", "max"):
        with tree.accumulate_weights(op=acc_op) as acc_plain:
            C.volume_render(tree._spec(), rs, options(tree, step_size=1e-3))
        tree.mark_empty_leaves()
        with tree.accumulate_weights(op=acc_op) as acc_marked:
            assert tree._spec().child_marks is not None
            C.volume_render(tree._spec(), rs, options(tree, step_size=1e-3))
        tree.clear_leaf_marks()
        wa, wb = acc_plain.value, acc_marked.value
        assert torch.allclose(wa, wb, rtol=1e-5, atol=1e-7) if acc_op == "sum" else torch.equal(wa, wb)


def test_marks_on_a_tree_deeper_than_the_integer_walk(gpu, oracle_mod):
    from test_gpu_deep import rays_through
    tree, point = synth.deep_tree(27, "SH4", seed=27)
    g = torch.Generator().manual_seed(4)
    sigma = tree.data.data[..., -1]
    sigma[torch.rand(sigma.shape, generator=g) < 0.5] = 0.0          # half of the cells lose their density
    rays = rays_through(point, 3000, seed=27)
    opt = options(tree, step_size=1e-4)
    want = oracle_mod.volume_render(oracle_mod.Tree.from_n3tree(tree), rays.origins, rays.dirs, rays.viewdirs, opt)
    tree = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    plain, marked = tree._spec(), tree._spec()
    marked.child_marks = C.mark_empty_leaves(plain)
    assert (marked.child_marks == -2).any()
    out = C.volume_render(marked, rs, opt)
    assert torch.equal(C.volume_render(plain, rs, opt), out)
    assert np.array_equal(out.cpu().numpy(), want)


def test_tree_drops_its_marks_when_it_changes(gpu):
    tree = sparse_tree("SH4", gpu, seed=9, depth=5)
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0].to(gpu)
    with torch.no_grad():
        before = r.render_persp(c2w, width=64, height=48, fx=50.0, fast=True)
        assert tree.mark_empty_leaves() is tree
        assert tree._spec().child_marks is not None
        assert torch.equal(r.render_persp(c2w, width=64, height=48, fx=50.0, fast=True), before)

    def marked_again():
        tree.mark_empty_leaves()
        assert tree._spec().child_marks is not None

    # a write through the view: an empty leaf becomes dense, and the next render shows it
    pts = torch.rand(4000, 3, generator=torch.Generator().manual_seed(1)).to(gpu)
    tree[pts, -1:] = 150.0
    assert tree._spec().child_marks is None
    with torch.no_grad():
        after = r.render_persp(c2w, width=64, height=48, fx=50.0, fast=True)
    assert not torch.equal(after, before)
    marked_again()
    with torch.no_grad():
        assert torch.equal(r.render_persp(c2w, width=64, height=48, fx=50.0, fast=True), after)
    # an in-place torch operation on the parameter
    with torch.no_grad():
        tree.data.mul_(0.5)
    assert tree._spec().child_marks is None
    marked_again()
    # an optimizer step
    opt = torch.optim.SGD([tree.data], lr=1e-3)
    rays = synth.sphere_rays(500, seed=3)
    out = r(svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.viewdirs.to(gpu)))
    out.sum().backward()
    opt.step()
    assert tree._spec().child_marks is None
    marked_again()
    # structure
    tree.refine()
    assert tree._spec().child_marks is None
    marked_again()
    tree.clear_leaf_marks()
    assert tree._spec().child_marks is None
    # moving the tree
    marked_again()
    moved = tree.to("cpu").to(gpu)
    assert moved._spec().child_marks is None


def test_mark_empty_leaves_argument_checks(gpu):
    tree = synth.dense_tree(2, "SH4", seed=1).to(gpu)
    spec = tree._spec()
    spec.child_marks = torch.zeros(3, dtype=torch.int32, device=gpu)
    rays = synth.sphere_rays(8, seed=0)
    with pytest.raises(RuntimeError, match="child_marks"):
        C.volume_render(spec, rays_spec(rays, gpu), options(tree))
    spec.child_marks = tree.child.clone().long()
    with pytest.raises(RuntimeError, match="child_marks"):
        C.volume_render(spec, rays_spec(rays, gpu), options(tree))
    spec.child_marks = tree.child.cpu()
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        C.volume_render(spec, rays_spec(rays, gpu), options(tree))


def test_large_multi_pose_launch_marks_the_leaves_for_itself(gpu, monkeypatch):
    """volume_render_images with many rays per cell of the tree makes the marks for that call; the
    pictures are the ones rendered without."""
    tree = sparse_tree("SH9", gpu, seed=3, depth=5)
    cam = cam_spec(torch.stack(synth.orbit_poses(3, seed=4, radius=2.5)).to(gpu), 160, 120, 130.0)
    opt = options(tree, step_size=1e-3, fast=True)
    assert 3 * 160 * 120 > C.AUTO_MARK_RAYS_PER_CELL * tree.child.numel()
    monkeypatch.setattr(C, "AUTO_MARK_MIN_RAYS", 3 * 160 * 120)   # (the floor on the number of rays: just met)
    made = []
    real = C.mark_empty_leaves
    monkeypatch.setattr(C, "mark_empty_leaves", lambda t, *how: made.append(how) or real(t, *how))
    with_marks = C.volume_render_images(tree._spec(), cam, opt)
    assert made == [(opt.sigma_thresh, False)]          # made with the call's own threshold: they decide the shading
    monkeypatch.setattr(C, "AUTO_MARK_RAYS_PER_CELL", None)
    without = C.volume_render_images(tree._spec(), cam, opt)
    assert len(made) == 1 and torch.equal(with_marks, without)
    monkeypatch.setattr(C, "AUTO_MARK_RAYS_PER_CELL", 0.7)
    small = cam_spec(torch.stack(synth.orbit_poses(2, seed=4, radius=2.5)).to(gpu), 16, 12, 13.0)
    C.volume_render_images(tree._spec(), small, opt)                          # too few rays to pay
    C.volume_render_images(tree._spec(), cam, options(tree, step_size=1e-3, sigma_thresh=-1.0))
    C.volume_render_images(tree._spec(), cam, options(tree, step_size=1e-3, density_softplus=True))
    assert len(made) == 1
    # a call that takes notes works on every leaf with density: its marks are made with threshold 0
    out, notes = C.volume_render_images_noted(tree._spec(), cam, opt)
    assert notes is not None and made[1:] == [(0.0, False)] and torch.equal(out, with_marks)
    # with the softplus, a threshold above 0 marks leaves too
    soft = options(tree, step_size=1e-3, density_softplus=True, fast=True)
    a = C.volume_render_images(tree._spec(), cam, soft)
    assert made[2:] == [(soft.sigma_thresh, True)]
    monkeypatch.setattr(C, "AUTO_MARK_RAYS_PER_CELL", None)
    assert torch.equal(C.volume_render_images(tree._spec(), cam, soft), a)


@pytest.mark.parametrize("softplus", [False, True])
def test_marks_made_with_a_threshold(gpu, softplus):
    """svox_mark_leaves_below: a leaf is marked exactly when trace_ray would skip it (rt_kernel.cu:276-278)."""
    tree = synth.dense_tree(3, "SH4", seed=2, zero_fraction=0.3, sigma="lognormal")
    tree.data.data[0, 0, 0, 1, -1] = float("nan")
    tree.data.data[1, 1, 0, 1, -1] = -1.0
    tree = tree.to(gpu)
    thresh = 0.75
    marks = C.mark_empty_leaves(tree._spec(), thresh, softplus)
    raw = tree.data.data[..., -1]
    sigma = torch.log(1 + torch.exp(raw - 1)) if softplus else raw
    keep = sigma > thresh
    near = (sigma - thresh).abs() < 1e-5          # (the device's logf may round another way right at the threshold)
    want = torch.where(tree.child != 0, tree.child, torch.where(keep, torch.zeros_like(tree.child), torch.full_like(tree.child, -2)))
    agree = (marks == want) | (near & (tree.child == 0))
    assert bool(agree.all()) and (marks == -2).any() and (marks == 0).any()
    spec = tree._spec()
    with pytest.raises(RuntimeError, match="sigma_thresh"):
        C.mark_empty_leaves(spec, -1.0)


@pytest.mark.parametrize("flags", [0, 2, 4, 8])
@pytest.mark.parametrize("fmt", ["RGBA", "SH9", "SH16"])
def test_marks_that_decide_the_shading(gpu, oracle_mod, fmt, flags):
    """Marks made with the render's own sigma_thresh: the forward kernels shade every leaf the marks let through
    without a look at its density first.  Pictures equal the oracle's bit for bit on every forward kernel; calls that
    need the leaves such marks hide (a smaller threshold, the backward pass, notes, se_grad) leave them aside."""
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format=fmt, seed=31, sigma_range=(0.002, 60.0))
    rays = synth.sphere_rays(3000, seed=9)
    opt = options(tree, step_size=1e-3, sigma_thresh=0.5, stop_thresh=1e-2, rgb_padding=0.001)
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    c2w = synth.orbit_poses(2, seed=4, radius=2.5)
    want_img = np.stack([oracle_mod.volume_render_image(ot, p, 60.0, 60.0, 75, 53, opt) for p in c2w])
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    cam = cam_spec(torch.stack(c2w).to(gpu), 75, 53, 60.0)
    decided = dev._spec()
    decided.child_marks = C.mark_empty_leaves(dev._spec(), opt.sigma_thresh)
    decided.child_marks_thresh = opt.sigma_thresh
    sigma = dev.data.data[..., -1]
    between = ((sigma > 0) & (sigma <= 0.5) & (dev.child == 0)).sum().item()
    assert between > 100 and (decided.child_marks == -2).sum().item() > between     # leaves only these marks hide
    go = (torch.randn(3000, 3, generator=torch.Generator().manual_seed(1)) * 1e-2).to(gpu)
    C.set_debug_flags(flags)
    try:
        assert np.array_equal(C.volume_render(decided, rs, opt).cpu().numpy(), want)
        assert np.array_equal(C.volume_render_images(decided, cam, opt).cpu().numpy(), want_img)
        # a smaller threshold needs leaves the marks hide: the marks are left aside
        low = options(tree, step_size=1e-3, sigma_thresh=0.1, stop_thresh=1e-2, rgb_padding=0.001)
        want_low = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, low)
        assert np.array_equal(C.volume_render(decided, rs, low).cpu().numpy(), want_low)
        assert not np.array_equal(want_low, want)
        # a larger threshold may use them as plain marks
        high = options(tree, step_size=1e-3, sigma_thresh=2.0, stop_thresh=1e-2, rgb_padding=0.001)
        want_high = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, high)
        assert np.array_equal(C.volume_render(decided, rs, high).cpu().numpy(), want_high)
        if flags in (0, 2):
            want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go.cpu())
            for workspace in (True, False):
                g = C.volume_render_backward(decided, rs, opt, go, workspace=workspace)
                err, ok = grad_close(g.cpu().numpy(), want_g, what=f"marks with a threshold, workspace {workspace}")
                assert ok, err
            out, notes = C.volume_render_noted(decided, rs, opt)
            assert np.array_equal(out.cpu().numpy(), want)
            g = C.volume_render_backward_noted(decided, rs, opt, go, notes)
            err, ok = grad_close(g.cpu().numpy(), want_g, what="marks with a threshold, notes")
            assert ok, err
    finally:
        C.set_debug_flags(0)


def test_the_tree_keeps_marks_made_with_a_threshold(gpu, oracle_mod):
    tree = synth.shell_tree(depth=5, n_spheres=5, data_format="SH4", seed=3, sigma_range=(0.002, 60.0))
    rays = synth.sphere_rays(2000, seed=2)
    ot = oracle_mod.Tree.from_n3tree(tree)
    dev = on_gpu(tree, gpu)
    r = svox.VolumeRenderer(dev, step_size=1e-3)
    r.sigma_thresh = 0.5
    opt = r._get_options(True)
    dev.mark_empty_leaves(sigma_thresh=0.5)
    spec = dev._spec()
    assert spec.child_marks is not None and spec.child_marks_thresh == 0.5 and not spec.child_marks_softplus
    grays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.viewdirs.to(gpu))
    with torch.no_grad():
        out = r(grays, fast=True)
    assert np.array_equal(out.cpu().numpy(), oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt))
    # a training step on the same tree: notes and backward pass see every leaf with density
    go = torch.randn(2000, 3, generator=torch.Generator().manual_seed(5)) * 1e-2
    r(grays, fast=True).backward(go.to(gpu))
    want_g = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go)
    err, ok = grad_close(dev.data.grad.cpu().numpy(), want_g)
    assert ok, err
