"""Trees deeper than the walk's shortcuts reach: more levels than the per-lane path memory holds
(11) and more than the integer cell coordinates resolve (24, where the kernels switch to the
reference's floating-point walk).  GPU against the oracle."""
import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu


def rays_through(point, n, seed):
    """Rays from a sphere around the cube towards targets that close in on `point` at every scale."""
    g = torch.Generator().manual_seed(seed)
    origins = point[None] + 2.0 * synth.unit_vectors(n, g)
    scale = 2.0 ** -torch.randint(1, 30, (n, 1), generator=g).float()
    targets = point[None] + (torch.rand(n, 3, generator=g) * 2 - 1) * scale
    dirs = targets - origins
    dirs = dirs / dirs.norm(dim=1, keepdim=True)
    return svox.Rays(origins.contiguous(), dirs.contiguous(), dirs.clone())


@pytest.mark.parametrize("levels", [12, 14, 27])
@pytest.mark.parametrize("fmt", ["SH4", "RGBA"])
def test_deep_tree_render(gpu, oracle_mod, levels, fmt):
    tree, point = synth.deep_tree(levels, data_format=fmt, seed=levels)
    rays = rays_through(point, 4000, seed=levels)
    opt = options(tree, step_size=1e-4)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref, ref_stats = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt, want_stats=True)
    # the rays do reach the deep end of the chain
    assert ref_stats["levels"] / ref_stats["samples"] > 3.0
    dev = on_gpu(tree, gpu)
    rs = rays_spec(rays, gpu)
    for generic in (0, 1):
        C.set_debug_flags(generic)
        try:
            out = C.volume_render(dev._spec(), rs, opt).cpu().numpy()
            stats = C.volume_render_stats(dev._spec(), rs, opt)
        finally:
            C.set_debug_flags(0)
        assert np.array_equal(out, ref), generic
        assert stats["samples"] == ref_stats["samples"] and stats["levels"] == ref_stats["levels"]
    # Gradients of all 4000 rays.  Thousands of rays add into under a hundred leaves here, so the
    # reference value is the oracle's exact sum (fp32 terms added in float64), and the bar is 1e-4
    # relative beyond the order slack of fp32 additions (util.grad_close: sequential fp32 sums of
    # these very terms in shuffled orders differ from the exact sum by up to 1.6e-4).
    go = torch.randn(len(rays.origins), 3, generator=torch.Generator().manual_seed(1))
    want, slack = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go, n_threads=4,
                                                    want_slack=True)
    for workspace in (True, False):
        got = C.volume_render_backward(dev._spec(), rs, opt, go.to(gpu), workspace=workspace).cpu().numpy()
        err, ok = grad_close(got, want, slack=slack)
        assert ok, (workspace, err)
    out, notes = C.volume_render_noted(dev._spec(), rs, opt)
    assert np.array_equal(out.cpu().numpy(), ref)
    got = C.volume_render_backward_noted(dev._spec(), rs, opt, go.to(gpu), notes).cpu().numpy()
    err, ok = grad_close(got, want, slack=slack)
    assert ok, ("noted", err)
    colour = torch.rand(len(rays.origins), 3, generator=torch.Generator().manual_seed(2))
    want = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, colour, opt, n_threads=4, want_slack=True)
    for workspace in (True, False):
        got = C.se_grad(dev._spec(), rs, colour.to(gpu), opt, workspace=workspace)
        assert np.array_equal(got[0].cpu().numpy(), want[0])
        for g, w, sl in zip(got[1:], want[1:3], want[3:]):
            err, ok = grad_close(g.cpu().numpy(), w, slack=sl)
            assert ok, (workspace, err)


@pytest.mark.parametrize("levels", [14, 27])
def test_deep_tree_queries(gpu, oracle_mod, levels):
    tree, point = synth.deep_tree(levels, data_format="SH4", seed=levels)
    g = torch.Generator().manual_seed(5)
    n = 20000
    scale = 2.0 ** -torch.randint(1, 30, (n, 1), generator=g).float()
    pts = (point[None] + (torch.rand(n, 3, generator=g) * 2 - 1) * scale).clamp(0, 1).contiguous()
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref_vals, ref_ids, ref_levels = oracle_mod.query_vertical(ot, pts, want_levels=True)
    # (fp32 points cannot single out the very last cells of a 27-level chain)
    assert ref_levels.max() == levels if levels <= 24 else ref_levels.max() > 24
    dev = on_gpu(tree, gpu)
    vals, ids = dev(pts.to(gpu), want_node_ids=True)
    assert np.array_equal(ids.cpu().numpy(), ref_ids)
    assert np.array_equal(vals.detach().cpu().numpy(), ref_vals)
    # small integers: thousands of them add up exactly in fp32, whatever the order of the atomics
    go = torch.randint(-8, 9, (n, tree.data_dim), generator=g).float()
    want = oracle_mod.query_vertical_backward(ot, pts, go)
    got = C.query_vertical_backward(dev._spec(), pts.to(gpu), go.to(gpu)).cpu().numpy()
    assert np.array_equal(got, want)
