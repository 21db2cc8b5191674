"""GPU parity of the point-query operators against the CPU oracle (bit-exact bar for ids, values,
corners; 1e-4 relative for the atomically summed query gradient)."""
import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import on_gpu

pytestmark = pytest.mark.gpu


def edge_points(dtype=torch.float32):
    hi = np.frombuffer(np.uint32(0x3F7FFFEF).tobytes(), dtype=np.float32)[0]
    vals = [0.0, -0.0, -1.0, 1.0, 2.0, 0.5, 0.25, 0.75, hi, np.nextafter(np.float32(1), np.float32(0)),
            1.0 - 2.0 ** -24, 0.125, 1e-30, np.nan, np.inf, -np.inf, 0.49999997, 0.50000006]
    g = np.array(np.meshgrid(vals, vals[:6], vals[:4], indexing="ij")).reshape(3, -1).T
    return torch.tensor(g, dtype=dtype)


def trees():
    yield "dense16_rgba", synth.dense_tree(3, "RGBA", seed=0)
    yield "dense8_sh9", synth.dense_tree(2, "SH9", seed=1, sigma="lognormal", coeff_std=0.5, zero_fraction=0.5)
    yield "shell7_sh4", synth.shell_tree(depth=7, n_spheres=6, data_format="SH4", seed=2)
    t = svox.N3Tree(N=3, data_dim=5, init_refine=2)
    t.data.data.normal_(generator=torch.Generator().manual_seed(3))
    yield "n3_dense", t
    t = synth.dense_tree(1, "SH16", seed=4)
    t.invradius.data[:] = torch.tensor([0.4, 0.5, 0.8])
    t.offset.data[:] = torch.tensor([0.1, 0.2, -0.05])
    yield "scaled_sh16", t


@pytest.mark.parametrize("name,tree", list(trees()), ids=lambda x: x if isinstance(x, str) else "")
@pytest.mark.parametrize("generic", [0, 1])
def test_query_vertical_matches_oracle(gpu, oracle_mod, name, tree, generic):
    g = torch.Generator().manual_seed(11)
    pts = torch.cat([torch.rand(20000, 3, generator=g) * 1.2 - 0.1, edge_points()]).contiguous()
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref_vals, ref_ids = oracle_mod.query_vertical(ot, pts)
    dev_tree = on_gpu(tree, gpu)
    C.set_debug_flags(generic)
    try:
        vals, ids = dev_tree(pts.to(gpu), want_node_ids=True)
    finally:
        C.set_debug_flags(0)
    assert ids.dtype == torch.int64 and vals.shape == (pts.shape[0], tree.data_dim)
    assert np.array_equal(ids.cpu().numpy(), ref_ids)
    assert np.array_equal(vals.detach().cpu().numpy(), ref_vals)


def test_query_local_coordinates_and_empty(gpu, oracle_mod):
    tree = synth.dense_tree(2, "RGBA", seed=5)
    tree.invradius.data[:] = 0.25
    pts = torch.rand(1000, 3, generator=torch.Generator().manual_seed(1))
    ot = oracle_mod.Tree.from_n3tree(tree, world=False)
    ref_vals, ref_ids = oracle_mod.query_vertical(ot, pts)
    dev_tree = on_gpu(tree, gpu)
    vals, ids = dev_tree(pts.to(gpu), want_node_ids=True, world=False)
    assert np.array_equal(ids.cpu().numpy(), ref_ids)
    assert np.array_equal(vals.detach().cpu().numpy(), ref_vals)
    vals, ids = dev_tree(torch.zeros(0, 3, device=gpu), want_node_ids=True)
    assert vals.shape == (0, 4) and ids.shape == (0,)


@pytest.mark.parametrize("generic", [0, 1])
def test_query_backward_matches_oracle_and_index_add(gpu, oracle_mod, generic):
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format="SH4", seed=7)
    g = torch.Generator().manual_seed(3)
    pts = torch.rand(50000, 3, generator=g)
    go = torch.randn(50000, tree.data_dim, generator=g)
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref = oracle_mod.query_vertical_backward(ot, pts, go)
    dev_tree = on_gpu(tree, gpu)
    C.set_debug_flags(generic)
    try:
        vals = dev_tree(pts.to(gpu))
        vals.backward(go.to(gpu))
    finally:
        C.set_debug_flags(0)
    grad = dev_tree.data.grad.cpu().numpy()
    assert grad.shape == tuple(tree.data.shape)
    # float64 index_add as the order-free truth
    _, ids = oracle_mod.query_vertical(ot, pts)
    truth = np.zeros((tree.child.numel(), tree.data_dim))
    np.add.at(truth, ids, go.numpy().astype(np.float64))
    truth = truth.reshape(grad.shape)
    scale = np.abs(truth).max()
    assert np.abs(grad - truth).max() <= 1e-5 * scale
    assert np.abs(ref - truth).max() <= 1e-5 * scale
    # column sums are preserved
    assert np.allclose(grad.reshape(-1, tree.data_dim).sum(0), go.numpy().astype(np.float64).sum(0), rtol=1e-3, atol=1e-2)


def test_assign_vertical(gpu, oracle_mod):
    tree = synth.dense_tree(2, "SH4", seed=9)
    leaves = tree._all_leaves()
    corners = synth._leaf_corners(tree, leaves)
    pick = torch.randperm(leaves.shape[0], generator=torch.Generator().manual_seed(2))[:200]
    pts = (corners[pick] + 0.3 / 8).contiguous()   # distinct leaves: no race
    vals = torch.randn(200, tree.data_dim, generator=torch.Generator().manual_seed(4))
    ref_tree = oracle_mod.Tree(tree.data.data.clone(), tree.child, tree.parent_depth, tree.offset, tree.invradius)
    oracle_mod.assign_vertical(ref_tree, pts, vals)
    dev_tree = on_gpu(tree, gpu)
    dev_tree.set(pts.to(gpu), vals.to(gpu))
    assert np.array_equal(dev_tree.data.data.cpu().numpy(), ref_tree.data)
    # partial rows through the view API: tree[P, :3] = x
    dev_tree[pts.to(gpu), :3] = 7.0
    got = dev_tree(pts.to(gpu))
    assert torch.all(got[:, :3] == 7.0) and torch.equal(got[:, 3:].cpu(), vals[:, 3:])


@pytest.mark.parametrize("name,tree", list(trees()), ids=lambda x: x if isinstance(x, str) else "")
def test_calc_corners_matches_oracle(gpu, oracle_mod, name, tree):
    leaves = tree._all_leaves()
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref = oracle_mod.calc_corners(ot, leaves)
    dev_tree = on_gpu(tree, gpu)
    got = dev_tree._calc_corners(leaves.to(gpu))
    assert np.array_equal(got.cpu().numpy(), ref)
    if tree.N == 2:
        assert np.array_equal(ref, synth._leaf_corners(tree, leaves).numpy())
    # a point just inside the corner maps back to the same leaf
    view = dev_tree[:]
    lengths = view.lengths_local.to(gpu)
    probe = got + 0.25 * lengths[:, None]
    _, ids = dev_tree(probe, want_node_ids=True, world=False)
    assert torch.equal(ids.cpu(), tree._pack_index(leaves))


def test_double_precision_query(gpu, oracle_mod):
    tree = synth.dense_tree(2, "RGBA", seed=12, dtype=torch.float64)
    pts = torch.rand(5000, 3, dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    ot = oracle_mod.Tree.from_n3tree(tree)
    ref_vals, ref_ids = oracle_mod.query_vertical(ot, pts)
    vals, ids = on_gpu(tree, gpu)(pts.to(gpu), want_node_ids=True)
    assert np.array_equal(ids.cpu().numpy(), ref_ids)
    assert np.array_equal(vals.detach().cpu().numpy(), ref_vals)


def test_errors_mirror_reference_checks(gpu):
    tree = on_gpu(synth.dense_tree(1, "RGBA", seed=0), gpu)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        C.query_vertical(tree._spec(), torch.rand(4, 3))
    with pytest.raises(RuntimeError, match="must be contiguous"):
        C.query_vertical(tree._spec(), torch.rand(3, 4, device=gpu).T)
    with pytest.raises(RuntimeError, match="scalar type"):
        C.query_vertical(tree._spec(), torch.rand(4, 3, device=gpu, dtype=torch.float64))


def test_from_grid_and_merge_on_the_gpu(gpu, oracle_mod):
    """from_grid / set_grid write every grid cell into its leaf (svox/svox.py:868-897); a tree with
    merged (freed) nodes still queries and renders like the oracle."""
    g = torch.Generator().manual_seed(11)
    grid = torch.rand(16, 16, 16, 4, generator=g)
    grid[..., -1] *= 6
    tree = svox.N3Tree.from_grid(grid, data_format="RGBA", device=gpu)
    assert tree.n_leaves == 16 ** 3
    from svox_amd.tree import gen_grid
    centres = gen_grid(16).reshape(-1, 3).to(gpu)
    assert torch.equal(tree(centres, world=False).detach().cpu(), grid.reshape(-1, 4))
    # merge half of the frontier nodes: their node rows become free (-1) inside the table
    sel = torch.arange(0, tree.n_frontier, 2)
    assert tree.merge(sel)
    tree.check_integrity()
    host = tree.clone(device="cpu")
    ot = oracle_mod.Tree.from_n3tree(host)
    pts = torch.rand(5000, 3, generator=g)
    ref_vals, ref_ids = oracle_mod.query_vertical(ot, pts)
    vals, ids = tree(pts.to(gpu), want_node_ids=True)
    assert np.array_equal(ids.cpu().numpy(), ref_ids) and np.array_equal(vals.detach().cpu().numpy(), ref_vals)
    rays = synth.sphere_rays(2000, seed=3)
    from util import options, rays_spec
    opt = options(host, step_size=1e-3)
    ref = oracle_mod.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    out = C.volume_render(tree._spec(), rays_spec(rays, gpu), opt)
    assert np.array_equal(out.cpu().numpy(), ref)
