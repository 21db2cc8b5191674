"""Host-side Python layer: tree construction and bookkeeping, views, option packing, argument
checks.  No GPU and no kernels."""
import json
import os

import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))


def test_quick_start_transcript():
    """docs/source/quick.rst:70-85 of the reference."""
    gold = json.load(open(os.path.join(HERE, "golden", "quick_view.json")))
    tree = svox.N3Tree()
    assert list(tree.shape) == gold["shape"]
    tree[0] += 1
    assert tree[:, :3].values.tolist() == gold["after_add_one_to_leaf0_cols0to3"]
    tree[:, -1:] = -1
    assert tree[:2].values.tolist() == gold["after_set_last_col_minus1_first2"]
    assert "N3TreeView(tensor(" in repr(tree[:2])
    assert len(tree) == 8 and tree.numel() == 32 and tree.size(1) == 4 and tree.ndim == 2


@pytest.mark.parametrize("N,levels", [(2, 3), (3, 2), (2, 0)])
def test_uniform_refinement_counts_and_order(N, levels):
    tree = svox.N3Tree(N=N, init_refine=levels)
    nodes = sum(N ** (3 * i) for i in range(levels + 1))
    assert tree.capacity == nodes and tree.n_internal == nodes
    assert tree.n_leaves == N ** (3 * (levels + 1))
    assert tree.check_integrity()
    assert tree.max_depth == levels
    # children are created in lexicographic (node, x, y, z) order of the leaves they split
    if levels > 0:
        root_links = tree.child[0].reshape(-1)
        assert root_links.tolist() == list(range(1, N ** 3 + 1))
        first_child = 1
        pd = tree.parent_depth
        assert pd[first_child].tolist() == [0, 1]
        assert pd[N ** 3].tolist() == [N ** 3 - 1, 1]
    assert tree.child.dtype == torch.int32 and tree.parent_depth.dtype == torch.int32
    assert tree.data.shape == (nodes, N, N, N, 4)


def test_refine_selected_leaves_and_depth_limit():
    tree = svox.N3Tree(depth_limit=1)
    tree.data.data[0, 1, 0, 1] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    resized = tree.refine(sel=(torch.tensor([0]), torch.tensor([1]), torch.tensor([0]), torch.tensor([1])))
    assert resized and tree.n_internal == 2 and tree.n_leaves == 15
    assert tree.child[0, 1, 0, 1] == 1 and tree.parent_depth[1].tolist() == [5, 1]
    # children start as copies of the split leaf, which keeps its own record
    assert torch.equal(tree.data.data[1], torch.tensor([1.0, 2.0, 3.0, 4.0]).expand(2, 2, 2, 4))
    assert tree.data.data[0, 1, 0, 1].tolist() == [1.0, 2.0, 3.0, 4.0]
    tree.refine()       # depth 0 leaves split, depth 1 leaves are at the limit
    assert tree.n_internal == 2 + 7 and tree.check_integrity()
    assert not tree.refine()  # everything is at the limit now
    assert tree.max_depth == 1
    tree._refine_at(0, (0, 0, 0))      # already refined: no-op
    assert tree.n_internal == 9


def test_refine_at_zeroes_the_parent_record():
    tree = svox.N3Tree()
    tree.data.data[0, 0, 1, 1] = 5.0
    tree._refine_at(0, (0, 1, 1))
    assert tree.n_internal == 2 and torch.all(tree.data.data[1] == 5.0)
    assert torch.all(tree.data.data[0, 0, 1, 1] == 0.0)


def test_pack_unpack_round_trip_and_all_leaves_order():
    tree = svox.N3Tree(N=3, init_refine=1)
    leaves = tree._all_leaves()
    assert leaves.shape == (729, 4)
    assert torch.equal(tree._unpack_index(tree._pack_index(leaves)), leaves)
    packed = tree._pack_index(leaves)
    assert torch.all(packed[1:] > packed[:-1])


def test_views_by_index_mask_and_channel():
    tree = svox.N3Tree(init_refine=1, data_format="SH1")
    tree.data.data.copy_(torch.arange(tree.data.numel(), dtype=torch.float32).reshape(tree.data.shape))
    leaves = tree._all_leaves()
    v = tree[5]
    assert v.values.shape == (4,) and torch.equal(v.values.detach(), tree.data.data[tuple(leaves[5])])
    assert tree[3:9].values.shape == (6, 4)
    mask = torch.zeros(64, dtype=torch.bool)
    mask[[1, 7]] = True
    assert tree[mask].shape == (2, 4)
    assert tree[:, -1].values.shape == (64,)
    sub = tree[:, torch.tensor([0, 3])]
    assert sub.values.shape == (64, 2)
    tree[:, torch.tensor([0, 3])] = 9.0
    assert torch.all(tree[:, 0].values == 9.0) and torch.all(tree[:, 1].values != 9.0)
    assert tree.depths.tolist() == [1] * 64
    assert torch.allclose(tree.lengths_local, torch.full((64,), 0.25))
    assert (tree[:2] + 1).shape == (2, 4) and float((tree[0] * 0).sum().detach()) == 0.0
    tree += 1.0
    tree *= 2.0
    assert float(tree[:1, 0].values[0].detach()) == 20.0


def test_view_goes_stale_and_tree_can_be_locked():
    tree = svox.N3Tree()
    view = tree[:]
    tree.refine()
    with pytest.raises(RuntimeError, match="invalidated"):
        _ = view.values
    with tree.accumulate_weights() as acc:
        assert acc.value.shape == tree.child.shape
        with pytest.raises(RuntimeError, match="locked"):
            tree.refine()
    tree.refine()


def test_expand_and_shrink_move_coefficients():
    tree = svox.N3Tree(data_format="SH1")
    tree.data.data[..., :] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    tree.expand("SH4")
    assert tree.data_dim == 13 and repr(tree.data_format) == "SH4"
    row = tree.data.data[0, 0, 0, 0].tolist()
    assert row == [1, 0, 0, 0, 2, 0, 0, 0, 3, 0, 0, 0, 4]
    tree.shrink("SH1")
    assert tree.data.data[0, 0, 0, 0].tolist() == [1, 2, 3, 4]
    rgba = svox.N3Tree()
    rgba.data.data[..., :] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    rgba.expand("RGBA", data_dim=6)
    assert rgba.data.data[0, 0, 0, 0].tolist() == [1, 2, 3, 0, 0, 4]


def test_data_format_parsing():
    f = svox.DataFormat("SH16")
    assert (f.format, f.basis_dim, f.data_dim) == (1, 16, 49) and repr(f) == "SH16"
    f = svox.DataFormat("RGBA")
    assert (f.format, f.basis_dim, f.data_dim) == (0, -1, None) and repr(f) == "RGBA"
    assert svox.DataFormat("").format == 0
    assert (svox.DataFormat("SG7").format, svox.DataFormat("ASG3").format) == (2, 3)
    with pytest.raises(AssertionError):
        svox.DataFormat("SH5")
    with pytest.raises(AssertionError):
        svox.DataFormat("SH36")
    assert svox.N3Tree(data_format="SH9").data_dim == 28 and svox.N3Tree().data_dim == 4
    with pytest.raises(AssertionError):
        svox.N3Tree(data_format="SH9", data_dim=5)


def test_render_options_packing():
    tree = svox.N3Tree(data_format="SH9")
    r = svox.VolumeRenderer(tree, step_size=2e-3, background_brightness=0.5, rgb_padding=0.01)
    o = r._get_options(False)
    assert (o.format, o.basis_dim, o.min_comp, o.max_comp) == (1, 9, 0, 8)
    assert (o.sigma_thresh, o.stop_thresh, o.ndc_width) == (0.0, 0.0, -1)
    o = r._get_options(True)
    assert (o.sigma_thresh, o.stop_thresh) == (1e-2, 1e-2)
    r.sigma_thresh = 0.5
    assert r._get_options(True).sigma_thresh == 0.5 and r._get_options(True).stop_thresh == 1e-2
    r2 = svox.VolumeRenderer(tree, ndc=svox.NDCConfig(100, 50, 80.0), min_comp=2, max_comp=4)
    o = r2._get_options()
    assert (o.ndc_width, o.ndc_height, o.ndc_focal, o.min_comp, o.max_comp) == (100, 50, 80.0, 2, 4)
    packed = o._pack()
    assert packed.basis_dim == 9 and abs(packed.step_size - 1e-3) < 1e-9 and packed.density_softplus == 0
    rgba = svox.VolumeRenderer(svox.N3Tree())._get_options()
    assert (rgba.format, rgba.basis_dim, rgba.max_comp) == (0, -1, -2)
    assert C.out_data_dim(0, -1, 4) == 3 and C.out_data_dim(1, 9, 28) == 3


def test_persp_rays_geometry():
    c2w = synth.look_at_pose([3.0, 0.5, 0.5])
    rays = svox.VolumeRenderer.persp_rays(c2w, 8, 6, 10.0)
    assert rays.origins.shape == (48, 3) and torch.allclose(rays.origins[0], torch.tensor([3.0, 0.5, 0.5]))
    assert torch.allclose(rays.dirs.norm(dim=1), torch.ones(48), atol=1e-6)
    centre = rays.dirs.reshape(6, 8, 3)[3, 4]       # pixel (ix = W/2, iy = H/2) looks along -back
    assert torch.allclose(centre, torch.tensor([-1.0, 0.0, 0.0]), atol=1e-6)


def test_no_cpu_fallback_and_argument_checks():
    tree = synth.dense_tree(1, "RGBA", seed=0)
    with pytest.raises(RuntimeError, match="only the HIP path"):
        tree(torch.rand(3, 3))
    with pytest.raises(RuntimeError, match="only the HIP path"):
        tree.set(torch.rand(3, 3), torch.rand(3, 4))
    with pytest.raises(RuntimeError, match="only the HIP path"):
        svox.VolumeRenderer(tree)(synth.sphere_rays(4))
    with pytest.raises(RuntimeError, match="only the HIP path"):
        svox.VolumeRenderer(tree).render_persp(synth.look_at_pose([2.0, 2, 2]))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        C.query_vertical(tree._spec(), torch.rand(3, 3))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        C.calc_corners(tree._spec(), torch.zeros(2, 4, dtype=torch.long))
    with pytest.raises(AssertionError):
        tree(torch.rand(3, 3, requires_grad=True))


def test_save_load_round_trip(tmp_path):
    """npz persistence (svox/svox.py:835-865, 899-938): the file holds the reference's keys, `data` as
    float16; load gives back exactly the float16-rounded tree."""
    tree = synth.shell_tree(depth=4, n_spheres=2, data_format="SH4", seed=3)
    original = tree.data.data.clone()
    path = str(tmp_path / "tree.npz")
    tree.save(path)
    z = np.load(path)
    assert sorted(z.files) == sorted(["data_dim", "child", "parent_depth", "n_internal", "n_free", "invradius3",
                                      "offset", "depth_limit", "geom_resize_fact", "data", "data_format"])
    assert z["data"].dtype == np.float16 and z["child"].dtype == np.int32 and str(z["data_format"]) == "SH4"
    back = svox.N3Tree.load(path)
    assert torch.equal(back.child, tree.child) and torch.equal(back.parent_depth, tree.parent_depth)
    assert back.n_internal == tree.n_internal and repr(back.data_format) == "SH4"
    assert back.data.dtype == torch.float32
    assert torch.equal(back.data.data, original[:tree.n_internal].half().float())      # exactly the fp16 rounding
    assert not torch.equal(back.data.data, original[:tree.n_internal])                 # ... which is lossy
    assert torch.equal(back.invradius, tree.invradius) and torch.equal(back.offset, tree.offset)
    assert back.depth_limit == tree.depth_limit and back.geom_resize_fact == tree.geom_resize_fact
    assert int(back._n_free) == 0 and back.check_integrity()
    # saving what was loaded is a fixed point: float16 values survive float16 storage
    path2 = str(tmp_path / "again.npz")
    back.save(path2, compress=False)
    again = svox.N3Tree.load(path2, dtype=torch.float64)
    assert again.data.dtype == torch.float64 and torch.equal(again.data.data.float(), back.data.data)
    # an SG tree keeps its lobes
    sg = svox.N3Tree(data_format="SG2", init_refine=1, extra_data=torch.rand(2, 4))
    sg.save(str(tmp_path / "sg.npz"))
    assert torch.equal(svox.N3Tree.load(str(tmp_path / "sg.npz")).extra_data, sg.extra_data)


def test_load_reads_the_legacy_file_layout(tmp_path):
    """Files written before `invradius3`, `n_free` and `data_format` existed (svox/svox.py:920-934):
    a scalar `invradius` fills all three axes, `n_free` defaults to 0, the format to None (the
    renderer then infers SH from data_dim, svox/renderer.py:171-176)."""
    tree = synth.dense_tree(2, "SH4", seed=4, sigma="lognormal")
    n = tree.n_internal
    path = str(tmp_path / "legacy.npz")
    np.savez(path, data_dim=np.int64(tree.data_dim), child=tree.child[:n].numpy(), parent_depth=tree.parent_depth[:n].numpy(),
             n_internal=np.int64(n), invradius=np.float64(0.25), offset=np.array([0.5, 0.25, 0.125]),
             depth_limit=np.int64(7), geom_resize_fact=np.float64(1.5), data=tree.data.data[:n].numpy().astype(np.float16))
    back = svox.N3Tree.load(path)
    assert torch.equal(back.invradius, torch.full((3,), 0.25)) and back.invradius.dtype == torch.float32
    assert torch.equal(back.offset, torch.tensor([0.5, 0.25, 0.125])) and back.offset.dtype == torch.float32
    assert int(back._n_free) == 0 and back.data_format is None and back.depth_limit == 7
    assert back.geom_resize_fact == 1.5 and back.N == 2 and back.data_dim == 13 and back.n_internal == n
    assert torch.equal(back.data.data, tree.data.data[:n].half().float()) and back.check_integrity()
    with pytest.warns(UserWarning, match="Legacy N3Tree"):
        r = svox.VolumeRenderer(back)
    assert repr(r.data_format) == "SH4"
    # a freed node count that is stored is honoured
    blob = dict(np.load(path))
    blob["n_free"] = np.int64(2)
    np.savez(str(tmp_path / "freed.npz"), **blob)
    assert int(svox.N3Tree.load(str(tmp_path / "freed.npz"))._n_free) == 2


def test_generators_are_seeded():
    a = synth.shell_tree(depth=5, n_spheres=3, data_format="SH1", seed=5)
    b = synth.shell_tree(depth=5, n_spheres=3, data_format="SH1", seed=5)
    c = synth.shell_tree(depth=5, n_spheres=3, data_format="SH1", seed=6)
    assert torch.equal(a.child, b.child) and torch.equal(a.data.data, b.data.data)
    assert a.child.shape != c.child.shape or not torch.equal(a.child, c.child)
    assert a.check_integrity() and 0 < a.info["occupancy"] < 0.5
    r1, r2 = synth.sphere_rays(10, seed=1), synth.sphere_rays(10, seed=1)
    assert torch.equal(r1.origins, r2.origins) and torch.allclose((r1.origins - 0.5).norm(dim=1), torch.full((10,), 2.0))
    noise = synth.shell_tree(depth=6, data_format="SH1", seed=2, geometry="noise")
    assert noise.check_integrity() and noise.info["occupied_leaves"] > 0


def test_frontier_reductions_and_merge():
    """merge() undoes refine() on frontier nodes; reductions see the N^3 child records
    (svox/svox.py:436-580)."""
    tree = svox.N3Tree(N=2, data_format="RGBA", init_refine=1)                 # 1 + 8 nodes, 64 leaves
    g = torch.Generator().manual_seed(0)
    tree.data.data.copy_(torch.rand(tree.data.shape, generator=g))
    assert tree.n_frontier == 8 and (tree.frontier_depth == 1).all()
    block = tree.data.data[tree._frontier].view(8, 8, 4)
    assert torch.equal(tree.reduce_frontier(torch.mean), block.mean(dim=1))
    assert torch.equal(tree.max_frontier(dim=-1), block[..., -1].max(dim=1)[0])
    diam = tree.diam_frontier()
    brute = torch.stack([torch.cdist(b, b).max() for b in block])
    assert torch.allclose(diam, brute)
    out = tree.reduce_frontier(torch.mean, grad=True)
    out.sum().backward()
    assert tree.data.grad is not None and tree.data.grad[1:].abs().sum() > 0
    tree.data.grad = None
    # merge three of the eight frontier nodes with max
    picked = tree._frontier[torch.tensor([0, 3, 5])]
    want = tree.data.data[picked].view(3, 8, 4).max(dim=1)[0]
    parents = tuple(tree._unpack_index(tree.parent_depth[picked, 0].long()).T)
    assert tree.merge(torch.tensor([0, 3, 5]), op=torch.max)
    assert torch.equal(tree.data.data[parents], want)
    assert (tree.child[parents] == 0).all() and (tree.child[picked] == -1).all()
    assert tree.n_leaves == 64 - 3 * 8 + 3 and tree.n_frontier == 5
    tree.check_integrity()
    assert tree.shrink_to_fit() and tree.capacity == 6
    tree.check_integrity()
    assert tree.n_leaves == 43
    # merging everything that is left leaves the root alone
    assert tree.merge()
    tree.shrink_to_fit()
    assert tree.capacity == 1 and tree.n_leaves == 8
    with pytest.raises(RuntimeError, match="Cannot merge root"):
        tree.merge()


def test_gen_grid_centres():
    from svox_amd.tree import gen_grid
    grid = gen_grid(4)
    assert grid.shape == (4, 4, 4, 3)
    assert torch.allclose(grid[1, 2, 3], torch.tensor([0.375, 0.625, 0.875]))


def test_tree_keeps_marks_only_while_it_is_unchanged():
    """The bookkeeping around N3Tree.mark_empty_leaves() (the marks themselves come from a kernel):
    _spec() hands the marks on while nothing has changed and drops them after a write through a view,
    an in-place torch operation, a change of structure or a move; one large call makes its own."""
    tree = svox.N3Tree(data_format="SH4", init_refine=2)

    def pretend_marked():
        tree._leaf_marks = torch.zeros_like(tree.child)
        tree._leaf_marks_key = tree._marks_key()

    assert tree._spec().child_marks is None
    pretend_marked()
    assert tree._spec().child_marks is tree._leaf_marks
    assert tree._spec(world=False).child_marks is tree._leaf_marks
    tree[0, -1:] = 5.0                      # a view writes through data.data: no version counter moves
    assert tree._spec().child_marks is None
    pretend_marked()
    with torch.no_grad():
        tree.data.add_(1.0)
    assert tree._spec().child_marks is None and tree._leaf_marks is None
    pretend_marked()
    tree.refine(sel=(torch.tensor([0]), torch.tensor([0]), torch.tensor([0]), torch.tensor([0])))
    assert tree._spec().child_marks is None
    pretend_marked()
    tree.clear_leaf_marks()
    assert tree._spec().child_marks is None
    pretend_marked()
    tree.double()                           # new storage for data
    assert tree._spec().child_marks is None
    # the size from which a call marks the leaves for itself
    spec = tree.float()._spec()
    opt = svox.VolumeRenderer(tree)._get_options(True)
    assert C.AUTO_MARK_RAYS_PER_CELL * tree.child.numel() > 10
    assert C._marks_for_this_call(spec, opt, 10) is None
    spec.child_marks = torch.zeros_like(tree.child)
    assert C._marks_for_this_call(spec, opt, 10 ** 9) is None       # the caller brought marks


def test_notes_budget_grows_when_the_notes_ran_out_and_shrinks_when_they_are_not_used():
    from svox_amd.renderer import NotesBudget
    from svox_amd import csrc as C
    b = NotesBudget()
    base = int(C.BACKWARD_RECORDS_PER_RAY)
    assert b.records_per_ray() == base
    b.adjust(asked=10, pool=10)          # every stock handed out: the notes ran out (or just fitted)
    assert b.factor == 2 and b.records_per_ray() == 2 * base
    b.adjust(asked=40, pool=30)
    assert b.factor == 4
    b.adjust(asked=20, pool=30)          # fits, and more than a quarter is used: stay
    assert b.factor == 4
    b.adjust(asked=7, pool=30)           # under a quarter: halve
    assert b.factor == 2
    b.adjust(asked=0, pool=30)
    b.adjust(asked=0, pool=30)
    assert b.factor == 1                 # never below the start
    for _ in range(10):
        b.adjust(asked=99, pool=1)
    assert b.factor == NotesBudget.MAX_FACTOR
    import copy
    import pickle
    assert copy.deepcopy(b).factor == b.factor and pickle.loads(pickle.dumps(b)).factor == b.factor


def test_notes_pool_info_matches_the_documented_workspace_layout():
    import ctypes
    from svox_amd.csrc import _abi
    lib = _abi.load_library()
    n = 1000
    nbytes = int(lib.svox_volume_render_backward_workspace_bytes(n, 30))
    offset, pool = ctypes.c_int64(), ctypes.c_int64()
    assert lib.svox_notes_pool_info(n, nbytes, ctypes.byref(offset), ctypes.byref(pool)) == 0
    # chunks, then one bit per ray (rounded to 16 bytes), then 256 bytes whose second half starts with the counter
    chunks = (nbytes - 256 - 16 * ((n + 127) // 128)) // 384
    assert chunks == 2 * n
    assert offset.value == chunks * 384 + 16 * ((n + 127) // 128) + 128 and offset.value % 8 == 0
    assert pool.value == (chunks - n + 63) // 64
    assert lib.svox_notes_pool_info(n, 384 * (n - 1), ctypes.byref(offset), ctypes.byref(pool)) == -2
    assert lib.svox_notes_pool_info(n, nbytes, None, ctypes.byref(pool)) == -1


def test_the_public_names_of_the_reference_are_all_there():
    """Every public method and property of the reference's N3Tree (svox/svox.py:57-1113), N3TreeView
    (svox/helpers.py:27-358, with the operators it forwards to `.values`) and VolumeRenderer
    (svox/renderer.py:114-469), plus the names svox/__init__.py exports."""
    from svox_amd.view import N3TreeView
    tree_names = """__call__ __getitem__ __setitem__ __iadd__ __isub__ __imul__ __idiv__ __len__ __repr__
        accumulate_weights capacity check_integrity clone diam_frontier expand forward from_grid frontier_depth
        load max_depth max_frontier merge n_frontier n_internal n_leaves ndim numel partial reduce_frontier refine
        save set set_grid shape shrink shrink_to_fit size snap tree2world world2tree
        depths lengths lengths_local corners corners_local values values_local sample sample_local aux
        normal_ clamp_ uniform_ relu_ sigmoid_ nan_to_num_""".split()
    view_names = """__repr__ __setitem__ __torch_function__ aux clamp_ corners corners_local depths lengths
        lengths_local nan_to_num_ ndim normal_ refine relu_ sample sample_local set shape sigmoid_ uniform_
        values values_nograd
        __floordiv__ __mod__ __div__ __eq__ __ne__ __ge__ __gt__ __le__ __lt__ __floor__ __ceil__ __round__
        __len__ item size dim numel __add__ __mul__ __sub__ __truediv__ __radd__ __rsub__ __rmul__ __rdiv__
        __abs__ __pos__ __neg__ clamp clamp_max clamp_min relu sigmoid max min mean sum __getitem__""".split()
    renderer_names = "forward render_persp se_grad se_grad_persp persp_rays data_format _get_options".split()
    assert [n for n in tree_names if not hasattr(svox.N3Tree, n)] == []
    assert [n for n in view_names if not hasattr(N3TreeView, n)] == []
    assert [n for n in renderer_names if not hasattr(svox.VolumeRenderer, n)] == []
    for name in ("N3Tree", "VolumeRenderer", "NDCConfig", "Rays", "DataFormat", "LocalIndex"):
        assert hasattr(svox, name), name
    # the in-place division the reference spells __idiv__ works as `/=`
    tree = svox.N3Tree(data_dim=4, init_refine=1)
    tree.data.data.fill_(3.0)
    tree /= 2.0
    assert torch.all(tree[:].values == 1.5)            # (the leaves; cells of inner nodes are no part of tree[:])
    assert torch.equal((tree[0] / 3.0), tree[0].values / 3.0)
