"""What pins the CPU oracle (oracle/svox_oracle.cpp) -- no GPU needed.

Each test fixes one of the oracle's functions against something the oracle did not produce:
the reference's recorded output, a closed form, a library routine, brute force, finite differences,
or torch.autograd through an independently written restatement of the reference's fallback.
"""
import json
import os

import numpy as np
import pytest
import torch

import svox_amd as svox
from oracle import oracle, torch_fallback
from svox_amd import synth
from util import options

HERE = os.path.dirname(os.path.abspath(__file__))


# ------------------------------------------------------------------------------------------
# exp / sigmoid
# ------------------------------------------------------------------------------------------
def ulp_err(got, x):
    true = np.exp(x.astype(np.float64))
    ulp = np.spacing(true.astype(np.float32)).astype(np.float64)
    return np.abs(got.astype(np.float64) - true) / ulp


def test_expf_is_within_one_ulp_and_handles_the_ends():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.uniform(-87, 88.7, 40000), rng.uniform(-2, 2, 20000),
                        np.linspace(-87, 88.7, 5001), [0.0, -0.0, 1.0, -1.0]]).astype(np.float32)
    got = oracle.expf(x)
    assert ulp_err(got, x).max() <= 1.0
    assert oracle.expf(np.float32(0.0)) == 1.0
    assert np.all(oracle.expf(np.array([-87.5, -100, -1e30, -np.inf], np.float32)) == 0.0)
    assert np.all(np.isinf(oracle.expf(np.array([88.8, 1e30, np.inf], np.float32))))
    assert np.isnan(oracle.expf(np.float32(np.nan)))
    # nothing subnormal ever comes out
    tiny = oracle.expf(np.linspace(-87, -86, 1001).astype(np.float32))
    assert tiny.min() >= np.finfo(np.float32).tiny


# ------------------------------------------------------------------------------------------
# basis functions
# ------------------------------------------------------------------------------------------
def real_sh_scipy(dirs, degree):
    """Textbook real spherical harmonics from scipy's complex ones, index l*l + l + m."""
    from scipy.special import sph_harm_y
    x, y, z = dirs.T
    theta = np.arccos(np.clip(z, -1, 1))
    phi = np.arctan2(y, x)
    out = np.zeros((dirs.shape[0], (degree + 1) ** 2))
    for l in range(degree + 1):
        for m in range(-l, l + 1):
            Y = sph_harm_y(l, abs(m), theta, phi)
            if m == 0:
                v = Y.real
            elif m > 0:
                v = np.sqrt(2) * (-1) ** m * Y.real
            else:
                v = np.sqrt(2) * (-1) ** m * Y.imag
            out[:, l * l + l + m] = v
    return out


@pytest.mark.parametrize("basis_dim", [1, 4, 9, 16, 25])
def test_sh_basis_is_the_textbook_one_up_to_the_reference_sign(basis_dim):
    rng = np.random.default_rng(1)
    d = rng.normal(size=(500, 3))
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    got = oracle.basis(svox.DataFormat.SH, basis_dim, d.astype(np.float64))
    degree = int(round(basis_dim ** 0.5)) - 1
    std = real_sh_scipy(d, degree)
    # the reference's table carries a factor (-1)^m relative to the textbook real harmonics
    sign = np.array([(-1.0) ** m for l in range(degree + 1) for m in range(-l, l + 1)])
    assert np.abs(got - std * sign).max() < 2e-6
    got32 = oracle.basis(svox.DataFormat.SH, basis_dim, d.astype(np.float32))
    assert np.abs(got32 - std * sign).max() < 5e-6
    # same numbers as the reference's Python table, restated in torch
    fb = torch_fallback.eval_sh_bases(basis_dim, torch.from_numpy(d)).numpy()
    assert np.abs(got - fb).max() < 2e-6


def test_sg_and_asg_lobes_follow_their_formulas():
    rng = np.random.default_rng(2)
    d = rng.normal(size=(64, 3))
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    mu = rng.normal(size=(6, 3))
    mu /= np.linalg.norm(mu, axis=1, keepdims=True)
    lam = rng.uniform(0.5, 5, size=(6, 1))
    got = oracle.basis(svox.DataFormat.SG, 6, d, np.concatenate([lam, mu], 1))
    want = np.exp(lam.T * (d @ mu.T - 1.0)) / 6
    assert np.abs(got - want).max() < 1e-6     # expf is single precision in every build
    frames = np.linalg.qr(rng.normal(size=(5, 3, 3)))[0]
    lxy = rng.uniform(0.5, 3, size=(5, 2))
    extra = np.concatenate([lxy, frames.reshape(5, 9)], 1)
    got = oracle.basis(svox.DataFormat.ASG, 5, d, extra)
    ax, ay, az = frames[:, 0], frames[:, 1], frames[:, 2]
    want = (d @ az.T) * np.exp(-lxy[:, 0] * (d @ ax.T) ** 2 - lxy[:, 1] * (d @ ay.T) ** 2) / 5
    assert np.abs(got - want).max() < 1e-6


# ------------------------------------------------------------------------------------------
# point queries
# ------------------------------------------------------------------------------------------
def descend_python(child, N, p):
    """Ten-line tree walk in Python integers / floats."""
    p = [min(max(float(c), 0.0), float(np.float32(1.0) - np.float32(1e-6))) for c in p]
    node = 0
    for level in range(1, 40):
        p = [c * N for c in p]
        idx = [int(np.floor(c)) for c in p]
        p = [c - i for c, i in zip(p, idx)]
        skip = int(child[node, idx[0], idx[1], idx[2]])
        if skip == 0:
            return ((node * N + idx[0]) * N + idx[1]) * N + idx[2], level
        node += skip
    raise AssertionError("no leaf")


def test_query_matches_brute_force_on_dense_and_sparse_trees():
    g = torch.Generator().manual_seed(0)
    for tree in (synth.dense_tree(3, "RGBA", seed=0), synth.shell_tree(depth=6, n_spheres=4, data_format="SH1", seed=1)):
        pts = torch.rand(400, 3, generator=g) * 1.1 - 0.05
        ot = oracle.Tree.from_n3tree(tree)
        vals, ids, levels = oracle.query_vertical(ot, pts, want_levels=True)
        child = tree.child.numpy()
        flat = tree.data.detach().numpy().reshape(-1, tree.data_dim)
        for q in range(pts.shape[0]):
            leaf, lv = descend_python(child, 2, pts[q].tolist())
            assert ids[q] == leaf and levels[q] == lv
            assert np.array_equal(vals[q], flat[leaf])


def test_dense_tree_leaf_is_the_grid_cell_and_layout_is_breadth_first():
    tree = synth.dense_tree(3, "RGBA", seed=3)        # 16^3 leaves
    ot = oracle.Tree.from_n3tree(tree)
    rng = np.random.default_rng(5)
    pts = rng.uniform(0, 1, size=(2000, 3)).astype(np.float32)
    _, ids = oracle.query_vertical(ot, pts)
    cells = np.floor(pts.astype(np.float64) * 16).astype(np.int64)
    # breadth-first layout of repeated refine(): the node of level l containing grid cell c has
    # index (number of nodes above level l) + Morton-like rank of its parent path
    node = np.zeros(len(pts), dtype=np.int64)
    first = 0
    count = 1
    for level in range(3):
        bit = (cells >> (3 - level)) & 1
        cell_in_node = bit[:, 0] * 4 + bit[:, 1] * 2 + bit[:, 2]
        rank = (node - first) * 8 + cell_in_node
        first += count
        count *= 8
        node = first + rank
    bit = cells & 1
    want = node * 8 + bit[:, 0] * 4 + bit[:, 1] * 2 + bit[:, 2]
    assert np.array_equal(ids, want)


def test_query_clamps_like_the_reference():
    tree = synth.dense_tree(1, "RGBA", seed=0)        # 4^3 leaves
    ot = oracle.Tree.from_n3tree(tree)
    hi = np.frombuffer(np.uint32(0x3F7FFFEF).tobytes(), np.float32)[0]
    pts = np.array([[-5, -0.0, 0.0], [1.0, 2.0, 1e9], [hi, hi, hi], [np.nan, 0.1, 0.1],
                    [np.float32(1) - np.float32(2 ** -24), 0.5, 0.25]], np.float32)
    _, ids = oracle.query_vertical(ot, pts)
    last = descend_python(tree.child.numpy(), 2, [0.9999, 0.9999, 0.9999])[0]
    assert ids[0] == descend_python(tree.child.numpy(), 2, [0, 0, 0])[0]
    assert ids[1] == last and ids[2] == last
    assert ids[3] == descend_python(tree.child.numpy(), 2, [0.9999, 0.1, 0.1])[0]   # NaN -> upper bound
    assert ids[4] == descend_python(tree.child.numpy(), 2, [0.9999, 0.5, 0.25])[0]
    assert float(np.float32(1.0 - 1e-6)) == float(hi)


def test_query_backward_is_index_add():
    tree = synth.shell_tree(depth=5, n_spheres=3, data_format="SH1", seed=4)
    g = torch.Generator().manual_seed(2)
    pts = torch.rand(3000, 3, generator=g)
    go = torch.randn(3000, 4, generator=g)
    ot = oracle.Tree.from_n3tree(tree)
    grad = oracle.query_vertical_backward(ot, pts, go)
    _, ids = oracle.query_vertical(ot, pts)
    want = np.zeros((tree.child.numel(), 4))
    np.add.at(want, ids, go.numpy().astype(np.float64))
    assert np.abs(grad.reshape(-1, 4) - want).max() < 1e-5


def test_corners_closed_form_and_round_trip():
    tree = synth.shell_tree(depth=6, n_spheres=3, data_format="SH1", seed=6)
    leaves = tree._all_leaves()
    ot = oracle.Tree.from_n3tree(tree)
    corners = oracle.calc_corners(ot, leaves)
    depth = tree.parent_depth[leaves[:, 0], 1].numpy()
    size = 2.0 ** -(depth + 1.0)
    # a corner is a multiple of the leaf size, and the leaf's centre queries back to the leaf
    assert np.array_equal(corners / size[:, None], np.round(corners / size[:, None]))
    centre = (corners + 0.5 * size[:, None]).astype(np.float32)
    _, ids = oracle.query_vertical(oracle.Tree.from_n3tree(tree, world=False), centre)
    assert np.array_equal(ids, tree._pack_index(leaves).numpy())
    assert np.array_equal(corners, synth._leaf_corners(tree, leaves).numpy())


# ------------------------------------------------------------------------------------------
# forward rendering
# ------------------------------------------------------------------------------------------
def test_reference_docs_example_is_reproduced():
    """docs/source/ex_opt_toy.rst:20-44: 20 + 20 gradient steps on one ray, SH1 then SH4."""
    gold = json.load(open(os.path.join(HERE, "golden", "ex_opt_toy.json")))
    setup = gold["setup"]
    t = svox.N3Tree(data_format=setup["data_format"])
    t.data.data[0, 0, 0, 0, :-1] = setup["leaf_colour_coeffs"]
    t.data.data[0, 0, 0, 0, -1] = setup["leaf_sigma"]
    r = svox.VolumeRenderer(t)
    o = np.array([setup["ray_origin"]], np.float32)
    d = np.array([setup["ray_dir"]], np.float32)
    target = np.array([setup["target"]], np.float32)

    def phase():
        printed = []
        for i in range(setup["steps_per_phase"]):
            ot = oracle.Tree.from_n3tree(t)
            opt = r._get_options(False)
            rend = oracle.volume_render(ot, o, d, d, opt)
            if i % setup["print_every"] == 0:
                printed.append(rend[0].copy())
            grad = oracle.volume_render_backward(ot, o, d, d, opt, (2 * (rend - target)).astype(np.float32))
            t.data.data -= setup["lr"] * torch.from_numpy(grad)
        return np.array(printed)

    p1 = phase()
    # first printed line is a closed form: one leaf of length 0.5 (+ step) at sigma 0.5, grey colour
    att = np.exp(-(0.5 + 1e-3) * 0.5)
    assert abs(p1[0, 0] - ((1 - att) * 0.5 + att)) < 1e-7
    t.expand(setup["expand_to"])
    p2 = phase()
    assert np.abs(p1 - np.array(gold["phase1"])).max() < 1.5e-7
    assert np.abs(p2 - np.array(gold["phase2"])).max() < 1.5e-7


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_constant_density_closed_form(dtype):
    """Uniform 16^3 grid, constant sigma and colour, axis-aligned ray: 16 leaves.  Every step runs to
    the leaf's exit plus step_size, so the next sample starts step_size inside its leaf and the step
    lengths telescope to chord + step_size."""
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    tree = svox.N3Tree(init_refine=3, dtype=tdt)
    sigma, colour, step, bg = 3.0, 0.7, 1e-3, 0.25
    tree.data.data[..., :3] = colour
    tree.data.data[..., 3] = sigma
    opt = options(tree, step_size=step, background_brightness=bg)
    o = np.array([[0.3, 0.61, -1.0], [0.3, 2.0, 0.4], [-3.0, 0.2, 0.7]], dtype)
    d = np.array([[0, 0, 1.0], [0, -1.0, 0], [2.0, 0, 0]], dtype)      # the last one is not unit length
    ot = oracle.Tree.from_n3tree(tree)
    out, stats = oracle.volume_render(ot, o, d, d, opt, want_stats=True)
    assert stats["samples"] == 48 and stats["levels"] == 48 * 4
    depth = sigma * (1.0 + step)
    want = (1 - np.exp(-depth)) / (1 + np.exp(-colour)) + np.exp(-depth) * bg
    assert np.abs(out[:2] - want).max() < (2e-6 if dtype == np.float32 else 1e-7)
    # a direction of length 2 halves delta_scale: optical depth is measured in units of |dir|
    want2 = (1 - np.exp(-depth / 2)) / (1 + np.exp(-colour)) + np.exp(-depth / 2) * bg
    assert np.abs(out[2] - want2).max() < (2e-6 if dtype == np.float32 else 1e-7)
    visits = oracle.trace_visits(ot, o, d, d, 0, opt)
    assert len(visits["leaf"]) == 16 and len(set(visits["leaf"].tolist())) == 16
    assert abs(visits["delta_t"][0] - (1 / 16 + step)) < 1e-6
    assert np.allclose(visits["delta_t"][1:], 1 / 16, atol=1e-6)
    assert np.allclose(np.diff(visits["t"]), visits["delta_t"][:-1], atol=1e-6)


def test_diagonal_ray_visits_the_cells_a_dense_walk_finds():
    tree = svox.N3Tree(init_refine=2, dtype=torch.float64)      # 8^3
    tree.data.data[..., 3] = 1.0
    opt = options(tree, step_size=1e-4)
    o = np.array([[-0.2, 0.13, 0.05]])
    d = np.array([[0.8, 0.45, 0.39]])
    d /= np.linalg.norm(d)
    ot = oracle.Tree.from_n3tree(tree)
    visits = oracle.trace_visits(ot, o, d, d, 0, opt)
    # dense sampling of the same segment: the ordered set of grid cells it passes through
    ts = np.linspace(0, 3, 600001)
    p = o + ts[:, None] * d
    inside = np.all((p >= 0) & (p < 1), axis=1)
    cells = np.floor(p[inside] * 8).astype(int)
    keys = cells[:, 0] * 64 + cells[:, 1] * 8 + cells[:, 2]
    order = keys[np.concatenate([[True], keys[1:] != keys[:-1]])]
    _, ids = oracle.query_vertical(ot, (np.array([[c // 64, (c // 8) % 8, c % 8] for c in order]) + 0.5) / 8)
    # the marcher may skip a cell whose crossing is shorter than step_size, never add one
    it = iter(ids.tolist())
    assert all(any(v == w for w in it) for v in visits["leaf"].tolist())
    assert len(visits["leaf"]) >= len(ids) - 3
    # step lengths telescope: chord plus the final overshoot of one step_size
    chord = ts[inside][-1] - ts[inside][0]
    assert abs(visits["delta_t"].sum() - (chord + 1e-4)) < 2e-5


def test_forward_invariants():
    tree = synth.dense_tree(3, "RGBA", seed=0)
    rays = synth.sphere_rays(512, seed=1)
    ot = oracle.Tree.from_n3tree(tree)
    # rays that miss the cube return exactly the background
    out = oracle.volume_render(ot, rays.origins, -rays.dirs, rays.viewdirs, options(tree, background_brightness=0.3))
    assert np.all(out == np.float32(0.3))
    # a threshold above every sigma leaves exactly the background too
    opt = options(tree, sigma_thresh=1e9, stop_thresh=0.0, background_brightness=0.6)
    out = oracle.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)
    assert np.all(out == np.float32(0.6))
    # saturated colours and white background: weights and the remaining light sum to one
    t2 = synth.dense_tree(3, "RGBA", seed=0)
    t2.data.data[..., :3] = 40.0
    out = oracle.volume_render(oracle.Tree.from_n3tree(t2), rays.origins, rays.dirs, rays.viewdirs, options(t2))
    assert np.abs(out - 1.0).max() < 1e-5
    # min_comp > max_comp renders mid grey where opaque
    t3 = svox.N3Tree(data_format="SH4", init_refine=1)
    t3.data.data.normal_(generator=torch.Generator().manual_seed(0))
    t3.data.data[..., -1] = 1e4
    out = oracle.volume_render(oracle.Tree.from_n3tree(t3), rays.origins, rays.dirs, rays.viewdirs,
                               options(t3, min_comp=2, max_comp=1))
    assert np.abs(out - 0.5).max() < 1e-6


def test_early_stop_rescales_and_skips_the_background():
    tree = svox.N3Tree(init_refine=1)
    tree.data.data[..., :3] = 0.0
    tree.data.data[..., 3] = 20.0
    o = np.array([[0.4, 0.4, -1.0]], np.float32)
    d = np.array([[0, 0, 1.0]], np.float32)
    ot = oracle.Tree.from_n3tree(tree)
    opt = options(tree, step_size=1e-3, sigma_thresh=0.0, stop_thresh=1e-2, background_brightness=0.0)
    out = oracle.volume_render(ot, o, d, d, opt)
    # after the first leaf (0.25 + step long) light = exp(-5.02) < 1e-2: colour/(1-light), no background
    assert np.abs(out - 0.5).max() < 1e-6
    visits = oracle.trace_visits(ot, o, d, d, 0, opt)
    assert len(visits["leaf"]) == 1


def test_fp32_and_fp64_oracles_agree():
    tree = synth.shell_tree(depth=5, n_spheres=4, data_format="SH9", seed=2)
    rays = synth.sphere_rays(800, seed=3)
    opt = options(tree, step_size=1e-3)
    out32 = oracle.volume_render(oracle.Tree.from_n3tree(tree), rays.origins, rays.dirs, rays.viewdirs, opt)
    t64 = tree.double()
    out64 = oracle.volume_render(oracle.Tree.from_n3tree(t64), rays.origins.double(), rays.dirs.double(),
                                 rays.viewdirs.double(), opt)
    # a sample that lands within rounding of a cell face may pick the other cell in one precision
    err = np.abs(out32 - out64).max(axis=1)
    assert np.median(err) < 1e-6 and np.mean(err > 1e-4) < 0.02


def test_fallback_restatement_agrees_with_the_oracle():
    """The reference's PyTorch fallback (restated, batch bug fixed) and the kernel semantics agree to
    rounding on a scene where their documented differences do not bite."""
    tree = synth.dense_tree(3, "RGBA", seed=0)
    rays = synth.sphere_rays(1024, seed=0)
    ot = oracle.Tree.from_n3tree(tree)
    ref = oracle.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, options(tree))
    out = torch_fallback.render(tree.data.detach(), tree.child, tree.parent_depth, tree.invradius, tree.offset,
                                rays.origins, rays.dirs, rays.viewdirs, -1).numpy()
    err = np.abs(out - ref).max(axis=1)
    assert np.median(err) < 1e-6 and err.max() < 1e-3
    t2 = synth.dense_tree(2, "SH9", seed=1, sigma="lognormal", coeff_std=0.5)
    ref = oracle.volume_render(oracle.Tree.from_n3tree(t2), rays.origins, rays.dirs, rays.viewdirs, options(t2))
    out = torch_fallback.render(t2.data.detach(), t2.child, t2.parent_depth, t2.invradius, t2.offset,
                                rays.origins, rays.dirs, rays.viewdirs, 9).numpy()
    err = np.abs(out - ref).max(axis=1)
    assert np.median(err) < 1e-6 and err.max() < 1e-3


# ------------------------------------------------------------------------------------------
# backward
# ------------------------------------------------------------------------------------------
def test_gradient_matches_finite_differences_in_double():
    tree = svox.N3Tree(data_format="SH4", init_refine=1, dtype=torch.float64)     # 64 leaves
    g = torch.Generator().manual_seed(0)
    tree.data.data.normal_(generator=g)
    tree.data.data[..., -1] = tree.data.data[..., -1].abs() * 3
    rays = synth.sphere_rays(40, seed=4, dtype=torch.float64)
    go = torch.randn(40, 3, generator=g, dtype=torch.float64).numpy()
    opt = options(tree, step_size=1e-3, rgb_padding=0.01)
    o, d, v = rays.origins.numpy(), rays.dirs.numpy(), rays.viewdirs.numpy()

    def loss(data):
        ot = oracle.Tree(data, tree.child, tree.parent_depth, tree.offset, tree.invradius)
        return float((oracle.volume_render(ot, o, d, v, opt) * go).sum())

    base = tree.data.detach().numpy().copy()
    grad = oracle.volume_render_backward(oracle.Tree(base, tree.child, tree.parent_depth, tree.offset,
                                                     tree.invradius), o, d, v, opt, go)
    rng = np.random.default_rng(0)
    flat = np.flatnonzero(np.abs(grad) > 1e-6)
    assert flat.size > 100
    worst = 0.0
    for idx in rng.choice(flat, 60, replace=False):
        # exp is evaluated in single precision inside the double oracle, so steps must be coarse
        h = 1e-2
        plus, minus = base.copy(), base.copy()
        plus.flat[idx] += h
        minus.flat[idx] -= h
        fd = (loss(plus) - loss(minus)) / (2 * h)
        worst = max(worst, abs(fd - grad.flat[idx]) / max(abs(grad.flat[idx]), 1e-3))
    assert worst < 5e-3


def test_gradient_matches_autograd_through_the_fallback_restatement():
    for fmt, basis in (("RGBA", -1), ("SH4", 4)):
        tree = synth.dense_tree(2, fmt, seed=7, sigma="lognormal", coeff_std=0.7)
        rays = synth.sphere_rays(600, seed=5)
        go = torch.randn(600, 3, generator=torch.Generator().manual_seed(3))
        data = tree.data.detach().clone().requires_grad_(True)
        out = torch_fallback.render(data, tree.child, tree.parent_depth, tree.invradius, tree.offset,
                                    rays.origins, rays.dirs, rays.viewdirs, basis)
        out.backward(go)
        grad = oracle.volume_render_backward(oracle.Tree.from_n3tree(tree), rays.origins, rays.dirs,
                                             rays.viewdirs, options(tree), go)
        want = data.grad.numpy()
        assert np.abs(grad - want).max() <= 2e-4 * np.abs(want).max()


def test_backward_ignores_thresholds_and_misses():
    tree = synth.dense_tree(2, "RGBA", seed=9)
    rays = synth.sphere_rays(200, seed=6)
    go = torch.randn(200, 3, generator=torch.Generator().manual_seed(1))
    ot = oracle.Tree.from_n3tree(tree)
    g_plain = oracle.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, options(tree), go)
    g_fast = oracle.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, options(tree, fast=True), go)
    assert np.array_equal(g_plain, g_fast)            # rt_kernel.cu:377,441 test sigma > 0 only
    g_miss = oracle.volume_render_backward(ot, rays.origins, -rays.dirs, rays.viewdirs, options(tree), go)
    assert not g_miss.any()


def test_exact_sum_mode_is_the_float64_sum_of_the_per_ray_terms():
    """exact_sum: every ray's terms as the reference forms them (fp32), added in float64, rounded once.
    Pinned without the oracle's own adder: each ray alone gives at most one term per element, so the
    per-ray gradients ARE the terms; numpy adds them in float64.  Also: the result does not depend on
    the order of the rays or the thread count, and the plain fp32 order stays close to it."""
    tree = synth.dense_tree(2, "SH4", seed=13, sigma="lognormal", coeff_std=0.7)
    n = 240
    rays = synth.sphere_rays(n, seed=12)
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(5))
    ref_colour = torch.rand(n, 3, generator=torch.Generator().manual_seed(6))
    ot = oracle.Tree.from_n3tree(tree)
    opt = options(tree, step_size=1e-3)
    o, d, v = rays.origins, rays.dirs, rays.viewdirs

    exact = oracle.volume_render_backward(ot, o, d, v, opt, go, exact_sum=True)
    _, se_exact, hess_exact = oracle.se_grad(ot, o, d, v, ref_colour, opt, exact_sum=True)
    wide = np.zeros(tree.data.shape, dtype=np.float64)
    wide_se = np.zeros_like(wide)
    wide_hess = np.zeros_like(wide)
    for r in range(n):
        sl = slice(r, r + 1)
        one = oracle.volume_render_backward(ot, o[sl], d[sl], v[sl], opt, go[sl], exact_sum=False)
        # one ray: exact and plain modes agree to the bit (nothing to reorder)
        if r < 5:
            assert np.array_equal(one, oracle.volume_render_backward(ot, o[sl], d[sl], v[sl], opt, go[sl], exact_sum=True))
        wide += one
        _, g1, h1 = oracle.se_grad(ot, o[sl], d[sl], v[sl], ref_colour[sl], opt, exact_sum=False)
        wide_se += g1
        wide_hess += h1
    assert np.array_equal(exact, wide.astype(np.float32))
    # (se_grad adds one term per channel to a density entry, rt_kernel.cu:687-702: a single ray already
    # sums three of them in fp32 there, so only the colour entries are term-by-term)
    assert np.array_equal(se_exact[..., :-1], wide_se.astype(np.float32)[..., :-1])
    assert np.array_equal(hess_exact[..., :-1], wide_hess.astype(np.float32)[..., :-1])
    assert np.abs(se_exact[..., -1] - wide_se[..., -1]).max() <= 1e-6 * np.abs(wide_se[..., -1]).max()
    assert np.abs(hess_exact[..., -1] - wide_hess[..., -1]).max() <= 1e-6 * np.abs(wide_hess[..., -1]).max()

    perm = torch.randperm(n, generator=torch.Generator().manual_seed(9))
    shuffled = oracle.volume_render_backward(ot, o[perm].contiguous(), d[perm].contiguous(), v[perm].contiguous(), opt,
                                             go[perm].contiguous(), exact_sum=True, n_threads=4)
    assert np.array_equal(shuffled, exact)
    shuffled_se = oracle.se_grad(ot, o[perm].contiguous(), d[perm].contiguous(), v[perm].contiguous(),
                                 ref_colour[perm].contiguous(), opt, exact_sum=True, n_threads=4)
    assert np.array_equal(shuffled_se[1], se_exact) and np.array_equal(shuffled_se[2], hess_exact)

    plain = oracle.volume_render_backward(ot, o, d, v, opt, go, exact_sum=False)
    assert not np.array_equal(plain, exact)          # fp32 adds in ray order do round differently ...
    assert np.abs(plain - exact).max() <= 1e-5 * np.abs(exact).max()    # ... but only in the last bits
    # the image entry points share the adder
    c2w = synth.orbit_poses(1, seed=2, radius=2.5)[0]
    gi = torch.randn(24, 32, 3, generator=torch.Generator().manual_seed(7))
    a = oracle.volume_render_image_backward(ot, c2w, 30.0, 30.0, 32, 24, opt, gi, exact_sum=True)
    b = oracle.volume_render_image_backward(ot, c2w, 30.0, 30.0, 32, 24, opt, gi, exact_sum=True, n_threads=3)
    assert np.array_equal(a, b)
    plain = oracle.volume_render_image_backward(ot, c2w, 30.0, 30.0, 32, 24, opt, gi, exact_sum=False)
    assert np.abs(a - plain).max() <= 1e-5 * np.abs(a).max()


def test_order_slack_is_what_fp32_sums_in_shuffled_orders_stray_by():
    """The slack the exact-sum mode reports (sqrt(n) * 2^-24 * sum |term| per element) against what it
    models: the same fp32 terms added sequentially in fp32, in several ray orders, on a scene where
    4000 rays pass through a few dozen leaves.  The sums stay within 1.5 slack of the exact sum and
    reach a good part of it, so GPU tests that allow twice the slack allow the reference's own
    nondeterminism and little more."""
    from util import grad_close
    tree, point = synth.deep_tree(14, data_format="RGBA", seed=14)
    g = torch.Generator().manual_seed(14)
    n = 4000
    origins = point[None] + 2.0 * synth.unit_vectors(n, g)
    scale = 2.0 ** -torch.randint(1, 30, (n, 1), generator=g).float()
    dirs = point[None] + (torch.rand(n, 3, generator=g) * 2 - 1) * scale - origins
    dirs = (dirs / dirs.norm(dim=1, keepdim=True)).contiguous()
    origins = origins.contiguous()
    go = torch.randn(n, 3, generator=torch.Generator().manual_seed(1))
    ot = oracle.Tree.from_n3tree(tree)
    opt = options(tree, step_size=1e-4)
    exact, slack = oracle.volume_render_backward(ot, origins, dirs, dirs, opt, go, want_slack=True, n_threads=4)
    nz = slack > 0
    assert nz.sum() > 1000
    worst, relative = [], []
    for seed in range(4):
        perm = torch.randperm(n, generator=torch.Generator().manual_seed(seed))
        plain = oracle.volume_render_backward(ot, origins[perm].contiguous(), dirs[perm].contiguous(),
                                              dirs[perm].contiguous(), opt, go[perm].contiguous(), exact_sum=False)
        worst.append(float((np.abs(plain.astype(np.float64) - exact)[nz] / slack[nz]).max()))
        relative.append(grad_close(plain, exact)[0])
        assert grad_close(plain, exact, slack=slack)[1]
    assert 0.3 < max(worst) < 1.5, worst
    assert max(relative) > 5e-5, relative    # the orders alone use up most of (or more than) a 1e-4 bar here


# ------------------------------------------------------------------------------------------
# camera rays and NDC
# ------------------------------------------------------------------------------------------
def test_image_rays_match_persp_rays_and_convert_to_ndc():
    tree = svox.N3Tree()
    c2w = synth.look_at_pose([2.0, -1.5, 1.2])
    W, H, fx, fy = 37, 23, 40.0, 44.0
    ot = oracle.Tree.from_n3tree(tree)
    o, d, v = oracle.image_rays(ot, c2w, fx, fy, W, H, options(tree))
    want = svox.VolumeRenderer.persp_rays(c2w, W, H, fx, fy)
    assert np.abs(d - want.dirs.numpy()).max() < 1e-6
    assert np.abs(o - want.origins.numpy()).max() < 1e-6
    assert np.array_equal(v, d)
    # NDC: the world ray is mapped as convert_to_ndc does, then normalised; vdir stays the world dir
    c2w = torch.tensor([[1.0, 0, 0, 0.2], [0, 1, 0, -0.1], [0, 0, 1, 0.5]])
    opt = options(tree, ndc=svox.NDCConfig(W, H, fx))
    o, d, v = oracle.image_rays(ot, c2w, fx, fx, W, H, opt)
    base = svox.VolumeRenderer.persp_rays(c2w, W, H, fx, fx)
    from svox_amd.renderer import convert_to_ndc
    no, nd = convert_to_ndc(base.origins.double(), base.dirs.double(), fx, W, H)
    nd = nd / nd.norm(dim=-1, keepdim=True)
    assert np.abs(o - no.numpy()).max() < 1e-5
    assert np.abs(d - nd.numpy()).max() < 1e-5
    assert np.abs(v - base.dirs.numpy()).max() < 1e-6


def test_pathological_rays_terminate():
    """Degenerate rays must end (the reference would loop forever where t cannot advance)."""
    tree = synth.shell_tree(depth=5, n_spheres=4, data_format="SH4", seed=17)
    nan, inf = float("nan"), float("inf")
    o = np.array([[0.5, 0.5, -1.0], [nan, 0.5, 0.5], [1e8, 1e8, 1e8], [0.5, 0.5, 1e30], [0.5, 0.5, -1.0]], np.float32)
    d = np.array([[0.0, 0.0, 0.0], [0.0, 0.0, 1.0], [-1.0, -1.0, -1.0], [0.0, 0.0, -1.0], [0.0, 0.0, inf]], np.float32)
    ot = oracle.Tree.from_n3tree(tree)
    for step in (1e-3, 1e-9, 0.0):
        out, stats = oracle.volume_render(ot, o, d, d, options(tree, step_size=step), want_stats=True)
        assert stats["samples"] < 10000
        grad = oracle.volume_render_backward(ot, o, d, d, options(tree, step_size=step), np.ones((5, 3), np.float32))
        assert grad.shape == tuple(tree.data.shape)


# ------------------------------------------------------------------------------------------
# squared-error gradient and Gauss-Newton Hessian diagonal (se_grad)
# ------------------------------------------------------------------------------------------
def _se_case(fmt, dtype=torch.float64, n_rays=24, seed=11):
    tree = svox.N3Tree(data_format=fmt, init_refine=1, dtype=dtype)
    g = torch.Generator().manual_seed(seed)
    tree.data.data.normal_(generator=g)
    tree.data.data[..., -1] = tree.data.data[..., -1].abs() * 3
    tree.data.data[0, 0, 0, 1, -1] = 0.0            # an empty leaf among the others
    rays = synth.sphere_rays(n_rays, seed=seed, dtype=dtype)
    ref = torch.rand(n_rays, 3, generator=g, dtype=dtype)
    return tree, rays, ref


@pytest.mark.parametrize("fmt,basis", [("RGBA", -1), ("SH4", 4)])
def test_se_grad_is_the_gradient_and_jacobian_row_norm_of_the_squared_error(fmt, basis):
    """colour = render; grad = d/d(data) of 0.5 |render - ref|^2; hessdiag = sum over rays and channels
    of (d render_c / d data)^2 -- both from torch.autograd through the fallback restatement."""
    tree, rays, ref = _se_case(fmt)
    opt = options(tree, step_size=1e-3)
    ot = oracle.Tree.from_n3tree(tree)
    colour, grad, hess = oracle.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt)

    data = tree.data.detach().clone().requires_grad_(True)
    out = torch_fallback.render(data, tree.child, tree.parent_depth, tree.invradius, tree.offset, rays.origins,
                                rays.dirs, rays.viewdirs, basis)
    assert np.abs(colour - out.detach().numpy()).max() < 2e-6
    assert np.abs(colour - oracle.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, opt)).max() < 1e-6
    (want_grad,) = torch.autograd.grad(0.5 * ((out - ref) ** 2).sum(), data, retain_graph=True)
    want_hess = torch.zeros_like(data)
    for r in range(out.shape[0]):
        for c in range(3):
            (row,) = torch.autograd.grad(out[r, c], data, retain_graph=True)
            want_hess += row ** 2
    assert np.abs(grad - want_grad.numpy()).max() <= 1e-4 * np.abs(want_grad.numpy()).max()
    assert np.abs(hess - want_hess.numpy()).max() <= 1e-4 * np.abs(want_hess.numpy()).max()
    assert (hess >= 0).all() and hess[..., -1].max() > 0 and hess[..., 0].max() > 0


def test_se_grad_agrees_with_the_backward_march_on_the_residual():
    for fmt in ("RGBA", "SH9"):
        tree = synth.dense_tree(2, fmt, seed=21, sigma="lognormal", coeff_std=0.7)
        rays = synth.sphere_rays(500, seed=8)
        ref = torch.rand(500, 3, generator=torch.Generator().manual_seed(2))
        ot = oracle.Tree.from_n3tree(tree)
        opt = options(tree, step_size=1e-3, rgb_padding=0.02, background_brightness=0.7)
        colour, grad, hess = oracle.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt)
        want = oracle.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, colour - ref.numpy())
        assert np.abs(grad - want).max() <= 2e-5 * np.abs(want).max()
        # thresholds play no part (rt_kernel.cu:536, 584, 651 test sigma > 0 only)
        again = oracle.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, options(
            tree, step_size=1e-3, rgb_padding=0.02, background_brightness=0.7, fast=True))
        assert all(np.array_equal(a, b) for a, b in zip((colour, grad, hess), again))
        # rays that miss: background colour, no gradient (rt_kernel.cu:504-510)
        c_miss, g_miss, h_miss = oracle.se_grad(ot, rays.origins, -rays.dirs, rays.viewdirs, ref, opt)
        assert np.all(c_miss == np.float32(0.7)) and not g_miss.any() and not h_miss.any()


def test_se_grad_softplus_terms_follow_from_the_plain_ones():
    """With density_softplus the density entries are the plain ones (on a tree that stores
    softplus(raw) directly) times sigmoid(raw - 1), and the Hessian entry gains
    sigmoid' * sum_c d(render_c)/d(sigma), which the backward march with grad_out = 1 gives
    (rt_kernel.cu:683-695)."""
    tree, rays, ref = _se_case("SH4", seed=13)
    raw = tree.data.data[..., -1].clone()
    soft = torch.log1p(torch.exp(raw - 1))
    plain = svox.N3Tree(data_format="SH4", init_refine=1, dtype=torch.float64)
    plain.data.data.copy_(tree.data.data)
    # what the march sees as sigma: logf(1 + expf(raw - 1)) evaluated in single precision
    seen = np.log((1 + oracle.expf((raw - 1).numpy().astype(np.float32))).astype(np.float32)).astype(np.float64)
    assert np.abs(seen - soft.numpy()).max() < 1e-6
    plain.data.data[..., -1] = torch.from_numpy(seen)
    o, d, v = rays.origins, rays.dirs, rays.viewdirs
    c_s, g_s, h_s = oracle.se_grad(oracle.Tree.from_n3tree(tree), o, d, v, ref, options(tree, density_softplus=True))
    c_p, g_p, h_p = oracle.se_grad(oracle.Tree.from_n3tree(plain), o, d, v, ref, options(plain))
    ones = oracle.volume_render_backward(oracle.Tree.from_n3tree(plain), o, d, v, options(plain),
                                         np.ones((o.shape[0], 3)))
    # (numpy's float32 log and the C library's logf may differ in the last place)
    assert np.allclose(c_s, c_p, rtol=0, atol=1e-6)
    assert np.allclose(g_s[..., :-1], g_p[..., :-1], rtol=1e-5, atol=1e-8)
    sg = 1 / (1 + np.exp(-(raw.numpy() - 1)))
    live = seen > 0
    assert np.allclose(g_s[..., -1][live], (g_p[..., -1] * sg)[live], rtol=1e-5, atol=1e-9)
    want_h = h_p[..., -1] * sg * sg + ones[..., -1] * sg * (1 - sg)
    assert np.allclose(h_s[..., -1][live], want_h[live], rtol=1e-5, atol=1e-9)


def test_se_grad_image_is_se_grad_on_the_image_rays():
    tree = synth.dense_tree(2, "SH4", seed=5)
    c2w = synth.look_at_pose(torch.tensor([0.5, 0.5, 0.5]) + 2.5 * torch.tensor([0.3, -0.5, 0.8]))
    ot = oracle.Tree.from_n3tree(tree)
    opt = options(tree, step_size=1e-3)
    W, H, fx = 20, 14, 25.0
    ref = torch.rand(H, W, 3, generator=torch.Generator().manual_seed(4))
    colour, grad, hess = oracle.se_grad_image(ot, c2w, fx, fx, W, H, ref, opt)
    o, d, v = oracle.image_rays(ot, c2w, fx, fx, W, H, opt)
    # image_rays returns tree-space origins; this tree's transform is the identity
    c2, g2, h2 = oracle.se_grad(ot, o, d, v, ref.reshape(-1, 3), opt)
    assert np.array_equal(colour.reshape(-1, 3), c2) and np.array_equal(grad, g2) and np.array_equal(hess, h2)


# ------------------------------------------------------------------------------------------
# dense-grid weight render (grid_weight_render)
# ------------------------------------------------------------------------------------------
def test_grid_weight_render_axis_aligned_closed_form():
    """One pixel looking straight down -z through a uniform grid: 8 cells, step lengths
    1/8 + step, 1/8, 1/8, ...; weights are the compositing weights; one hit per cell."""
    reso, s, step = 8, 3.0, 1e-3
    data = np.full((reso, reso, reso), s, np.float32)
    c2w = torch.tensor([[1.0, 0, 0, 0.3], [0, 1, 0, 0.6], [0, 0, 1, 2.0]])
    tree = svox.N3Tree(data_format="RGBA")
    opt = options(tree, step_size=step)
    weight, hit = oracle.grid_weight_render(data, c2w, 1e9, 1e9, 1, 1, opt, np.zeros(3), np.ones(3))
    want_hit = np.zeros_like(data)
    want_hit[2, 4, :] = 1
    assert np.array_equal(hit, want_hit)
    first = np.exp(-s * (1 / reso + step))
    later = np.exp(-s / reso)
    want = np.array([1 - first] + [first * later ** (k - 1) * (1 - later) for k in range(1, reso)])
    assert np.abs(weight[2, 4, ::-1] - want).max() < 1e-5
    assert weight.sum() == weight[2, 4].sum()
    # a threshold above the density: nothing is recorded
    weight, hit = oracle.grid_weight_render(data, c2w, 1e9, 1e9, 1, 1, options(tree, step_size=step, sigma_thresh=5.0),
                                            np.zeros(3), np.ones(3))
    assert not weight.any() and not hit.any()


def test_grid_weight_render_equals_max_accumulation_on_the_dense_tree():
    """A dense 16^3 tree is the same volume as its 16^3 grid of leaf densities: the tree march with a
    max-accumulator gives, leaf by leaf, what the grid march gives cell by cell."""
    tree = svox.N3Tree(data_format="RGBA", init_refine=3, radius=0.7, center=[0.4, 0.5, 0.6])
    g = torch.Generator().manual_seed(3)
    tree.data.data.normal_(generator=g)
    tree.data.data[..., -1] = (tree.data.data[..., -1] * 4).clamp_min(0)     # about half the cells empty
    reso = 16
    ax = (torch.arange(reso) + 0.5) / reso
    centres = torch.stack(torch.meshgrid(ax, ax, ax, indexing="ij"), -1).reshape(-1, 3)
    ot = oracle.Tree.from_n3tree(tree, world=False)
    values, ids = oracle.query_vertical(ot, centres)
    sigma_grid = values[:, -1].reshape(reso, reso, reso)
    c2w = synth.look_at_pose(torch.tensor([0.4, 0.5, 0.6]) + 2.0 * torch.tensor([0.5, 0.3, 0.8]),
                             target=torch.tensor([0.4, 0.5, 0.6]))
    opt = options(tree, step_size=1e-3, sigma_thresh=0.5)
    W, H, fx = 40, 30, 30.0
    weight, hit = oracle.grid_weight_render(sigma_grid, c2w, fx, fx, W, H, opt, tree.offset, tree.invradius)
    ow = oracle.Tree.from_n3tree(tree)
    ow.weight_accum = np.zeros(tree.child.shape, np.float32)
    ow.weight_accum_max = True
    _, stats = oracle.volume_render_image(ow, c2w, fx, fx, W, H, opt, want_stats=True)
    assert stats["samples_shaded"] > 1000
    assert np.array_equal(weight.reshape(-1), ow.weight_accum.reshape(-1)[ids])
    assert hit.sum() == stats["samples_shaded"]
    assert not hit[sigma_grid <= 0.5].any() and not weight[sigma_grid <= 0.5].any()


def test_weight_accumulation_sums_to_the_opacity_of_the_rays():
    """Colours all sigmoid(0) = 0.5 and a white background: out = 0.5 * sum(w) + (1 - sum(w)), so the
    accumulator's total must be sum over rays of 2 - 2 * out (rt_kernel.cu:298-304)."""
    tree = synth.dense_tree(3, "RGBA", seed=2)
    tree.data.data[..., :-1] = 0.0
    rays = synth.sphere_rays(300, seed=12)
    ot = oracle.Tree.from_n3tree(tree)
    ot.weight_accum = np.zeros(tree.child.shape, np.float32)
    out = oracle.volume_render(ot, rays.origins, rays.dirs, rays.viewdirs, options(tree, background_brightness=1.0))
    assert abs(ot.weight_accum.sum(dtype=np.float64) - (2 - 2 * out[:, 0].astype(np.float64)).sum()) < 2e-3
    assert not ot.weight_accum[tree.child.numpy() != 0].any()      # only leaves receive weight
