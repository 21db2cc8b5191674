"""Seeded synthetic trees, rays and cameras for tests and benchmarks.

All generators take a torch.Generator-style integer seed and build on the CPU by default so that
the same bits can be handed to the GPU library and to a CPU checker.
"""
import math

import torch

from .formats import Rays
from .tree import N3Tree


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    return g


def unit_vectors(n, gen):
    v = torch.randn(n, 3, generator=gen)
    return v / v.norm(dim=-1, keepdim=True)


def sphere_rays(n, seed=0, radius=2.0, dtype=torch.float32):
    """Origins on a sphere of `radius` around the cube centre, aimed at uniform points in the cube."""
    g = _gen(seed)
    origins = 0.5 + radius * unit_vectors(n, g)
    targets = torch.rand(n, 3, generator=g)
    dirs = targets - origins
    dirs = dirs / dirs.norm(dim=-1, keepdim=True)
    origins, dirs = origins.to(dtype).contiguous(), dirs.to(dtype).contiguous()
    return Rays(origins=origins, dirs=dirs, viewdirs=dirs.clone())


def look_at_pose(position, target=(0.5, 0.5, 0.5), up=(0.0, 0.0, 1.0)):
    """(3, 4) camera-to-world matrix, OpenGL convention: columns right, up, back, position."""
    pos = torch.as_tensor(position, dtype=torch.float64)
    back = pos - torch.as_tensor(target, dtype=torch.float64)
    back = back / back.norm()
    upv = torch.as_tensor(up, dtype=torch.float64)
    right = torch.linalg.cross(upv, back)
    if right.norm() < 1e-6:
        right = torch.linalg.cross(torch.tensor([0.0, 1.0, 0.0], dtype=torch.float64), back)
    right = right / right.norm()
    true_up = torch.linalg.cross(back, right)
    return torch.stack([right, true_up, back, pos], dim=1).float()


def orbit_poses(n, seed=0, radius=4.0):
    g = _gen(seed)
    return [look_at_pose(0.5 + radius * u) for u in unit_vectors(n, g)]


def dense_tree(levels, data_format="RGBA", seed=0, device="cpu", zero_fraction=0.0, sigma="relu_normal",
               coeff_std=1.0, dtype=torch.float32):
    """Uniformly refined tree with a (2^(levels+1))^3 leaf grid and random leaf records.

    sigma: "relu_normal" -> relu(N(0, 10)); "lognormal" -> exp(N(0, 1)).
    RGBA colours ~ U(0, 1); SH coefficients ~ N(0, coeff_std).  A Bernoulli(zero_fraction) mask zeroes
    whole leaf records.
    """
    g = _gen(seed)
    tree = N3Tree(N=2, data_format=data_format, init_refine=levels, device="cpu", dtype=dtype)
    shape = tree.data.shape
    if tree.data_format.format == 0:
        vals = torch.rand(shape, generator=g)
    else:
        vals = torch.randn(shape, generator=g) * coeff_std
    if sigma == "relu_normal":
        sg = torch.relu(torch.randn(shape[:-1], generator=g) * 10.0)
    else:
        sg = torch.exp(torch.randn(shape[:-1], generator=g))
    vals[..., -1] = sg
    if zero_fraction > 0:
        keep = torch.rand(shape[:-1], generator=g) >= zero_fraction
        vals = vals * keep[..., None]
    tree.data.data[:] = vals.to(dtype)
    return tree.to(device) if str(device) != "cpu" else tree


def deep_tree(levels, data_format="SH4", seed=0, base_refine=2, dtype=torch.float32):
    """Octree that is `levels` levels deep along one root-to-leaf chain: a dense 2^base_refine grid
    whose leaf at a seeded point is split again and again.  Returns (tree, point): the point lies in
    the deepest leaf.  Densities are positive everywhere, growing towards the deep end, so that rays
    through the point shade leaves of every size."""
    g = _gen(seed)
    tree = N3Tree(N=2, data_format=data_format, init_refine=base_refine, depth_limit=levels + 2, dtype=dtype)
    point = 0.2 + 0.6 * torch.rand(3, generator=g, dtype=torch.float64)
    while True:
        child = tree.child
        node, q, depth = 0, point.clone(), 0
        while True:
            q = q * 2
            idx = q.floor().long()
            q = q - idx
            depth += 1
            skip = int(child[node, idx[0], idx[1], idx[2]])
            if skip == 0:
                break
            node += skip
        if depth >= levels:
            break
        tree.refine(sel=(torch.tensor([node]), idx[0:1], idx[1:2], idx[2:3]))
    shape = tree.data.shape
    vals = torch.randn(shape, generator=g) * 0.5
    node_depth = tree.parent_depth[:, 1].to(torch.float32)
    sigma = (0.5 + torch.rand(shape[:-1], generator=g)) * (2.0 + node_depth)[:, None, None, None]
    vals[..., -1] = sigma
    tree.data.data[:] = vals.to(dtype)
    return tree, point.to(dtype)


def _sdf_spheres(p, centers, radii):
    """Distance to the surface of the union of spheres (exact outside, a lower bound inside)."""
    d = (p[:, None, :] - centers[None]).norm(dim=-1) - radii[None]
    return d.min(dim=1).values


def _sphere_geometry(gen, n_spheres, shell, dev):
    centers = (0.2 + 0.6 * torch.rand(n_spheres, 3, generator=gen)).to(dev)
    radii = (0.05 + 0.15 * torch.rand(n_spheres, generator=gen)).to(dev)

    def may_touch(cen, size):
        return _sdf_spheres(cen, centers, radii).abs() <= (math.sqrt(3.0) / 2.0) * size + shell

    def occupied(cen):
        return _sdf_spheres(cen, centers, radii).abs() <= shell

    return may_touch, occupied


def _noise_geometry(gen, dev, threshold=0.80, lattice=17, slab_z=0.25, slab_half=0.004):
    """Blobs where seeded trilinear value noise exceeds `threshold`, plus a thin slab z ~ slab_z."""
    R = lattice
    grid = torch.rand(R, R, R, generator=gen).to(dev)

    def noise(p):
        q = p.clamp(0, 1) * (R - 1)
        i0 = q.floor().clamp(max=R - 2).long()
        fx, fy, fz = (q - i0).unbind(-1)
        x0, y0, z0 = i0.unbind(-1)

        def c(a, b, e):
            return grid[x0 + a, y0 + b, z0 + e]

        lo = (c(0, 0, 0) * (1 - fx) + c(1, 0, 0) * fx) * (1 - fy) + (c(0, 1, 0) * (1 - fx) + c(1, 1, 0) * fx) * fy
        hi = (c(0, 0, 1) * (1 - fx) + c(1, 0, 1) * fx) * (1 - fy) + (c(0, 1, 1) * (1 - fx) + c(1, 1, 1) * fx) * fy
        return lo * (1 - fz) + hi * fz

    def may_touch(cen, size):
        # the interpolant is multilinear inside a lattice cell, so over a tree cell that lies inside
        # one (size <= 1/(R-1), aligned because R-1 is a power of two) its maximum is at a corner
        blob = size > 1.0 / (R - 1) - 1e-9
        half = 0.5 * size[:, None]
        for dx in (-1.0, 1.0):
            for dy in (-1.0, 1.0):
                for dz in (-1.0, 1.0):
                    corner = cen + half * torch.tensor([dx, dy, dz], device=cen.device)
                    blob = blob | (noise(corner) > threshold)
        slab = (cen[:, 2] - slab_z).abs() <= slab_half + 0.5 * size
        return blob | slab

    def occupied(cen):
        return (noise(cen) > threshold) | ((cen[:, 2] - slab_z).abs() <= slab_half)

    return may_touch, occupied


def shell_tree(depth=9, n_spheres=24, data_format="SH16", seed=0, device="cpu", shell_voxels=2.0,
               coeff_std=0.3, sigma_range=(20.0, 200.0), geometry="spheres", chunk=1 << 20,
               noise_threshold=0.80):
    """Sparse octree refined down to a 2^depth grid only where the geometry is; finest-level leaves
    inside the geometry get sigma ~ U(sigma_range), every other leaf sigma 0; colour coefficients
    ~ N(0, coeff_std).

    geometry "spheres": shell of `shell_voxels` finest voxels around the surface of a union of seeded
                        spheres (centres U(.2,.8)^3, radii U(.05,.2)).
    geometry "noise":   blobs where seeded value noise exceeds `noise_threshold`, plus a thin slab
                        (a forward-facing scene).
    Built on `device` with torch ops: refine() level by level on the cells that may touch the
    geometry (conservative test on the cell centre and size).
    """
    g = _gen(seed)
    dev = torch.device(device)
    voxel = 2.0 ** (-depth)
    if geometry == "spheres":
        may_touch, occupied_fn = _sphere_geometry(g, n_spheres, shell_voxels * voxel, dev)
    else:
        may_touch, occupied_fn = _noise_geometry(g, dev, threshold=noise_threshold)

    tree = N3Tree(N=2, data_format=data_format, depth_limit=depth - 1, device=device)
    for level in range(1, depth):
        leaves = tree._all_leaves().to(dev)
        corners = _leaf_corners(tree, leaves)
        size = 2.0 ** (-(tree.parent_depth[leaves[:, 0], 1].float() + 1.0))
        pick = torch.zeros(leaves.shape[0], dtype=torch.bool, device=dev)
        for s in range(0, leaves.shape[0], chunk):
            cen = corners[s:s + chunk] + 0.5 * size[s:s + chunk, None]
            pick[s:s + chunk] = may_touch(cen, size[s:s + chunk])
        sel = tuple(leaves[pick].T)
        if sel[0].numel() == 0:
            break
        tree.refine(sel=sel)
    # leaf records
    gd = torch.Generator(device=dev)
    gd.manual_seed(int(seed) + 1)
    n_int = tree.n_internal
    data = torch.randn(tree.data.shape, generator=gd, device=dev) * coeff_std
    leaves = tree._all_leaves().to(dev)
    corners = _leaf_corners(tree, leaves)
    depth_of = tree.parent_depth[leaves[:, 0], 1]
    size = 2.0 ** (-(depth_of.float() + 1.0))
    occupied = torch.zeros(leaves.shape[0], dtype=torch.bool, device=dev)
    for s in range(0, leaves.shape[0], chunk):
        cen = corners[s:s + chunk] + 0.5 * size[s:s + chunk, None]
        occupied[s:s + chunk] = occupied_fn(cen) & (depth_of[s:s + chunk] == depth - 1)
    sig = torch.zeros(tree.child.shape, dtype=torch.float32, device=dev)
    lo, hi = sigma_range
    vals = lo + (hi - lo) * torch.rand(int(occupied.sum().item()), generator=gd, device=dev)
    occ = leaves[occupied]
    sig[occ[:, 0], occ[:, 1], occ[:, 2], occ[:, 3]] = vals
    data[..., -1] = sig
    data[n_int:] = 0
    tree.data.data[:] = data
    tree.info = {"leaves": int(leaves.shape[0]), "occupied_leaves": int(occupied.sum().item()),
                 "nodes": int(n_int), "occupancy": float(occupied.sum().item()) * voxel ** 3}
    return tree


def _leaf_corners(tree, leaves):
    """Lower corners (tree coordinates) of leaf cells [node, x, y, z] with plain torch ops:
    the cell index at level l contributes cell / N^l; levels are walked from the leaf to the root."""
    N = tree.N
    cur = leaves[:, 0].clone()
    acc = leaves[:, 1:].to(torch.float64)
    level = tree.parent_depth[cur, 1].long() + 1
    corner = torch.zeros(leaves.shape[0], 3, dtype=torch.float64, device=leaves.device)
    while bool((level > 0).any()):
        w = torch.where(level > 0, float(N) ** (-level.double()), torch.zeros_like(level, dtype=torch.float64))
        corner = corner + acc * w[:, None]
        par = tree._unpack_index(tree.parent_depth[cur, 0].long())
        acc = par[:, 1:].to(torch.float64)
        cur = par[:, 0]
        level = level - 1
    return corner.float()
