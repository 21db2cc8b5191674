"""N3Tree: the sparse voxel N^3-tree container (octree for N = 2).

API and tensor layout follow the reference's `svox.N3Tree` (svox/svox.py:57-1103) so that code
written against it runs unchanged; every operation that the reference hands to its CUDA extension
goes to the HIP library through `svox_amd.csrc`.  The pure-PyTorch fallbacks of the reference are
not part of this package: a tree whose tensors are not on a GPU can be built, refined, indexed by
leaf number and saved, but point queries and rendering raise.

Tensor layout (the contract the kernels consume):
  data          (M, N, N, N, K) float   every cell of every node holds K numbers; sigma is last
  child         (M, N, N, N)   int32    offset from this node to the child node, 0 = leaf cell
  parent_depth  (M, 2)         int32    [packed index of the parent cell, depth of the node]
  invradius, offset (3,)       float    tree = offset + world * invradius
Nodes are appended in refinement order, so a child always has a larger index than its parent.
"""
import math
import os.path as osp
from warnings import warn

import numpy as np
import torch
from torch import nn

from . import csrc as _C
from .formats import DataFormat, LocalIndex  # noqa: F401
from .view import N3TreeView


class _QueryVerticalFunction(torch.autograd.Function):
    """values, node_ids = query(data, spec, points); gradient flows to `data` only
    (svox/svox.py:38-54)."""

    @staticmethod
    def forward(ctx, data, tree_spec, indices):
        values, node_ids = _C.query_vertical(tree_spec, indices)
        ctx.mark_non_differentiable(node_ids)
        ctx.tree_spec = tree_spec
        ctx.save_for_backward(indices)
        return values, node_ids

    @staticmethod
    def backward(ctx, grad_values, _grad_ids):
        if not ctx.needs_input_grad[0]:
            return None, None, None
        (indices,) = ctx.saved_tensors
        grad = _C.query_vertical_backward(ctx.tree_spec, indices, grad_values.contiguous())
        return grad, None, None


def _no_fallback(what):
    raise RuntimeError(
        f"{what}: this build has only the HIP path (tensors must live on a GPU and cuda=True); "
        "the reference's PyTorch fallback is not included")


class N3Tree(nn.Module):
    """PyTorch N^3-tree with HIP acceleration on MI355X.

    `data` is an nn.Parameter whose size changes on refine / expand / shrink_to_fit; optimisers
    built before such a call must be re-made (a call that resized returns True).
    """

    def __init__(self, N=2, data_dim=None, depth_limit=10, init_reserve=1, init_refine=0,
                 geom_resize_fact=1.0, radius=0.5, center=(0.5, 0.5, 0.5), data_format="RGBA",
                 extra_data=None, device="cpu", dtype=torch.float32, map_location=None):
        super().__init__()
        assert N >= 2
        assert depth_limit >= 0
        if map_location is not None:
            warn("map_location has been renamed to device and may be removed")
            device = map_location
        assert dtype in (torch.float32, torch.float64), "Unsupported dtype"
        self.N = int(N)
        self.data_format = DataFormat(data_format) if data_format is not None else None
        self.data_dim = data_dim
        self._maybe_auto_data_dim()

        # a uniform tree refined r times has 1 + N^3 + ... + N^(3r) nodes (svox/svox.py:118-120)
        reserve = int(init_reserve) + sum((self.N ** i) ** 3 for i in range(1, init_refine + 1))
        N_ = self.N
        self.register_parameter("data", nn.Parameter(
            torch.zeros(reserve, N_, N_, N_, self.data_dim, dtype=dtype, device=device)))
        self.register_buffer("child", torch.zeros(reserve, N_, N_, N_, dtype=torch.int32, device=device))
        self.register_buffer("parent_depth", torch.zeros(reserve, 2, dtype=torch.int32, device=device))
        self.register_buffer("_n_internal", torch.tensor(1, device=device))
        self.register_buffer("_n_free", torch.tensor(0, device=device))

        if isinstance(radius, (int, float)):
            radius = [radius] * 3
        radius_t = torch.tensor(radius, dtype=dtype, device=device)
        center_t = torch.tensor(list(center), dtype=dtype, device=device)
        self.register_buffer("invradius", 0.5 / radius_t)
        self.register_buffer("offset", 0.5 * (1.0 - center_t / radius_t))

        self.depth_limit = depth_limit
        self.geom_resize_fact = geom_resize_fact
        if extra_data is not None:
            assert isinstance(extra_data, torch.Tensor)
            self.register_buffer("extra_data", extra_data.to(dtype=dtype, device=device))
        else:
            self.extra_data = None

        self._ver = 0
        self._invalidate()
        self._lock_tree_structure = False
        self._weight_accum = None
        self._weight_accum_op = None
        self.refine(repeats=init_refine)

    # ------------------------------------------------------------------ point access
    def set(self, indices, values, cuda=True):
        """Write `values` (Q, K') into the leaves containing the world points `indices` (Q, 3).
        Two points in the same leaf race (svox/svox.py:158-206, svox_kernel.cu:80-89)."""
        assert len(indices.shape) == 2
        assert not indices.requires_grad
        assert not values.requires_grad
        indices = indices.to(device=self.data.device)
        values = values.to(device=self.data.device)
        if not cuda or not self.data.is_cuda:
            _no_fallback("N3Tree.set")
        _C.assign_vertical(self._spec(), indices.contiguous(), values.contiguous())
        self.touch()   # a write torch's version counter of `data` has not seen

    def forward(self, indices, cuda=True, want_node_ids=False, world=True):
        """Leaf values at the points `indices` (Q, 3); differentiable w.r.t. `data`.

        :param want_node_ids: also return the packed leaf id node*N^3 + x*N^2 + y*N + z (int64)
        :param world: points are world coordinates (else tree-local [0, 1]^3)
        :return: (Q, data_dim)[, (Q,)]     (svox/svox.py:208-272)
        """
        assert not indices.requires_grad
        assert len(indices.shape) == 2
        if not cuda or not self.data.is_cuda:
            _no_fallback("N3Tree.forward")
        values, node_ids = _QueryVerticalFunction.apply(self.data, self._spec(world), indices.contiguous())
        return (values, node_ids) if want_node_ids else values

    def snap(self, indices):
        """Lower corner of the leaf containing each point (B, 3)."""
        return self[indices].corners

    # ------------------------------------------------------------------ copies / reshaping
    def partial(self, data_sel=None, data_format=None, dtype=None, device=None):
        """A copy of the tree keeping only the channels `data_sel` (svox/svox.py:286-334)."""
        device = self.data.device if device is None else device
        dtype = self.data.dtype if dtype is None else dtype
        if data_sel is None:
            channels, new_dim = None, self.data_dim
        else:
            channels = torch.arange(self.data_dim)[data_sel].reshape(-1)
            new_dim = channels.numel()
        other = N3Tree(N=self.N, data_dim=new_dim, data_format=data_format or str(self.data_format),
                       depth_limit=self.depth_limit, geom_resize_fact=self.geom_resize_fact,
                       dtype=dtype, device=device)

        def dup(x, dt=None):
            return x.detach().to(device=device, dtype=dt or x.dtype, copy=True)

        other.invradius = dup(self.invradius, dtype)
        other.offset = dup(self.offset, dtype)
        other.child = dup(self.child)
        other.parent_depth = dup(self.parent_depth)
        other._n_internal = dup(self._n_internal)
        other._n_free = dup(self._n_free)
        other.extra_data = dup(self.extra_data, dtype) if self.extra_data is not None else None
        if data_format is None:
            other.data_format = self.data_format
        src = self.data.data if channels is None else self.data.data[..., channels.to(self.data.device)]
        other.data = nn.Parameter(dup(src.contiguous(), dtype))
        other._invalidate()
        return other

    def clone(self, device=None):
        return self.partial(device=device)

    def expand(self, data_format, data_dim=None, remap=None):
        """Change the per-leaf record (e.g. "SH1" -> "SH4").  By default coefficient i of channel c
        moves to slot c*new_basis + i and sigma stays last (svox/svox.py:336-400)."""
        assert isinstance(data_format, str), "Please specify valid data format"
        old_format, old_dim = self.data_format, self.data_dim
        self.data_format = DataFormat(data_format)
        self.data_dim = data_dim
        self._maybe_auto_data_dim()
        shrinking = self.data_dim < old_dim
        small_dim, big_dim = (self.data_dim, old_dim) if shrinking else (old_dim, self.data_dim)
        if remap is None:
            sigma = torch.tensor([big_dim - 1])
            if old_format is None or self.data_format.format == DataFormat.RGBA:
                remap = torch.cat([torch.arange(small_dim - 1), sigma])
            else:
                assert self.data_format.basis_dim >= 1, "Please manually specify data_dim for expand()"
                old_basis = old_format.basis_dim if old_format.basis_dim >= 0 else 1
                new_basis = self.data_format.basis_dim
                small_basis, big_basis = (new_basis, old_basis) if shrinking else (old_basis, new_basis)
                arr = torch.arange(small_basis)
                remap = torch.cat([arr, big_basis + arr, 2 * big_basis + arr, sigma])
        remap = torch.as_tensor(remap).to(self.data.device)
        old = self.data.data
        if shrinking:
            new = old[..., remap].contiguous()
        else:
            new = torch.zeros((*old.shape[:-1], self.data_dim), dtype=old.dtype, device=old.device)
            new[..., remap] = old
        self.data = nn.Parameter(new)
        self._invalidate()

    def shrink(self, data_format, data_dim=None, remap=None):
        self.expand(data_format, data_dim, remap)

    # ------------------------------------------------------------------ frontier (nodes whose cells are all leaves)
    @property
    def _frontier(self):
        """Indices of the live nodes all of whose cells are leaves (svox/svox.py:621-633)."""
        if self._last_frontier is None:
            n_int = self.n_internal
            all_leaves = (self.child[:n_int] == 0).reshape(n_int, -1).all(dim=1)
            live = self.parent_depth[:n_int, 0] != -1
            self._last_frontier = (all_leaves & live).nonzero(as_tuple=False).reshape(-1)
        return self._last_frontier

    @property
    def n_frontier(self):
        return self._frontier.shape[0]

    @property
    def frontier_depth(self):
        """Depth of every frontier node, (n_frontier,)."""
        return self.parent_depth[self._frontier, 1]

    def reduce_frontier(self, op=torch.mean, dim=None, grad=False):
        """Apply `op(x, dim=1)` to the (n_frontier, N^3, data_dim) block of child-leaf records of the
        frontier nodes; `dim` selects data channels first; `grad` keeps the result differentiable
        with respect to `data` (svox/svox.py:491-530)."""
        source = self.data if grad else self.data.data
        block = source[self._frontier].view(-1, self.N ** 3, self.data_dim)
        if dim is not None:
            block = block[..., dim]
        return op(block, dim=1)

    def max_frontier(self, dim=None, grad=False):
        """reduce_frontier with the maximum over the children (svox/svox.py:532-548)."""
        return self.reduce_frontier(op=lambda x, dim: torch.max(x, dim=dim)[0], dim=dim, grad=grad)

    def diam_frontier(self, dim=None, grad=False, scale=1.0):
        """Largest distance between the records of any two children of each frontier node
        (svox/svox.py:550-580)."""
        def diameter(x, dim):
            if x.ndim == 2:
                x = x[:, :, None]
            pairwise = torch.cdist(x * scale, x * scale)          # (B, N^3, N^3)
            return pairwise.reshape(x.shape[0], -1).max(dim=1)[0]
        return self.reduce_frontier(op=diameter, dim=dim, grad=grad)

    def merge(self, frontier_sel=None, op=torch.mean):
        """Collapse the selected frontier nodes (default all) into leaves of their parents: the
        parent cell takes `op` over the N^3 child records (the first result if `op` returns a
        tuple, as torch.max does), the node is marked free (child and parent link -1) and
        shrink_to_fit() reclaims it later.  Returns False if nothing was selected
        (svox/svox.py:436-475)."""
        if self._lock_tree_structure:
            raise RuntimeError("Tree locked")
        if self.n_internal - int(self._n_free.item()) <= 1:
            raise RuntimeError("Cannot merge root node")
        nodes = self._frontier if frontier_sel is None else self._frontier[frontier_sel]
        nodes = nodes.reshape(-1)
        nodes = nodes[nodes != 0]           # the root has no parent cell to fall back into
        if nodes.numel() == 0:
            return False
        with torch.no_grad():
            merged = op(self.data.data[nodes].view(-1, self.N ** 3, self.data_dim), dim=1)
            if isinstance(merged, tuple):
                merged = merged[0]
            parent_cells = tuple(self._unpack_index(self.parent_depth[nodes, 0].long()).T)
            self.data.data[parent_cells] = merged
            self.child[parent_cells] = 0
            self.parent_depth[nodes] = -1
            self.child[nodes] = -1
            self._n_free += nodes.shape[0]
        self._invalidate()
        return True

    # ------------------------------------------------------------------ dense grids
    @classmethod
    def from_grid(cls, grid, *args, **kwargs):
        """Tree with the resolution of the (D, D, D, data_dim) grid `grid`, D a power of two, holding
        the grid's values (svox/svox.py:868-883).  The tree must live on a GPU (`device=`)."""
        D = grid.shape[0]
        assert grid.ndim == 4 and grid.shape[1] == D and grid.shape[2] == D, \
            "Grid must be a 4D array with first 3 dims equal"
        log_d = int(math.log2(D))
        assert 2 ** log_d == D, "Grid size must be power of 2"
        kwargs["init_refine"] = log_d - 1
        kwargs.setdefault("data_dim", grid.shape[-1])
        tree = cls(*args, **kwargs)
        tree.set_grid(grid)
        return tree

    def set_grid(self, grid):
        """Write grid[i, j, k] into the leaf at the centre of grid cell (i, j, k)
        (svox/svox.py:885-897)."""
        D = grid.shape[0]
        assert grid.ndim == 4 and grid.shape[1] == D and grid.shape[2] == D and grid.shape[-1] == self.data_dim
        centres = gen_grid(D).reshape(-1, 3).to(device=self.data.device, dtype=self.data.dtype)
        self[LocalIndex(centres)] = grid.reshape(-1, self.data_dim).to(device=self.data.device, dtype=self.data.dtype)

    # ------------------------------------------------------------------ structure
    def refine(self, repeats=1, sel=None):
        """Split every selected leaf into N^3 children (respecting depth_limit).

        :param sel: optional (node, x, y, z) index tuple of leaves; default all leaves
        :return: True iff `data` was re-allocated   (svox/svox.py:636-705)

        New nodes take indices n_internal, n_internal+1, ... in the order of the selection (all
        leaves: lexicographic (node, x, y, z)); their cells start as copies of the split leaf's
        record, which itself stays in place.
        """
        if self._lock_tree_structure:
            raise RuntimeError("Tree locked")
        resized = False
        N = self.N
        with torch.no_grad():
            for rep in range(repeats):
                first_new = self.n_internal
                if sel is None:
                    sel = tuple(self._all_leaves().T)
                sel = tuple(torch.as_tensor(s).to(self.child.device).long() for s in sel)
                keep = (self.parent_depth[sel[0], 1] < self.depth_limit) & (self.child[sel] == 0)
                sel = tuple(s[keep] for s in sel)
                n_new = int(sel[0].shape[0])
                if n_new == 0:
                    break  # nothing left to split; earlier rounds may still have changed the tree
                end_new = first_new + n_new
                if end_new > self.capacity:
                    self._resize_add_cap(end_new - self.capacity)
                    resized = True
                parents = sel[0]
                new_ids = torch.arange(first_new, end_new, device=self.child.device)
                self.child[first_new:end_new] = 0
                self.child[sel] = (new_ids - parents).to(torch.int32)
                self.data.data[first_new:end_new] = self.data.data[sel][:, None, None, None]
                self.parent_depth[first_new:end_new, 0] = self._pack_index(
                    torch.stack(sel, dim=-1)).to(torch.int32)
                self.parent_depth[first_new:end_new, 1] = self.parent_depth[parents, 1] + 1
                if rep < repeats - 1:
                    # the next round splits exactly the cells of the nodes just made
                    cells = torch.arange(N ** 3, device=self.child.device)
                    sel = (new_ids.repeat_interleave(N ** 3),
                           (cells // (N * N)).repeat(n_new),
                           ((cells // N) % N).repeat(n_new),
                           (cells % N).repeat(n_new))
                self._n_internal += n_new
        if repeats > 0:
            self._invalidate()
        return resized

    def _refine_at(self, intnode_idx, xyzi):
        """Split the single leaf cell `xyzi` of node `intnode_idx`; unlike refine() the split cell's
        own record is zeroed (svox/svox.py:707-743)."""
        if self._lock_tree_structure:
            raise RuntimeError("Tree locked")
        assert min(xyzi) >= 0 and max(xyzi) < self.N
        if self.parent_depth[intnode_idx, 1] >= self.depth_limit:
            return
        x, y, z = xyzi
        if self.child[intnode_idx, x, y, z] != 0:
            return
        resized = False
        new_id = self.n_internal
        if new_id >= self.capacity:
            self._resize_add_cap(1)
            resized = True
        with torch.no_grad():
            self.child[new_id] = 0
            self.child[intnode_idx, x, y, z] = new_id - intnode_idx
            self.parent_depth[new_id, 0] = ((intnode_idx * self.N + x) * self.N + y) * self.N + z
            self.parent_depth[new_id, 1] = self.parent_depth[intnode_idx, 1] + 1
            self.data.data[new_id] = self.data.data[intnode_idx, x, y, z]
            self.data.data[intnode_idx, x, y, z] = 0
            self._n_internal += 1
        self._invalidate()
        return resized

    def shrink_to_fit(self):
        """Drop unused capacity (svox/svox.py:745-788; trees with freed nodes are compacted)."""
        if self._lock_tree_structure:
            raise RuntimeError("Tree locked")
        n_int, n_free = self.n_internal, int(self._n_free.item())
        new_cap = n_int - n_free
        if new_cap >= self.capacity:
            return False
        if n_free > 0:
            free = self.parent_depth[:n_int, 0] == -1
            shift = torch.cumsum(free, dim=0)
            live = torch.arange(n_int, device=free.device)[~free]
            par = tuple(self._unpack_index(self.parent_depth[live, 0].long()).T)
            par_shift = shift[par[0]]
            self.child[par] -= (shift[live] - par_shift).to(torch.int32)
            self.parent_depth[live, 0] -= (par_shift * self.N ** 3).to(torch.int32)
            self.data = nn.Parameter(self.data.data[live])
            self.child = self.child[live]
            self.parent_depth = self.parent_depth[live]
            self._n_internal.fill_(new_cap)
            self._n_free.zero_()
        else:
            self.data = nn.Parameter(self.data.data[:new_cap].clone())
            self.child = self.child[:new_cap].clone()
            self.parent_depth = self.parent_depth[:new_cap].clone()
        self._invalidate()
        return True

    def check_integrity(self):
        """Structural invariants (svox/svox.py:583-618): node 0 is the root, children come after
        their parents, links stay inside the table, parent and child links agree."""
        n_int, n_free = self.n_internal, int(self._n_free.item())
        assert n_int - n_free > 0, "Tree has no root"
        assert self.data.shape[0] == self.capacity, "Data capacity mismatch"
        assert self.child.shape[0] == self.capacity, "Child capacity mismatch"
        assert (self.parent_depth[0] == 0).all(), "Node at index 0 must be root"
        free = self.parent_depth[:n_int, 0] == -1
        ids = torch.arange(n_int, dtype=torch.long, device=self.child.device)[~free]
        links = self.child[ids]
        assert (links >= 0).all(), "Nodes not topologically sorted"
        targets = links.long() + ids[:, None, None, None]
        assert targets.max() < n_int, "Tree has an out-of-bounds child link"
        assert (self.parent_depth[targets.reshape(-1), 0] != -1).all(), \
            "Tree has a child link to a deleted node"
        ids = ids[ids != 0]
        if ids.numel() == 0:
            return True
        par = tuple(self._unpack_index(self.parent_depth[ids, 0].long()).T)
        assert par[0].max() < n_int and par[0].min() >= 0, "Parent link out-of-bounds"
        for i in range(1, 4):
            assert par[i].max() < self.N and par[i].min() >= 0, "Parent sublink out-of-bounds"
        assert (par[0] + self.child[par].long() == ids).all(), "parent->child cycle consistency failed"
        return True

    # ------------------------------------------------------------------ sizes
    @property
    def n_leaves(self):
        return self._all_leaves().shape[0]

    @property
    def n_internal(self):
        return int(self._n_internal.item())

    @property
    def capacity(self):
        return self.parent_depth.shape[0]

    @property
    def max_depth(self):
        return int(torch.max(self.depths).item())

    def accumulate_weights(self, op="sum"):
        """Context manager: while active, every rendered sample adds (or max-es) its compositing
        weight into a per-cell buffer (svox/svox.py:810-832, 1136-1161)."""
        return WeightAccumulator(self, op)

    # ------------------------------------------------------------------ persistence
    def save(self, path, shrink=True, compress=True):
        """npz with the reference's keys; `data` is stored as float16 (svox/svox.py:835-865)."""
        if shrink:
            self.shrink_to_fit()
        blob = {
            "data_dim": self.data_dim,
            "child": self.child.cpu(),
            "parent_depth": self.parent_depth.cpu(),
            "n_internal": self._n_internal.cpu().item(),
            "n_free": self._n_free.cpu().item(),
            "invradius3": self.invradius.cpu(),
            "offset": self.offset.cpu(),
            "depth_limit": self.depth_limit,
            "geom_resize_fact": self.geom_resize_fact,
            "data": self.data.data.half().cpu().numpy(),
        }
        if self.data_format is not None:
            blob["data_format"] = repr(self.data_format)
        if self.extra_data is not None:
            blob["extra_data"] = self.extra_data.cpu()
        (np.savez_compressed if compress else np.savez)(path, **blob)

    @classmethod
    def load(cls, path, device="cpu", dtype=torch.float32, map_location=None):
        """Inverse of save(); also reads files with the legacy scalar `invradius`
        (svox/svox.py:867-938)."""
        if map_location is not None:
            warn("map_location has been renamed to device and may be removed")
            device = map_location
        assert dtype in (torch.float32, torch.float64), "Unsupported dtype"
        tree = cls(dtype=dtype, device=device)
        z = np.load(path)
        tree.data_dim = int(z["data_dim"])
        tree.child = torch.from_numpy(z["child"]).to(device)
        tree.N = tree.child.shape[-1]
        tree.parent_depth = torch.from_numpy(z["parent_depth"]).to(device)
        tree._n_internal.fill_(int(z["n_internal"]))
        if "invradius3" in z.files:
            tree.invradius = torch.from_numpy(z["invradius3"].astype(np.float32)).to(device=device, dtype=dtype)
        else:
            tree.invradius = torch.full((3,), float(z["invradius"]), dtype=dtype, device=device)
        tree.offset = torch.from_numpy(z["offset"].astype(np.float32)).to(device=device, dtype=dtype)
        tree.depth_limit = int(z["depth_limit"])
        tree.geom_resize_fact = float(z["geom_resize_fact"])
        tree.data = nn.Parameter(torch.from_numpy(z["data"].astype(np.float32)).to(device=device, dtype=dtype))
        tree._n_free.fill_(int(z["n_free"]) if "n_free" in z.files else 0)
        tree.data_format = DataFormat(str(z["data_format"])) if "data_format" in z.files else None
        tree.extra_data = (torch.from_numpy(z["extra_data"]).to(device=device, dtype=dtype)
                           if "extra_data" in z.files else None)
        tree._invalidate()
        return tree

    # ------------------------------------------------------------------ tensor-like surface
    def __repr__(self):
        return (f"svox.N3Tree(N={self.N}, data_dim={self.data_dim}, depth_limit={self.depth_limit}, "
                f"capacity:{self.n_internal - int(self._n_free.item())}/{self.capacity}, "
                f"data_format:{self.data_format or 'RGBA'})")

    def __getitem__(self, key):
        return N3TreeView(self, key)

    def __setitem__(self, key, val):
        N3TreeView(self, key).set(val)

    def __iadd__(self, val):
        self[:] += val
        return self

    def __isub__(self, val):
        self[:] -= val
        return self

    def __imul__(self, val):
        self[:] *= val
        return self

    def __itruediv__(self, val):
        self[:] /= val
        return self

    __idiv__ = __itruediv__   # the name the reference defines (svox/svox.py:968)

    @property
    def ndim(self):
        return 2

    @property
    def shape(self):
        return torch.Size((self.n_leaves, self.data_dim))

    def size(self, dim):
        return self.data_dim if dim == 1 else self.n_leaves

    def numel(self):
        return self.data_dim * self.n_leaves

    def __len__(self):
        return self.n_leaves

    # ------------------------------------------------------------------ internals
    def _calc_corners(self, nodes, cuda=True):
        """Lower corners (tree coordinates) of the leaves `nodes` (Q, 4) [node, x, y, z]."""
        if not cuda or not self.data.is_cuda:
            _no_fallback("N3Tree._calc_corners")
        return _C.calc_corners(self._spec(), nodes.to(self.data.device).long().contiguous())

    def _pack_index(self, txyz):
        N = self.N
        return ((txyz[:, 0] * N + txyz[:, 1]) * N + txyz[:, 2]) * N + txyz[:, 3]

    def _unpack_index(self, flat):
        N = self.N
        z = flat % N
        rest = torch.div(flat, N, rounding_mode="floor")
        y = rest % N
        rest = torch.div(rest, N, rounding_mode="floor")
        x = rest % N
        node = torch.div(rest, N, rounding_mode="floor")
        return torch.stack((node, x, y, z), dim=-1)

    def _resize_add_cap(self, cap_needed):
        cap_needed = max(int(cap_needed), int(self.capacity * (self.geom_resize_fact - 1.0)))

        def grow(t):
            pad = torch.zeros((cap_needed, *t.shape[1:]), dtype=t.dtype, device=t.device)
            return torch.cat((t, pad), dim=0)

        self.data = nn.Parameter(grow(self.data.data))
        self.child = grow(self.child)
        self.parent_depth = grow(self.parent_depth)

    def _make_val_tensor(self, val):
        t = torch.tensor(val, dtype=self.data.dtype, device=self.data.device)
        while t.dim() < 2:
            t = t[None]
        if t.shape[-1] == 1:
            t = t.expand(-1, self.data_dim).contiguous()
        else:
            assert t.shape[-1] == self.data_dim
        return t

    def _all_leaves(self):
        """(n_leaves, 4) int64 [node, x, y, z] of every leaf cell, lexicographic, on the CPU."""
        if self._last_all_leaves is None:
            self._last_all_leaves = (self.child[:self.n_internal] == 0).nonzero(as_tuple=False).cpu().contiguous()
        return self._last_all_leaves

    def world2tree(self, indices):
        return torch.addcmul(self.offset, indices, self.invradius)

    def tree2world(self, indices):
        return (indices - self.offset) / self.invradius

    def _invalidate(self):
        self._ver += 1
        self._writes = getattr(self, "_writes", 0) + 1
        self._last_all_leaves = None
        self._last_frontier = None

    def touch(self):
        """Tells the tree that its values were written in a way torch's version counters do not see
        (a kernel of this package, or `tree.data.data[...] = ...`): kept marks of the empty leaves
        are dropped, and a backward pass that follows does not use notes its forward pass took of
        the old values.  Every write path of this package calls it; a caller that writes through
        `tree.data.data` itself must (no reference counterpart)."""
        self._writes = getattr(self, "_writes", 0) + 1
        self._leaf_marks = None

    def _spec(self, world=True):
        """The TreeSpec handed to the operators (svox/svox.py:1084-1103).  For tree-local queries
        offset / scaling stay None, which the library reads as the identity transform."""
        spec = _C.TreeSpec()
        spec.data = self.data
        spec.child = self.child
        spec.parent_depth = self.parent_depth
        spec.extra_data = self.extra_data
        spec.offset = self.offset if world else None
        spec.scaling = self.invradius if world else None
        spec._weight_accum = getattr(self, "_weight_accum", None)
        spec._weight_accum_max = getattr(self, "_weight_accum_op", None) == "max"
        spec.owner = self    # lets the autograd functions see the tree's write counter
        if getattr(self, "_leaf_marks", None) is not None:
            if self._leaf_marks_key == self._marks_key():
                spec.child_marks = self._leaf_marks
                spec.child_marks_thresh, spec.child_marks_softplus = getattr(self, "_leaf_marks_made_with", (0.0, False))
            else:
                self._leaf_marks = None      # the tree has changed since: the marks are void
        return spec

    # ------------------------------------------------------------------ marks of the empty leaves
    def mark_empty_leaves(self, sigma_thresh=0.0, density_softplus=False):
        """For a tree that will be rendered many times as it is (beyond the reference): note which
        leaves have no density, so that the renderers pass through them without reading it.  Renders
        are bit-identical and faster on sparse scenes.

        sigma_thresh, density_softplus: of the renders that will follow.  With 0 / False (the default) the marks
        serve every render, backward pass and se_grad call of a renderer without density_softplus.  Marks made
        with a renderer's own `sigma_thresh` (1e-2 for `fast=True`) let its forward renders also skip the leaves
        below the threshold and read a leaf's density together with its colour; calls that need those leaves
        (backward passes, renders with a smaller threshold) then run without marks.

        The marks describe the tree as it is now.  They are dropped by every method of the tree and
        its views that writes values or changes the structure, and by in-place torch operations on
        `tree.data` / `tree.child` (their version counters tell).  A write that bypasses both --
        `tree.data.data -= ...` as in svox's own toy example -- does not: call `tree.touch()`
        (or `clear_leaf_marks()`, or this method again) after such a write."""
        self._leaf_marks = None
        self._leaf_marks = _C.mark_empty_leaves(self._spec(), sigma_thresh, density_softplus)
        self._leaf_marks_made_with = (float(sigma_thresh), bool(density_softplus))
        self._leaf_marks_key = self._marks_key()
        return self

    def clear_leaf_marks(self):
        self._leaf_marks = None

    def _marks_key(self):
        return (self._ver, getattr(self, "_writes", 0), self.data._version, self.child._version,
                self.data.data_ptr(), self.child.data_ptr())

    def _maybe_auto_data_dim(self):
        fmt_dim = self.data_format.data_dim if self.data_format is not None else None
        if fmt_dim is not None:
            if self.data_dim is None:
                self.data_dim = fmt_dim
            else:
                assert fmt_dim == self.data_dim, "data_dim invalid for given data format"
        elif self.data_dim is None:
            self.data_dim = 4


def _forward_to_view():
    """tree.depths == tree[:].depths and so on (svox/svox.py:1114-1134)."""
    props = ["depths", "lengths", "lengths_local", "corners", "corners_local", "values", "values_local"]
    funcs = ["sample", "sample_local", "aux", "normal_", "clamp_", "uniform_", "relu_", "sigmoid_",
             "nan_to_num_"]
    for name in funcs:
        setattr(N3Tree, name, (lambda n: lambda self, *a, **k: getattr(self[:], n)(*a, **k))(name))
    for name in props:
        setattr(N3Tree, name, property((lambda n: lambda self: getattr(self[:], n))(name)))


_forward_to_view()


class WeightAccumulator:
    def __init__(self, tree, op):
        assert op in ("sum", "max"), "Unsupported accumulation"
        self.tree = tree
        self.op = op

    def __enter__(self):
        t = self.tree
        t._lock_tree_structure = True
        t._weight_accum = torch.zeros(t.child.shape, dtype=t.data.dtype, device=t.data.device)
        t._weight_accum_op = self.op
        self.weight_accum = t._weight_accum
        return self

    def __exit__(self, exc_type, exc, tb):
        t = self.tree
        t._weight_accum = None
        t._weight_accum_op = None
        t._lock_tree_structure = False

    @property
    def value(self):
        return self.weight_accum

    def __call__(self):
        return self.tree.aux(self.weight_accum)


def gen_grid(D):
    """Centres of a D^3 grid over [0, 1]^3, (D, D, D, 3) in xyz order (svox/svox.py:1163-1173)."""
    axis = (torch.arange(D) + 0.5) / D
    return torch.stack(torch.meshgrid(axis, axis, axis, indexing="ij"), dim=-1)
