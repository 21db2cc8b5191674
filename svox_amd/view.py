"""N3TreeView: a tensor-like window onto selected leaves of an N3Tree.

`tree[key]` builds one.  The tree is seen as a (n_leaves, data_dim) matrix:
  tree[i], tree[a:b], tree[mask], tree[idx_tensor]   leaves by position in the leaf list
  tree[x, y, z]                                       the leaf containing one world point
  tree[P], tree[LocalIndex(P)]                        leaves containing the points P (Q, 3)
any of them followed by a channel index: tree[:, :3], tree[P, -1:], tree[0, 0, 0, :-1].
Reference: svox/helpers.py:27-358.
"""
import torch

from .formats import LocalIndex


class N3TreeView:
    def __init__(self, tree, key):
        self.tree = tree
        self.single_key = False
        local = False
        if isinstance(key, tuple) and len(key) >= 3:
            # tree[x, y, z(, channels)]: one point
            point = torch.tensor(key[:3], dtype=tree.data.dtype, device=tree.data.device).reshape(1, 3)
            key = (point, *key[3:]) if len(key) > 3 else point
        rest = tuple(key[1:]) if isinstance(key, tuple) else ()
        leaf_key = key[0] if isinstance(key, tuple) else key
        if isinstance(leaf_key, LocalIndex):
            leaf_key, local = leaf_key.val, True
        if torch.is_tensor(leaf_key) and leaf_key.dim() == 2 and leaf_key.shape[1] == 3:
            pts = leaf_key.to(dtype=tree.data.dtype)
            _, packed = tree.forward(pts, want_node_ids=True, world=not local)
            self._packed_ids = packed.clone()
            cells = tuple(tree._unpack_index(packed).T)
        else:
            self._packed_ids = None
            if isinstance(leaf_key, int):
                leaf_key = torch.tensor([leaf_key])
                self.single_key = True
            cells = tuple(tree._all_leaves()[leaf_key].T)
        self.key = (*cells, *rest)
        self._tree_ver = tree._ver

    # -------------------------------------------------------------- reading and writing
    def _needs_two_step(self):
        # a tensor / list channel index cannot be combined with the four leaf index tensors
        return len(self.key) == 5 and not isinstance(self.key[-1], (slice, int))

    def _gather(self, data):
        out = data[self.key[:-1]][..., self.key[-1]] if self._needs_two_step() else data[self.key]
        return out[0] if self.single_key else out

    @property
    def values(self):
        """Selected values with autograd, (n, data_dim) (1-D for an int key)."""
        self._check_ver()
        return self._gather(self.tree.data)

    @property
    def values_nograd(self):
        self._check_ver()
        return self._gather(self.tree.data.data)

    def set(self, value):
        self._check_ver()
        if isinstance(value, N3TreeView):
            value = value.values_nograd
        data = self.tree.data.data
        self.tree.touch()      # the write below goes past data's version counter
        if self._needs_two_step():
            rows = data[self.key[:-1]]
            rows[..., self.key[-1]] = value
            data[self.key[:-1]] = rows
        else:
            data[self.key] = value

    def __setitem__(self, key, value):
        vals = self.values_nograd.clone()
        vals[key] = value
        self.set(vals)

    def refine(self, repeats=1):
        """Split the selected leaves (tree.refine with this view's cells)."""
        self._check_ver()
        return self.tree.refine(repeats, sel=self._unique_node_key())

    def aux(self, arr):
        """Index another (capacity, N, N, N[, C]) array the way this view indexes tree.data."""
        if self._needs_two_step():
            return arr[self.key[:-1]][..., self.key[-1]]
        return arr[self.key]

    # -------------------------------------------------------------- geometry
    @property
    def shape(self):
        return self.values_nograd.shape

    @property
    def ndim(self):
        return 2

    @property
    def depths(self):
        """Depth of each selected leaf (children of the root have depth 0), int32 (n,)."""
        self._check_ver()
        return self.tree.parent_depth[self.key[0], 1]

    @property
    def lengths_local(self):
        """Side length of each leaf in tree coordinates, (n,)."""
        self._check_ver()
        return self.tree.N ** (-self.depths.float() - 1.0)

    @property
    def lengths(self):
        """Side lengths in world units, (n, 3)."""
        return self.lengths_local[:, None] / self.tree.invradius

    @property
    def corners_local(self):
        """Lower corner of each leaf in tree coordinates, (n, 3)."""
        self._check_ver()
        return self.tree._calc_corners(self._indexer())

    @property
    def corners(self):
        """Lower corners in world coordinates, (n, 3)."""
        return (self.corners_local - self.tree.offset) / self.tree.invradius

    def sample(self, n_samples, device=None):
        """Uniform world-space points inside each selected leaf, (n, n_samples, 3)."""
        self._check_ver()
        device = self.tree.data.device if device is None else device
        corn = self.corners.to(device=device)
        length = self.lengths.to(device=device)
        u = torch.rand((corn.shape[0], n_samples, 3), device=device, dtype=length.dtype)
        return corn[:, None] + u * length[:, None]

    def sample_local(self, n_samples):
        self._check_ver()
        corn = self.corners_local
        length = self.lengths_local.to(corn.device)
        u = torch.rand((corn.shape[0], n_samples, 3), device=corn.device, dtype=corn.dtype)
        return corn[:, None] + u * length[:, None, None]

    # -------------------------------------------------------------- in-place helpers
    def normal_(self, mean=0.0, std=1.0):
        self.set(torch.randn_like(self.values_nograd) * std + mean)

    def uniform_(self, min=0.0, max=1.0):
        self.set(torch.rand_like(self.values_nograd) * (max - min) + min)

    def clamp_(self, min=None, max=None):
        self.set(torch.clamp(self.values_nograd, min, max))

    def relu_(self):
        self.set(torch.relu(self.values_nograd))

    def sigmoid_(self):
        self.set(torch.sigmoid(self.values_nograd))

    def nan_to_num_(self, inf_val=2e4):
        self.set(torch.nan_to_num(self.values_nograd, nan=0.0, posinf=inf_val, neginf=-inf_val))

    # -------------------------------------------------------------- plumbing
    def __repr__(self):
        return "N3TreeView(" + repr(self.values) + ")"

    def __torch_function__(self, func, types, args=(), kwargs=None):
        self._check_ver()
        unwrap = lambda a: a.values if isinstance(a, N3TreeView) else a  # noqa: E731
        return func(*[unwrap(a) for a in args], **(kwargs or {}))

    def _indexer(self):
        return torch.stack([torch.as_tensor(k).long().to(self.tree.data.device) for k in self.key[:4]], dim=-1)

    def _unique_node_key(self):
        if self._packed_ids is None:
            return self.key[:4]
        return tuple(self.tree._unpack_index(torch.unique(self._packed_ids)).T)

    def _check_ver(self):
        if self.tree._ver > self._tree_ver:
            self.key = self._packed_ids = None
            raise RuntimeError("N3TreeView has been invalidated because tree data layout has changed")


def _delegate_to_values():
    """Arithmetic, comparisons and reductions act on `.values` (svox/helpers.py:337-358)."""
    plain = ["__floordiv__", "__mod__", "__eq__", "__ne__", "__ge__", "__gt__", "__le__", "__lt__",
             "__floor__", "__ceil__", "__round__", "__len__", "item", "size", "dim", "numel"]
    with_grad = ["__add__", "__mul__", "__sub__", "__truediv__", "__radd__", "__rsub__", "__rmul__",
                 "__rtruediv__", "__abs__", "__pos__", "__neg__", "clamp", "clamp_max", "clamp_min",
                 "relu", "sigmoid", "max", "min", "mean", "sum", "__getitem__"]

    def make(name, grad):
        def method(self, *args, **kwargs):
            target = self.values if grad else self.values_nograd
            return getattr(target, name)(*args, **kwargs)
        method.__name__ = name
        return method

    for name in plain:
        setattr(N3TreeView, name, make(name, False))
    for name in with_grad:
        setattr(N3TreeView, name, make(name, True))
    # the reference also lists the Python 2 spellings of division
    N3TreeView.__div__ = N3TreeView.__truediv__
    N3TreeView.__rdiv__ = N3TreeView.__rtruediv__
    N3TreeView.__hash__ = object.__hash__


_delegate_to_values()
