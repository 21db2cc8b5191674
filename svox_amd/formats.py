"""Small value types of the public API: data formats, ray bundles, NDC settings, local indices.

Reference: svox/helpers.py:376-424 (LocalIndex, DataFormat), svox/renderer.py:36-37 (NDCConfig,
Rays).
"""
import re
from collections import namedtuple

NDCConfig = namedtuple("NDCConfig", ["width", "height", "focal"])
Rays = namedtuple("Rays", ["origins", "dirs", "viewdirs"])


class LocalIndex:
    """Marks a (Q, 3) point tensor as tree-local coordinates in [0, 1]^3: `tree[LocalIndex(p)]`."""

    def __init__(self, val):
        self.val = val


class DataFormat:
    """How the K numbers of a leaf are read by the renderer.

    "RGBA" (or ""): colours then sigma, basis_dim -1, data_dim left to the tree (default 4).
    "SH<n>", "SG<n>", "ASG<n>": n basis functions per colour channel, data_dim 3n + 1.
    SH needs a square n of at most 25.
    """

    RGBA = 0
    SH = 1
    SG = 2
    ASG = 3
    _NAMES = {RGBA: "RGBA", SH: "SH", SG: "SG", ASG: "ASG"}

    def __init__(self, txt):
        txt = "" if txt is None else str(txt)
        m = re.match(r"^([A-Za-z]*)(.*)$", txt)
        kind, digits = m.group(1), m.group(2)
        if digits == "":
            self.format = DataFormat.RGBA
            self.basis_dim = -1
            self.data_dim = None
            return
        self.basis_dim = int(digits)
        assert self.basis_dim > 0, "data_format basis_dim must be positive"
        self.data_dim = 3 * self.basis_dim + 1
        if kind == "SH":
            self.format = DataFormat.SH
            root = int(self.basis_dim ** 0.5)
            assert root * root == self.basis_dim, "SH basis dim must be square number"
            assert self.basis_dim <= 25, "SH only supported up to basis_dim 25"
        elif kind == "SG":
            self.format = DataFormat.SG
        elif kind == "ASG":
            self.format = DataFormat.ASG
        else:
            self.format = DataFormat.RGBA

    def __repr__(self):
        name = DataFormat._NAMES[self.format]
        return name + (str(self.basis_dim) if self.basis_dim >= 0 else "")

    def __eq__(self, other):
        return isinstance(other, DataFormat) and repr(self) == repr(other)

    def __hash__(self):
        return hash(repr(self))
