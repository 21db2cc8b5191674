"""svox_amd -- N^3-tree queries and differentiable volume rendering on AMD MI355X (gfx950).

Use it where `import svox` was used:  `import svox_amd as svox`.
"""
from .formats import DataFormat, LocalIndex, NDCConfig, Rays
from .renderer import VolumeRenderer
from .tree import N3Tree
from .view import N3TreeView

__version__ = "0.1.0"
__all__ = ["N3Tree", "N3TreeView", "VolumeRenderer", "NDCConfig", "Rays", "LocalIndex", "DataFormat"]
