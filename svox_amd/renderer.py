"""VolumeRenderer: differentiable volume rendering of an N3Tree on the GPU.

Mirrors `svox.VolumeRenderer` (svox/renderer.py:114-469): same constructor arguments, `forward(rays)`
for ray batches, `render_persp(c2w, ...)` for pinhole images, `persp_rays`, the `fast` switch and
the `sigma_thresh` / `stop_thresh` attribute overrides.  Rendering runs in the HIP kernels behind
`svox_amd.csrc`; gradients flow to `tree.data` only.
"""
from warnings import warn

import torch
from torch import nn

from . import csrc as _C
from .formats import DataFormat, NDCConfig, Rays  # noqa: F401


def _rays_spec_from_rays(rays):
    spec = _C.RaysSpec()
    spec.origins = rays.origins
    spec.dirs = rays.dirs
    spec.vdirs = rays.viewdirs
    return spec


def _make_camera_spec(c2w, width, height, fx, fy):
    spec = _C.CameraSpec()
    spec.c2w = c2w
    spec.width = width
    spec.height = height
    spec.fx = fx
    spec.fy = fy
    return spec


# Whether a forward pass that will be differentiated keeps notes for its backward pass (faster
# training steps; the forward pass itself takes longer, as it follows every ray to its end).
KEEP_NOTES = True


def _wants_notes(data):
    """True when a forward pass started now will be followed by a backward pass.  Asked before
    Function.apply: inside Function.forward gradient mode is always off, and needs_input_grad is
    also set inside torch.no_grad(), where no graph is recorded."""
    return KEEP_NOTES and torch.is_grad_enabled() and data.requires_grad


class NotesBudget:
    """How much room per ray the notes of a renderer's forward passes get.  It starts at
    csrc.BACKWARD_RECORDS_PER_RAY leaves per ray; a pass whose notes ran out of room (its rays are then
    marched by the backward pass: correct, but the noting was for nothing) doubles the room of the
    passes after it, up to MAX_FACTOR times the start (and to the memory limits of
    csrc._backward_workspace); passes that use less than a quarter of their room halve it again.

    Nothing here waits for the GPU: the counter a pass leaves is copied to pinned memory behind the
    pass, and looked at by a later pass only once the copy has arrived.  While the stream is being
    captured into a graph (torch.cuda.graph) nothing is observed: a replay cannot change the size of
    the buffers it was captured with, so the room stays what it was when the capture began."""

    MAX_FACTOR = 16

    def __init__(self):
        self.factor = 1
        self._pending = None      # (pinned int64[1], event, pool stocks) of the last pass looked after
        self._landing = None      # the pinned buffer, allocated on first use

    def __getstate__(self):
        # (a copy or a pickle of the renderer takes the figure along, not the buffer and the event)
        return {"factor": self.factor}

    def __setstate__(self, state):
        self.factor = state["factor"]
        self._pending = None
        self._landing = None

    def records_per_ray(self):
        self._settle()
        return int(_C.BACKWARD_RECORDS_PER_RAY) * self.factor

    def _settle(self):
        if self._pending is None or torch.cuda.is_current_stream_capturing():
            return
        landing, event, pool = self._pending
        if not event.query():
            return
        self._pending = None
        self.adjust(int(landing[0]), pool)

    def adjust(self, asked, pool):
        """One observation: `asked` stocks of chunks were asked for, the workspace had `pool`."""
        if asked > 0 and asked >= pool:
            self.factor = min(self.factor * 2, self.MAX_FACTOR)
        elif asked * 4 < pool and self.factor > 1:
            self.factor //= 2

    def observe(self, notes, n_rays):
        """Called right after the launch of a noted forward pass (on the current stream)."""
        if notes is None or self._pending is not None or torch.cuda.is_current_stream_capturing():
            return
        counter, pool = _C.notes_pool_use(notes, n_rays)
        if self._landing is None:
            self._landing = torch.empty(1, dtype=torch.int64, pin_memory=True)
        self._landing.copy_(counter, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._pending = (self._landing, event, pool)


class _VolumeRenderFunction(torch.autograd.Function):
    """svox/renderer.py:57-72.  The specs are kept on ctx as plain attributes, so the backward
    pass sees the tree as it is when backward runs.

    When a gradient will be asked for, the forward pass also leaves notes of the leaves it met
    (volume_render_noted) and the backward pass works from them instead of marching through the tree
    again.  The notes stand for the tree as it was: if tree.data or the rays were written to between
    the two passes (their version counters tell), the backward pass marches as the reference does."""

    @staticmethod
    def forward(ctx, data, tree, rays, opt, keep_notes=False, budget=None):
        ctx.tree, ctx.rays, ctx.opt = tree, rays, opt
        ctx.notes = None
        ctx.versions = _versions(tree, rays)
        if keep_notes:
            out, ctx.notes = _C.volume_render_noted(tree, rays, opt, budget.records_per_ray() if budget else None)
            if budget:
                budget.observe(ctx.notes, int(rays.origins.shape[0]))
            return out
        return _C.volume_render(tree, rays, opt)

    @staticmethod
    def backward(ctx, grad_out):
        if not ctx.needs_input_grad[0]:
            return None, None, None, None, None, None
        notes, ctx.notes = ctx.notes, None
        if ctx.versions != _versions(ctx.tree, ctx.rays):
            # the tree or the rays were written to since the forward pass: its notes and the marks of
            # the empty leaves it ran with describe the old values; march through the tree as it is
            notes, ctx.tree.child_marks = None, None
        if notes is not None:
            grad = _C.volume_render_backward_noted(ctx.tree, ctx.rays, ctx.opt, grad_out.contiguous(), notes)
        else:
            grad = _C.volume_render_backward(ctx.tree, ctx.rays, ctx.opt, grad_out.contiguous())
        return grad, None, None, None, None, None


def _tree_versions(tree):
    """What tells that a tree was written to: torch's version counters of data and child and, for
    writes those do not see (kernels of this package, N3TreeView.set, tree.touch()), the write
    counter of the N3Tree the spec was made from."""
    owner = getattr(tree, "owner", None)
    return (tree.data._version, tree.child._version, getattr(owner, "_writes", 0), getattr(owner, "_ver", 0))


def _versions(tree, rays):
    """Version counters of everything the notes of a forward pass depend on."""
    return _tree_versions(tree) + tuple(t._version for t in (rays.origins, rays.dirs, rays.vdirs))


class _VolumeRenderImageFunction(torch.autograd.Function):
    """svox/renderer.py:74-89; one pose (3, 4) / (4, 4) or, beyond the reference, a stack of poses
    rendered in one launch.  Notes are kept between the passes as in _VolumeRenderFunction."""

    @staticmethod
    def forward(ctx, data, tree, cam, opt, keep_notes=False, budget=None):
        ctx.tree, ctx.cam, ctx.opt = tree, cam, opt
        ctx.notes = None
        ctx.versions = _image_versions(tree, cam)
        if keep_notes:
            out, ctx.notes = _C.volume_render_images_noted(tree, cam, opt,
                                                           budget.records_per_ray() if budget else None)
            if budget:
                n_images = 1 if cam.c2w.dim() == 2 else int(cam.c2w.shape[0])
                budget.observe(ctx.notes, n_images * cam.height * cam.width)
            return out
        return _C.volume_render_image(tree, cam, opt) if cam.c2w.dim() == 2 else _C.volume_render_images(tree, cam, opt)

    @staticmethod
    def backward(ctx, grad_out):
        if not ctx.needs_input_grad[0]:
            return None, None, None, None, None, None
        notes, ctx.notes = ctx.notes, None
        if ctx.versions != _image_versions(ctx.tree, ctx.cam):
            notes, ctx.tree.child_marks = None, None     # as in _VolumeRenderFunction.backward
        grad = _C.volume_render_images_backward_noted(ctx.tree, ctx.cam, ctx.opt, grad_out.contiguous(), notes)
        return grad, None, None, None, None, None


_VolumeRenderImagesFunction = _VolumeRenderImageFunction


def _image_versions(tree, cam):
    return _tree_versions(tree) + (cam.c2w._version,)


def convert_to_ndc(origins, directions, focal, w, h, near=1.0):
    """Rays in normalised device coordinates of a forward-facing scene (svox/renderer.py:92-112).
    The image kernels apply the same map themselves and then normalise the direction; ray batches
    passed to `VolumeRenderer.forward` must be converted by the caller."""
    t = -(near + origins[..., 2]) / directions[..., 2]
    origins = origins + t[..., None] * directions
    ox, oy, oz = origins.unbind(-1)
    dx, dy, dz = directions.unbind(-1)
    sx, sy = -(2.0 * focal) / w, -(2.0 * focal) / h
    new_o = torch.stack([sx * (ox / oz), sy * (oy / oz), 1.0 + 2.0 * near / oz], -1)
    new_d = torch.stack([sx * (dx / dz - ox / oz), sy * (dy / dz - oy / oz), -2.0 * near / oz], -1)
    return new_o, new_d


class VolumeRenderer(nn.Module):
    """Stores rendering options for one tree; holds no tensors of its own.

    :param tree: N3Tree to render
    :param step_size: epsilon added to every leaf crossing
    :param background_brightness: 1.0 = white
    :param ndc: NDCConfig(width, height, focal) or None
    :param min_comp, max_comp: range of basis components to render (-1 = last);
           min_comp > max_comp renders 0.5 grey
    :param density_softplus: apply log(1 + exp(sigma - 1)) to the stored density
    :param rgb_padding: colours become sigmoid * (1 + 2 p) - p

    Memory and state beyond the reference's renderer (which holds nothing between calls):

    * A forward pass that will be differentiated (gradient mode on, `tree.data.requires_grad`) keeps
      notes of the leaves its rays met until `backward()` has run: 768 bytes per ray to begin with (30
      leaves per ray on average; 3.9 GB for eight 800x800 images; batches below 2^20 rays get up to four
      times the room per ray, `csrc.SMALL_BATCH_ROOM`); a pass whose notes ran out of room
      doubles the room of the next passes, up to 16 times, and passes that leave most of it unused
      halve it again (`renderer.notes_budget`, a `NotesBudget`).  At most
      `csrc.BACKWARD_WORKSPACE_LIMIT` (4 GiB) and at most a quarter of the device memory that is free
      at the time.  Where that leaves no room, or
      the allocation fails, the pass runs without notes and the backward pass marches through the tree
      twice, as the reference does: same results, slower.  The noted forward pass follows every ray to
      its end (no early stop), so it is slower than a forward pass under `torch.no_grad()`.  The notes
      are used once: a second `backward()` through a retained graph marches.  `renderer.KEEP_NOTES =
      False` switches the notes off.  If `tree.data`, the tree's structure, the rays or the camera are
      written to between the two passes -- through torch (version counters), a method of the tree or a
      view, or `tree.touch()` -- the backward pass drops the notes and any marks of empty leaves and
      marches through the tree as it then is, which is what the reference's backward pass sees.
      Only a write through `tree.data.data[...]` that is not followed by `tree.touch()` goes unseen.
    * A call of `render_persp` on a stack of poses with at least `csrc.AUTO_MARK_RAYS_PER_CELL` (0.7)
      rays per cell of the tree, and at least `csrc.AUTO_MARK_MIN_RAYS` (262 144) rays, first marks the
      empty leaves (one int32 per cell, freed after the
      call; 25 MB and 0.125 ms for a 512^3 tree of 774 k nodes) so that the march passes through them
      without reading their density.  Smaller calls do not; `N3Tree.mark_empty_leaves()` keeps marks
      on the tree for all of them.  Pictures are bit-identical either way.
    """

    def __init__(self, tree, step_size=1e-3, background_brightness=1.0, ndc=None, min_comp=0,
                 max_comp=-1, density_softplus=False, rgb_padding=0.0):
        super().__init__()
        self.tree = tree
        self.step_size = step_size
        self.background_brightness = background_brightness
        self.ndc_config = ndc
        self.min_comp = min_comp
        self.max_comp = max_comp
        self.density_softplus = density_softplus
        self.rgb_padding = rgb_padding
        if isinstance(tree.data_format, DataFormat):
            self._data_format = None
        else:
            warn("Legacy N3Tree (pre 0.2.18) without data_format, auto-infering SH deg")
            ddim = tree.data_dim
            self._data_format = DataFormat("" if ddim == 4 else f"SH{(ddim - 1) // 3}")
        self.tree._weight_accum = None
        self.notes_budget = NotesBudget()

    @property
    def data_format(self):
        return self._data_format or self.tree.data_format

    def _require_gpu(self, cuda, what):
        if not cuda or not self.tree.data.is_cuda:
            raise RuntimeError(
                f"{what}: this build has only the HIP path (tree on a GPU, cuda=True); the "
                "reference's PyTorch fallback renderer is not included")

    def forward(self, rays, cuda=True, fast=False):
        """Render a batch of rays -> (B, rgb_dim).  `fast` sets sigma_thresh = stop_thresh = 1e-2."""
        self._require_gpu(cuda, "VolumeRenderer.forward")
        return _VolumeRenderFunction.apply(self.tree.data, self.tree._spec(),
                                           _rays_spec_from_rays(rays), self._get_options(fast),
                                           _wants_notes(self.tree.data), self.notes_budget)

    def render_persp(self, c2w, width=800, height=800, fx=1111.111, fy=None, cuda=True, fast=False):
        """Render a pinhole image -> (height, width, rgb_dim).  c2w is (3, 4) or (4, 4), OpenGL
        convention (camera looks down -z, +y up); pixel (ix, iy) looks through its corner.

        Beyond the reference: a stack of poses (n, 3, 4) or (n, 4, 4) renders n images in one
        kernel launch and returns (n, height, width, rgb_dim)."""
        self._require_gpu(cuda, "VolumeRenderer.render_persp")
        if fy is None:
            fy = fx
        cam = _make_camera_spec(c2w.to(dtype=self.tree.data.dtype, device=self.tree.data.device).contiguous(),
                                width, height, fx, fy)
        fn = _VolumeRenderImagesFunction if c2w.dim() == 3 else _VolumeRenderImageFunction
        return fn.apply(self.tree.data, self.tree._spec(), cam, self._get_options(fast),
                        _wants_notes(self.tree.data), self.notes_budget)

    def se_grad(self, rays, colors):
        """Rendered colour plus gradient and Hessian diagonal (Gauss-Newton: squared Jacobian rows) of
        0.5 * sum (render - colors)^2 for a ray batch -> (colors (B, rgb_dim), grad, diag_hessian), the
        last two shaped like tree.data.  rgb_dim must be <= 4.  svox/renderer.py:324-348."""
        self._require_gpu(True, "VolumeRenderer.se_grad")
        return _C.se_grad(self.tree._spec(), _rays_spec_from_rays(rays), colors, self._get_options(False))

    def se_grad_persp(self, c2w, colors, width=800, height=800, fx=1111.111, fy=None):
        """Image version of se_grad: colors is (height, width, rgb_dim).  svox/renderer.py:350-385."""
        self._require_gpu(True, "VolumeRenderer.se_grad_persp")
        if fy is None:
            fy = fx
        cam = _make_camera_spec(c2w.to(dtype=self.tree.data.dtype, device=self.tree.data.device).contiguous(),
                                width, height, fx, fy)
        return _C.se_grad_persp(self.tree._spec(), cam, self._get_options(False), colors)

    @staticmethod
    def persp_rays(c2w, width=800, height=800, fx=1111.111, fy=None):
        """Row-major pinhole rays usable with forward() (svox/renderer.py:387-426; no NDC)."""
        if fy is None:
            fy = fx
        dev = c2w.device
        origins = c2w[None, :3, 3].expand(height * width, -1).contiguous()
        ys = torch.arange(height, dtype=torch.float64, device=dev)
        xs = torch.arange(width, dtype=torch.float64, device=dev)
        yy, xx = torch.meshgrid(ys, xs, indexing="ij")
        cam = torch.stack(((xx - width * 0.5) / float(fx), -(yy - height * 0.5) / float(fy),
                           -torch.ones_like(xx)), dim=-1)
        cam = cam / torch.norm(cam, dim=-1, keepdim=True)
        dirs = (cam.reshape(-1, 3) @ c2w[:3, :3].double().T).float().contiguous()
        return Rays(origins=origins, dirs=dirs, viewdirs=dirs)

    def _get_options(self, fast=False):
        """RenderOptions for one call (svox/renderer.py:432-469)."""
        fmt = self.data_format
        opts = _C.RenderOptions()
        opts.step_size = self.step_size
        opts.background_brightness = self.background_brightness
        opts.format = fmt.format
        opts.basis_dim = fmt.basis_dim
        opts.min_comp = self.min_comp
        opts.max_comp = self.max_comp + fmt.basis_dim if self.max_comp < 0 else self.max_comp
        opts.density_softplus = self.density_softplus
        opts.rgb_padding = self.rgb_padding
        if self.ndc_config is not None:
            opts.ndc_width = self.ndc_config.width
            opts.ndc_height = self.ndc_config.height
            opts.ndc_focal = self.ndc_config.focal
        else:
            opts.ndc_width = -1
        opts.sigma_thresh = opts.stop_thresh = 1e-2 if fast else 0.0
        if hasattr(self, "sigma_thresh"):
            opts.sigma_thresh = self.sigma_thresh
        if hasattr(self, "stop_thresh"):
            opts.stop_thresh = self.stop_thresh
        return opts
