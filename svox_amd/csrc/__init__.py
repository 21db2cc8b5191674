"""svox_amd.csrc -- the operator module the Python layer calls.

It presents the names of the reference's extension module `svox.csrc`
(svox/csrc/svox.cpp:63-122): the four spec classes with the same attributes and the free functions
`query_vertical`, `query_vertical_backward`, `assign_vertical`, `calc_corners`, `volume_render`,
`volume_render_image`, `volume_render_backward`, `volume_render_image_backward`.  Each function
checks its tensors the way the reference's `check()` methods do (svox/csrc/include/data_spec.hpp),
allocates the outputs with the reference's shapes / dtypes / devices and calls the matching
extern "C" entry point of libsvox_hip.so on torch's current stream.

There is no CPU implementation here: tensors that are not on a GPU raise, and a missing library
raises at the first call.
"""
import ctypes

import torch

from . import _abi
from ._abi import FORMAT_ASG, FORMAT_RGBA, FORMAT_SG, FORMAT_SH  # noqa: F401


class RaysSpec:
    """svox/csrc/include/data_spec.hpp:51-63"""

    def __init__(self):
        self.origins = None
        self.dirs = None
        self.vdirs = None


class TreeSpec:
    """svox/csrc/include/data_spec.hpp:65-89.  `offset` / `scaling` may be None (identity)."""

    def __init__(self):
        self.data = None
        self.child = None
        self.parent_depth = None
        self.extra_data = None
        self.offset = None
        self.scaling = None
        self._weight_accum = None
        self._weight_accum_max = False
        self.child_marks = None   # optional: what mark_empty_leaves returned for this tree (no reference counterpart)
        self.child_marks_thresh = 0.0        # ... and the sigma_thresh / density_softplus it was called with
        self.child_marks_softplus = False
        self.owner = None         # optional: the N3Tree this spec was made from (its write counter)


class CameraSpec:
    """svox/csrc/include/data_spec.hpp:91-104"""

    def __init__(self):
        self.c2w = None
        self.fx = 0.0
        self.fy = 0.0
        self.width = 0
        self.height = 0


class RenderOptions:
    """svox/csrc/include/data_spec.hpp:107-126"""

    def __init__(self):
        self.step_size = 1e-3
        self.background_brightness = 1.0
        self.format = FORMAT_RGBA
        self.basis_dim = -1
        self.ndc_width = -1
        self.ndc_height = -1
        self.ndc_focal = 1.0
        self.min_comp = 0
        self.max_comp = 0
        self.sigma_thresh = 0.0
        self.stop_thresh = 0.0
        self.density_softplus = False
        self.rgb_padding = 0.0

    def _pack(self):
        return _abi.RenderOptionsC(
            float(self.step_size), float(self.background_brightness), int(self.format),
            int(self.basis_dim), int(self.ndc_width), int(self.ndc_height), float(self.ndc_focal),
            int(self.min_comp), int(self.max_comp), float(self.sigma_thresh),
            float(self.stop_thresh), int(bool(self.density_softplus)), float(self.rgb_padding))


# --------------------------------------------------------------------------------------------
# checks (CHECK_INPUT and friends, data_spec.hpp:37-42)
# --------------------------------------------------------------------------------------------
def _check_input(x, name):
    if not isinstance(x, torch.Tensor):
        raise RuntimeError(f"{name} must be a tensor")
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _numel(x):
    return 0 if x is None else x.numel()


def _dtype_code(dtype, name):
    if dtype == torch.float32:
        return _abi.SVOX_F32
    if dtype == torch.float64:
        return _abi.SVOX_F64
    raise RuntimeError(f"{name} must be a float32 or float64 tensor, got {dtype}")


def _same_dtype(x, dtype, name):
    if x.dtype != dtype:
        raise RuntimeError(f"expected scalar type {dtype} for {name} but found {x.dtype}")


def _check_tree(tree):
    """TreeSpec::check, data_spec.hpp:75-88, plus the shape facts the kernels rely on."""
    _check_input(tree.data, "data")
    _check_input(tree.child, "child")
    _check_input(tree.parent_depth, "parent_depth")
    if _numel(tree.extra_data):
        _check_input(tree.extra_data, "extra_data")
    if tree.offset is not None:
        _check_input(tree.offset, "offset")
    if tree.scaling is not None:
        _check_input(tree.scaling, "scaling")
    if _numel(tree._weight_accum):
        _check_input(tree._weight_accum, "_weight_accum")
    if tree.data.dim() != 5 or tree.child.dim() != 4 or tree.parent_depth.dim() != 2:
        raise RuntimeError("data must be 5-D, child 4-D and parent_depth 2-D")
    if tree.child.dtype != torch.int32 or tree.parent_depth.dtype != torch.int32:
        raise RuntimeError("child and parent_depth must be int32 tensors")
    if tuple(tree.data.shape[:4]) != tuple(tree.child.shape):
        raise RuntimeError("data and child disagree on (capacity, N, N, N)")


def _pack_tree(tree, dtype=None, need_data=True):
    _check_tree(tree)
    dt = tree.data.dtype if dtype is None else dtype
    code = _dtype_code(dt, "data")
    if need_data:
        _same_dtype(tree.data, dt, "data")
    spec = _abi.TreeSpecC()
    spec.data = tree.data.data_ptr()
    spec.child = tree.child.data_ptr()
    spec.parent_depth = tree.parent_depth.data_ptr()
    extra = tree.extra_data if _numel(tree.extra_data) else None
    if extra is not None:
        _same_dtype(extra, dt, "extra_data")
        if extra.dim() != 2:
            raise RuntimeError("extra_data must be 2-D")
        spec.extra_data = extra.data_ptr()
        spec.extra_rows, spec.extra_cols = int(extra.shape[0]), int(extra.shape[1])
    else:
        spec.extra_data = None
        spec.extra_rows = spec.extra_cols = 0
    for attr in ("offset", "scaling"):
        t = getattr(tree, attr)
        if t is not None:
            _same_dtype(t, dt, attr)
            if t.numel() != 3:
                raise RuntimeError(f"{attr} must have 3 elements")
            setattr(spec, attr, t.data_ptr())
        else:
            setattr(spec, attr, None)
    wa = tree._weight_accum if _numel(tree._weight_accum) else None
    if wa is not None:
        _same_dtype(wa, dt, "_weight_accum")
        if wa.numel() != tree.child.numel():
            raise RuntimeError("_weight_accum must have one entry per cell of child")
        spec.weight_accum = wa.data_ptr()
    else:
        spec.weight_accum = None
    spec.weight_accum_max = int(bool(tree._weight_accum_max))
    marks = getattr(tree, "child_marks", None)
    if marks is not None:
        _check_input(marks, "child_marks")
        if marks.dtype != torch.int32 or marks.shape != tree.child.shape:
            raise RuntimeError("child_marks must be an int32 tensor shaped like child")
        spec.child_marks = marks.data_ptr()
        spec.child_marks_thresh = float(getattr(tree, "child_marks_thresh", 0.0))
        spec.child_marks_softplus = int(bool(getattr(tree, "child_marks_softplus", False)))
    else:
        spec.child_marks = None
        spec.child_marks_thresh = 0.0
        spec.child_marks_softplus = 0
    spec.capacity = int(tree.child.shape[0])
    spec.N = int(tree.child.shape[1])
    spec.data_dim = int(tree.data.shape[4])
    spec.dtype = code
    return spec


def _check_indices(indices, name="indices"):
    """check_indices, svox_kernel.cu:34-38"""
    _check_input(indices, name)
    if indices.dim() != 2:
        raise RuntimeError(f"{name} must be 2-D")
    if not indices.is_floating_point():
        raise RuntimeError(f"{name} must be a floating point tensor")


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _call(name, *args):
    lib = _abi.load_library()
    rc = getattr(lib, name)(*args)
    if rc != _abi.SVOX_OK:
        msg = lib.svox_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"svox.{name[5:]}: {msg} ({lib.svox_status_string(rc).decode()})")


def out_data_dim(fmt, basis_dim, data_dim):
    """get_out_data_dim, rt_kernel.cu:1009-1015"""
    if fmt != FORMAT_RGBA:
        return (data_dim - 1) // basis_dim
    return data_dim - 1


# --------------------------------------------------------------------------------------------
# queries
# --------------------------------------------------------------------------------------------
def query_vertical(tree, indices):
    """(values (Q, K) like indices, node_ids (Q,) int64 on child's device); svox_kernel.cu:120-143"""
    _check_indices(indices)
    spec = _pack_tree(tree, indices.dtype)
    if indices.shape[1] != 3:
        raise RuntimeError("indices must be (Q, 3)")
    Q, K = indices.shape[0], spec.data_dim
    values = torch.empty((Q, K), dtype=indices.dtype, device=indices.device)
    node_ids = torch.empty((Q,), dtype=torch.int64, device=tree.child.device)
    with torch.cuda.device(indices.device):
        _call("svox_query_vertical", ctypes.byref(spec), indices.data_ptr(), Q, values.data_ptr(),
              node_ids.data_ptr(), _stream(indices.device))
    return values, node_ids


def query_vertical_backward(tree, indices, grad_output):
    """zeros (M, N, N, N, grad_output.shape[1]) + scatter-add; svox_kernel.cu:160-182"""
    _check_indices(indices)
    _check_indices(grad_output, "grad_output")
    _same_dtype(grad_output, indices.dtype, "grad_output")
    spec = _pack_tree(tree, indices.dtype, need_data=False)
    Q, Kg = indices.shape[0], int(grad_output.shape[1])
    if grad_output.shape[0] != Q:
        raise RuntimeError("grad_output must have one row per point")
    N = spec.N
    grad_data = torch.empty((spec.capacity, N, N, N, Kg), dtype=grad_output.dtype,
                            device=grad_output.device)
    with torch.cuda.device(indices.device):
        _call("svox_query_vertical_backward", ctypes.byref(spec), indices.data_ptr(), Q,
              grad_output.data_ptr(), Kg, grad_data.data_ptr(), 0, _stream(indices.device))
    return grad_data


def assign_vertical(tree, indices, values):
    """store values into the leaves of the points; svox_kernel.cu:145-158"""
    _check_indices(indices)
    _check_indices(values, "values")
    _same_dtype(values, indices.dtype, "values")
    spec = _pack_tree(tree, indices.dtype)
    if values.shape[0] != indices.shape[0]:
        raise RuntimeError("values must have one row per point")
    with torch.cuda.device(indices.device):
        _call("svox_assign_vertical", ctypes.byref(spec), indices.data_ptr(), indices.shape[0],
              values.data_ptr(), int(values.shape[1]), _stream(indices.device))


def calc_corners(tree, indexer):
    """(Q, 3) lower corners of the leaves [node, x, y, z]; svox_kernel.cu:184-203"""
    spec = _pack_tree(tree, need_data=False)
    _check_input(indexer, "indexer")
    if indexer.dtype != torch.int64 or indexer.dim() != 2 or indexer.shape[1] != 4:
        raise RuntimeError("indexer must be an int64 (Q, 4) tensor")
    Q = indexer.shape[0]
    out = torch.empty((Q, 3), dtype=tree.data.dtype, device=tree.data.device)
    with torch.cuda.device(indexer.device):
        _call("svox_calc_corners", ctypes.byref(spec), indexer.data_ptr(), Q, out.data_ptr(),
              _stream(indexer.device))
    return out


# --------------------------------------------------------------------------------------------
# rendering
# --------------------------------------------------------------------------------------------
def _pack_rays(rays, dtype):
    """RaysSpec::check, data_spec.hpp:56-63"""
    for name in ("origins", "dirs", "vdirs"):
        t = getattr(rays, name)
        _check_input(t, name)
        if not t.is_floating_point():
            raise RuntimeError(f"{name} must be a floating point tensor")
        _same_dtype(t, dtype, name)
        if t.dim() != 2 or t.shape[1] != 3:
            raise RuntimeError(f"{name} must be (B, 3)")
    B = rays.origins.shape[0]
    if rays.dirs.shape[0] != B or rays.vdirs.shape[0] != B:
        raise RuntimeError("origins, dirs and vdirs must have the same number of rays")
    return _abi.RaysSpecC(rays.origins.data_ptr(), rays.dirs.data_ptr(), rays.vdirs.data_ptr(), B)


def _pack_camera(cam, dtype, batched=False):
    """CameraSpec::check, data_spec.hpp:98-103.  batched: c2w is (n, 3 or 4, 4)."""
    _check_input(cam.c2w, "c2w")
    if not cam.c2w.is_floating_point():
        raise RuntimeError("c2w must be a floating point tensor")
    want = 3 if batched else 2
    if cam.c2w.dim() != want or cam.c2w.shape[-1] != 4 or cam.c2w.shape[-2] not in (3, 4):
        raise RuntimeError("c2w must be (n, 3, 4) or (n, 4, 4)" if batched else "c2w must be (3, 4) or (4, 4)")
    _same_dtype(cam.c2w, dtype, "c2w")
    return _abi.CameraSpecC(cam.c2w.data_ptr(), float(cam.fx), float(cam.fy), int(cam.width),
                            int(cam.height))


def _render_out_dim(spec, opt):
    lib = _abi.load_library()
    od = lib.svox_out_data_dim(int(opt.format), int(opt.basis_dim), spec.data_dim)
    if od < 0:
        raise RuntimeError("invalid data format / basis_dim for this tree")
    return od


def volume_render(tree, rays, opt):
    """(B, out_dim) like rays.origins; rt_kernel.cu:1019-1036"""
    spec = _pack_tree(tree, rays.origins.dtype if isinstance(rays.origins, torch.Tensor) else None)
    rspec = _pack_rays(rays, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    out = torch.empty((rspec.n_rays, od), dtype=rays.origins.dtype, device=rays.origins.device)
    copt = opt._pack()
    marks = _attach_marks(spec, tree, opt, rspec.n_rays)  # noqa: F841
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render", ctypes.byref(spec), ctypes.byref(rspec), ctypes.byref(copt),
              out.data_ptr(), _stream(tree.data.device))
    return out


def volume_render_image(tree, cam, opt):
    """(H, W, out_dim) like tree.data; rt_kernel.cu:1038-1057"""
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    out = torch.empty((cspec.height, cspec.width, od), dtype=tree.data.dtype, device=tree.data.device)
    copt = opt._pack()
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_image", ctypes.byref(spec), ctypes.byref(cspec),
              ctypes.byref(copt), out.data_ptr(), _stream(tree.data.device))
    return out


# A render call (forward, noted forward or marching backward) with at least this many rays per cell of
# the tree marks the empty leaves first, for this call only (mark_empty_leaves costs about 24 ps per cell, passing through an
# empty leaf unread saves about 40 ps per ray on a sparse scene).  None: never.
AUTO_MARK_RAYS_PER_CELL = 0.7
# ... and at least this many rays: marks save memory traffic, which a launch that does not fill the GPU is
# not short of, while making them costs a small call a sixth of its time on the host (4096 rays on a 16^3
# tree: 72 -> 59 us per call).  Measured at 2.5 M rays and more, marking pays from 37 k cells to 6 M.
AUTO_MARK_MIN_RAYS = 1 << 18


def _marks_for_this_call(tree, opt, n_rays, every_positive_leaf=False):
    """Marks made for one large launch, or None where they would not pay or would not be used (the fp32
    octree kernels read them, and only for sigma_thresh >= 0).  A forward launch gets marks made with its own
    sigma_thresh (every leaf they let through is shaded); every_positive_leaf: the launch works on every leaf with
    density > 0 whatever the threshold (noting forward passes, backward passes), so the marks are made with 0."""
    if AUTO_MARK_RAYS_PER_CELL is None or getattr(tree, "child_marks", None) is not None:
        return None
    if tree.data.dtype != torch.float32 or tree.child.shape[1] != 2:
        return None
    if not opt.sigma_thresh >= 0 or n_rays < max(AUTO_MARK_MIN_RAYS, AUTO_MARK_RAYS_PER_CELL * tree.child.numel()):
        return None
    thresh = 0.0 if every_positive_leaf else float(opt.sigma_thresh)
    if opt.density_softplus and thresh <= 0.0:
        return None          # (the softplus of any stored density is > 0: nothing to mark)
    return mark_empty_leaves(tree, thresh, bool(opt.density_softplus)), thresh


def _attach_marks(spec, tree, opt, n_rays, every_positive_leaf=False):
    """Points the packed `spec` to marks made for this call, where they pay; returns the tensor,
    which the caller keeps until its launch is queued."""
    made = _marks_for_this_call(tree, opt, n_rays, every_positive_leaf)
    if made is None:
        return None
    marks, thresh = made
    spec.child_marks = marks.data_ptr()
    spec.child_marks_thresh = thresh
    spec.child_marks_softplus = int(bool(opt.density_softplus))
    return marks


def volume_render_images(tree, cam, opt):
    """(n, H, W, out_dim): n images in one launch; cam.c2w is (n, 3, 4) or (n, 4, 4).
    No counterpart in the reference, whose extension renders one image per call."""
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype, batched=True)
    n, stride = int(cam.c2w.shape[0]), int(cam.c2w.shape[1]) * 4
    od = _render_out_dim(spec, opt)
    out = torch.empty((n, cspec.height, cspec.width, od), dtype=tree.data.dtype, device=tree.data.device)
    copt = opt._pack()
    marks = _attach_marks(spec, tree, opt, n * cspec.height * cspec.width)  # noqa: F841 (kept alive for the launch)
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_images", ctypes.byref(spec), ctypes.byref(cspec), n, stride,
              ctypes.byref(copt), out.data_ptr(), _stream(tree.data.device))
    return out


def volume_render_images_backward(tree, cam, opt, grad_output, workspace=True):
    """zeros_like(tree.data) + scatter for volume_render_images (workspace: see volume_render_backward)."""
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype, batched=True)
    n, stride = int(cam.c2w.shape[0]), int(cam.c2w.shape[1]) * 4
    od = _render_out_dim(spec, opt)
    _check_grad(grad_output, (n, cspec.height, cspec.width, od), tree.data.dtype)
    grad = torch.empty_like(tree.data)
    copt = opt._pack()
    ws, ws_bytes = _backward_workspace(tree, n * cspec.height * cspec.width) if workspace else (None, 0)
    marks = _attach_marks(spec, tree, opt, n * cspec.height * cspec.width, True)  # noqa: F841
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_images_backward_ws", ctypes.byref(spec), ctypes.byref(cspec), n, stride,
              ctypes.byref(copt), grad_output.data_ptr(), grad.data_ptr(), 0,
              ws.data_ptr() if ws is not None else None, ws_bytes, _stream(tree.data.device))
    return grad


def volume_render_images_noted(tree, cam, opt, records_per_ray=None):
    """(images, notes): volume_render_images that also leaves the notes
    volume_render_images_backward_noted works from (see volume_render_noted).  cam.c2w is
    (n, 3, 4) / (n, 4, 4), or one pose (3, 4) / (4, 4), which gives (H, W, out_dim)."""
    single = cam.c2w.dim() == 2
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype, batched=not single)
    n, stride = (1, 12) if single else (int(cam.c2w.shape[0]), int(cam.c2w.shape[1]) * 4)
    od = _render_out_dim(spec, opt)
    shape = (cspec.height, cspec.width, od) if single else (n, cspec.height, cspec.width, od)
    out = torch.empty(shape, dtype=tree.data.dtype, device=tree.data.device)
    copt = opt._pack()
    ws, ws_bytes = _notes_workspace(tree, spec, copt, n * cspec.height * cspec.width, records_per_ray)
    marks = _attach_marks(spec, tree, opt, n * cspec.height * cspec.width, ws is not None)  # noqa: F841
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_images_noted", ctypes.byref(spec), ctypes.byref(cspec), n, stride,
              ctypes.byref(copt), out.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes,
              _stream(tree.data.device))
    return out, ws


def volume_render_images_backward_noted(tree, cam, opt, grad_output, notes):
    """The gradient of volume_render_images_noted's picture(s) from its notes (notes None: by marching)."""
    single = cam.c2w.dim() == 2
    if notes is None:
        fn = volume_render_image_backward if single else volume_render_images_backward
        return fn(tree, cam, opt, grad_output)
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype, batched=not single)
    n, stride = (1, 12) if single else (int(cam.c2w.shape[0]), int(cam.c2w.shape[1]) * 4)
    od = _render_out_dim(spec, opt)
    shape = (cspec.height, cspec.width, od) if single else (n, cspec.height, cspec.width, od)
    _check_grad(grad_output, shape, tree.data.dtype)
    grad = torch.empty_like(tree.data)
    copt = opt._pack()
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_images_backward_noted", ctypes.byref(spec), ctypes.byref(cspec), n, stride,
              ctypes.byref(copt), grad_output.data_ptr(), grad.data_ptr(), 0, notes.data_ptr(),
              notes.numel() * notes.element_size(), _stream(tree.data.device))
    return grad


def _check_grad(grad_output, shape, dtype):
    _check_input(grad_output, "grad_output")
    _same_dtype(grad_output, dtype, "grad_output")
    if tuple(grad_output.shape) != tuple(shape):
        raise RuntimeError(f"grad_output must have shape {tuple(shape)}, got {tuple(grad_output.shape)}")


# Leaves per ray (on average) the backward's workspace has room for, and the most memory it may take:
# BACKWARD_WORKSPACE_LIMIT bytes, and of what is free on the device at the time (memory torch holds
# in its cache counted as free) no more than BACKWARD_WORKSPACE_FREE_FRACTION.
BACKWARD_RECORDS_PER_RAY = 30
# Batches of fewer than 2^20 rays get up to four times that room per ray (the workspace stays below what
# 2^20 rays take, 768 MiB): a launch lasts as long as its longest ray, so the few rays of a small batch whose
# notes do not fit cost their backward pass a whole march (4 096 rays through a dense 16^3 tree, 26 of them
# without room: 213 us instead of 55).
SMALL_BATCH_ROOM = 4
BACKWARD_WORKSPACE_LIMIT = 4 << 30
BACKWARD_WORKSPACE_FREE_FRACTION = 0.25
_ASK_DEVICE_ABOVE = 64 << 20   # smaller workspaces are taken without asking the device what is free


def _backward_workspace(tree, n_rays, records_per_ray=None):
    """(tensor, bytes) of the backward's workspace for n_rays rays, or (None, 0): for a tree that is
    not fp32, where the limits leave no room for 15 leaves per ray, and where the allocation fails
    (the caller then runs without a workspace: same results, more marching).  records_per_ray: room
    for that many leaves per ray on average (default BACKWARD_RECORDS_PER_RAY), as far as the limits
    allow."""
    if n_rays <= 0 or tree.data.dtype != torch.float32:
        return None, 0
    size_of = _abi.load_library().svox_volume_render_backward_workspace_bytes
    per_ray = int(BACKWARD_RECORDS_PER_RAY if records_per_ray is None else records_per_ray)
    per_ray *= max(1, min(int(SMALL_BATCH_ROOM), (1 << 20) // int(n_rays)))
    limit = BACKWARD_WORKSPACE_LIMIT
    if size_of(n_rays, per_ray) > _ASK_DEVICE_ABOVE:
        device = tree.data.device
        free, _ = torch.cuda.mem_get_info(device)
        cached = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
        limit = min(limit, int((free + cached) * BACKWARD_WORKSPACE_FREE_FRACTION))
    while per_ray > 0 and size_of(n_rays, per_ray) > limit:
        per_ray -= 15
    nbytes = int(size_of(n_rays, per_ray)) if per_ray > 0 else 0
    if nbytes <= 0:
        return None, 0
    try:
        return torch.empty(nbytes // 8, dtype=torch.float64, device=tree.data.device), nbytes
    except torch.cuda.OutOfMemoryError:
        return None, 0


def _notes_workspace(tree, spec, copt, n_rays, records_per_ray=None):
    """_backward_workspace for the notes of a forward pass: (None, 0) also where the library would take no notes
    for this tree under these options (svox_notes_serve: the one-ray-per-lane kernels, a weight accumulator, a
    negative sigma_thresh) -- the pass then runs as the plain forward pass and its caller keeps nothing."""
    if _abi.load_library().svox_notes_serve(ctypes.byref(spec), ctypes.byref(copt)) != 1:
        return None, 0
    return _backward_workspace(tree, n_rays, records_per_ray)


def volume_render_backward(tree, rays, opt, grad_output, workspace=True):
    """zeros_like(tree.data) + scatter; rt_kernel.cu:1059-1083.

    workspace: let the kernel note, during the first march, the leaves the second march needs, so
    that a ray whose notes fit is marched once (fp32 octrees; room for BACKWARD_RECORDS_PER_RAY
    leaves per ray on average, at most BACKWARD_WORKSPACE_LIMIT bytes, from torch's allocator).
    The gradient is the same."""
    spec = _pack_tree(tree)
    rspec = _pack_rays(rays, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    _check_grad(grad_output, (rspec.n_rays, od), tree.data.dtype)
    grad = torch.empty_like(tree.data)
    copt = opt._pack()
    ws, ws_bytes = _backward_workspace(tree, rspec.n_rays) if workspace else (None, 0)
    marks = _attach_marks(spec, tree, opt, rspec.n_rays, True)  # noqa: F841
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_backward_ws", ctypes.byref(spec), ctypes.byref(rspec),
              ctypes.byref(copt), grad_output.data_ptr(), grad.data_ptr(), 0,
              ws.data_ptr() if ws is not None else None, ws_bytes, _stream(tree.data.device))
    return grad


def volume_render_backward_static(tree, rays, opt, grad_output, grad_data_out, accumulate=False):
    """volume_render_backward into the caller's `grad_data_out` (shaped like tree.data) with the
    library's own fixed workspace: nothing is allocated on the way, by torch or by the library, so the
    call can be recorded into a HIP graph.  At most _abi.STATIC_RAYS_MAX rays per call.  Calls that
    overlap in time on one GPU race on the shared workspace.  No counterpart in the reference."""
    spec = _pack_tree(tree)
    rspec = _pack_rays(rays, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    _check_grad(grad_output, (rspec.n_rays, od), tree.data.dtype)
    _check_input(grad_data_out, "grad_data_out")
    _same_dtype(grad_data_out, tree.data.dtype, "grad_data_out")
    if tuple(grad_data_out.shape) != tuple(tree.data.shape):
        raise RuntimeError("grad_data_out must have the shape of tree.data")
    # (the library's workspace is looked up for the current device, which is set from tree.data below)
    for name, x in (("grad_output", grad_output), ("grad_data_out", grad_data_out), ("rays.origins", rays.origins),
                    ("rays.dirs", rays.dirs), ("rays.vdirs", rays.vdirs), ("child", tree.child)):
        if x.device != tree.data.device:
            raise RuntimeError(f"{name} must be on the device of tree.data ({tree.data.device}), got {x.device}")
    copt = opt._pack()
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_backward_static", ctypes.byref(spec), ctypes.byref(rspec), ctypes.byref(copt),
              grad_output.data_ptr(), grad_data_out.data_ptr(), int(bool(accumulate)), _stream(tree.data.device))
    return grad_data_out


def notes_pool_use(notes, n_rays):
    """(counter, pool) of the notes a noted forward pass left for n_rays rays: `counter` is a
    one-element int64 view into `notes` (on the device) that holds how many 64-chunk stocks the pass
    asked for beyond the rays' own chunks, `pool` how many the workspace had.  counter >= pool: the
    workspace ran out and some rays will be marched by the backward pass."""
    offset, pool = ctypes.c_int64(0), ctypes.c_int64(0)
    _call("svox_notes_pool_info", int(n_rays), notes.numel() * notes.element_size(), ctypes.byref(offset),
          ctypes.byref(pool))
    return notes.view(torch.int64)[offset.value // 8: offset.value // 8 + 1], int(pool.value)


def volume_render_noted(tree, rays, opt, records_per_ray=None):
    """(out, notes): volume_render, which in the same march leaves in `notes` (a workspace tensor, or
    None where the library cannot take notes) what volume_render_backward_noted needs of the rays.
    records_per_ray: room for that many leaves per ray on average (default BACKWARD_RECORDS_PER_RAY).
    No counterpart in the reference: it is what an autograd function keeps between forward and
    backward."""
    spec = _pack_tree(tree, rays.origins.dtype if isinstance(rays.origins, torch.Tensor) else None)
    rspec = _pack_rays(rays, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    out = torch.empty((rspec.n_rays, od), dtype=rays.origins.dtype, device=rays.origins.device)
    copt = opt._pack()
    ws, ws_bytes = _notes_workspace(tree, spec, copt, rspec.n_rays, records_per_ray)
    marks = _attach_marks(spec, tree, opt, rspec.n_rays, ws is not None)  # noqa: F841
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_noted", ctypes.byref(spec), ctypes.byref(rspec), ctypes.byref(copt),
              out.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes, _stream(tree.data.device))
    return out, ws


def volume_render_backward_noted(tree, rays, opt, grad_output, notes):
    """volume_render_backward from the notes volume_render_noted left for the same tree, rays and
    options (notes None: volume_render_backward).  tree.data must not have changed in between."""
    if notes is None:
        return volume_render_backward(tree, rays, opt, grad_output)
    spec = _pack_tree(tree)
    rspec = _pack_rays(rays, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    _check_grad(grad_output, (rspec.n_rays, od), tree.data.dtype)
    grad = torch.empty_like(tree.data)
    copt = opt._pack()
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_backward_noted", ctypes.byref(spec), ctypes.byref(rspec), ctypes.byref(copt),
              grad_output.data_ptr(), grad.data_ptr(), 0, notes.data_ptr(), notes.numel() * notes.element_size(),
              _stream(tree.data.device))
    return grad


def volume_render_image_backward(tree, cam, opt, grad_output, workspace=True):
    """zeros_like(tree.data) + scatter; rt_kernel.cu:1085-1109 (workspace: see volume_render_backward)"""
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype)
    od = _render_out_dim(spec, opt)
    _check_grad(grad_output, (cspec.height, cspec.width, od), tree.data.dtype)
    grad = torch.empty_like(tree.data)
    copt = opt._pack()
    ws, ws_bytes = _backward_workspace(tree, cspec.height * cspec.width) if workspace else (None, 0)
    with torch.cuda.device(tree.data.device):
        _call("svox_volume_render_images_backward_ws", ctypes.byref(spec), ctypes.byref(cspec), 1, 12,
              ctypes.byref(copt), grad_output.data_ptr(), grad.data_ptr(), 0,
              ws.data_ptr() if ws is not None else None, ws_bytes, _stream(tree.data.device))
    return grad


def _check_color(color, shape, dtype):
    _check_input(color, "color")
    _same_dtype(color, dtype, "color")
    if tuple(color.shape) != tuple(shape):
        raise RuntimeError(f"color must have shape {tuple(shape)}, got {tuple(color.shape)}")


def _se_out_dim(spec, opt):
    od = _render_out_dim(spec, opt)
    if od > 4:
        raise RuntimeError("Tree's output dim cannot be > 4 for se_grad")   # rt_kernel.cu:1123-1125
    return od


def se_grad(tree, rays, color, opt, workspace=True):
    """(result (B, C), grad, hessdiag) of 0.5 * |render - color|^2, grad and hessdiag like tree.data;
    svox.cpp:115, rt_kernel.cu:1111-1139.  Argument order as in the reference: color before opt.
    With `workspace` (default) the rays are marched once and their notes used for the rest
    (svox_se_grad_ws); without, the rays are marched twice."""
    spec = _pack_tree(tree)
    rspec = _pack_rays(rays, tree.data.dtype)
    od = _se_out_dim(spec, opt)
    _check_color(color, (rspec.n_rays, od), tree.data.dtype)
    result = torch.empty((rspec.n_rays, od), dtype=tree.data.dtype, device=tree.data.device)
    grad = torch.empty_like(tree.data)
    hessdiag = torch.empty_like(tree.data)
    copt = opt._pack()
    ws, ws_bytes = _backward_workspace(tree, rspec.n_rays) if workspace else (None, 0)
    with torch.cuda.device(tree.data.device):
        _call("svox_se_grad_ws", ctypes.byref(spec), ctypes.byref(rspec), ctypes.byref(copt), color.data_ptr(),
              result.data_ptr(), grad.data_ptr(), hessdiag.data_ptr(), ws.data_ptr() if ws is not None else None,
              ws_bytes, _stream(tree.data.device))
    return result, grad, hessdiag


def se_grad_persp(tree, cam, opt, color, workspace=True):
    """Image version: color and result are (H, W, C); svox.cpp:116, rt_kernel.cu:1141-1173.
    Argument order as in the reference: opt before color.  `workspace` as in se_grad."""
    spec = _pack_tree(tree)
    cspec = _pack_camera(cam, tree.data.dtype)
    od = _se_out_dim(spec, opt)
    _check_color(color, (cspec.height, cspec.width, od), tree.data.dtype)
    result = torch.empty((cspec.height, cspec.width, od), dtype=tree.data.dtype, device=tree.data.device)
    grad = torch.empty_like(tree.data)
    hessdiag = torch.empty_like(tree.data)
    copt = opt._pack()
    ws, ws_bytes = _backward_workspace(tree, cspec.height * cspec.width) if workspace else (None, 0)
    with torch.cuda.device(tree.data.device):
        _call("svox_se_grad_image_ws", ctypes.byref(spec), ctypes.byref(cspec), ctypes.byref(copt),
              color.data_ptr(), result.data_ptr(), grad.data_ptr(), hessdiag.data_ptr(),
              ws.data_ptr() if ws is not None else None, ws_bytes, _stream(tree.data.device))
    return result, grad, hessdiag


def mark_empty_leaves(tree, sigma_thresh=0.0, density_softplus=False):
    """An int32 tensor shaped like tree.child: child with SVOX_EMPTY_LEAF (-2) in every leaf cell whose
    density (after the shifted softplus, with density_softplus) is not > sigma_thresh (no reference counterpart).
    Set as TreeSpec.child_marks -- with child_marks_thresh / child_marks_softplus saying how it was made -- it lets
    the render operators pass through such leaves without reading their density; a forward render with the same
    sigma_thresh then shades every leaf the marks let through and reads its density with its coefficients.  Calls
    that need leaves the marks hide leave them aside; results are bit-identical.
    It describes the tree as it is now: make it again, or leave it out, after a write to the
    densities or the structure."""
    spec = _pack_tree(tree)
    marks = torch.empty_like(tree.child)
    with torch.cuda.device(tree.data.device):
        _call("svox_mark_leaves_below", ctypes.byref(spec), float(sigma_thresh), int(bool(density_softplus)),
              marks.data_ptr(), _stream(tree.data.device))
    return marks


def grid_weight_render(data, cam, opt, offset, scaling):
    """[grid_weight, grid_hit], both zeros_like(data) + per-cell max weight / visit count of one
    camera's rays through the dense (reso, reso, reso) density grid `data`; svox.cpp:120,
    rt_kernel.cu:1174-1203."""
    _check_input(data, "data")
    if not data.is_floating_point():
        raise RuntimeError("data must be a floating point tensor")
    if data.dim() != 3 or not (data.shape[0] == data.shape[1] == data.shape[2]):
        raise RuntimeError("data must be a cubic (reso, reso, reso) grid")
    for name, x in (("offset", offset), ("scaling", scaling)):
        _check_input(x, name)
        _same_dtype(x, data.dtype, name)
        if x.numel() != 3:
            raise RuntimeError(f"{name} must have 3 elements")
    cspec = _pack_camera(cam, data.dtype)
    grid_weight = torch.empty_like(data)
    grid_hit = torch.empty_like(data)
    copt = opt._pack()
    with torch.cuda.device(data.device):
        _call("svox_grid_weight_render", data.data_ptr(), int(data.shape[0]),
              _abi.SVOX_F32 if data.dtype == torch.float32 else _abi.SVOX_F64, ctypes.byref(cspec),
              ctypes.byref(copt), offset.data_ptr(), scaling.data_ptr(), grid_weight.data_ptr(),
              grid_hit.data_ptr(), _stream(data.device))
    return [grid_weight, grid_hit]


def volume_render_stats(tree, rays_or_cam, opt):
    """Visit counts of one launch (dict); `rays_or_cam` is a RaysSpec or a CameraSpec."""
    spec = _pack_tree(tree)
    copt = opt._pack()
    counters = torch.zeros(8, dtype=torch.int64, device=tree.data.device)
    with torch.cuda.device(tree.data.device):
        if isinstance(rays_or_cam, RaysSpec):
            rspec = _pack_rays(rays_or_cam, tree.data.dtype)
            _call("svox_volume_render_stats", ctypes.byref(spec), ctypes.byref(rspec), None,
                  ctypes.byref(copt), counters.data_ptr(), _stream(tree.data.device))
        else:
            cspec = _pack_camera(rays_or_cam, tree.data.dtype)
            _call("svox_volume_render_stats", ctypes.byref(spec), None, ctypes.byref(cspec),
                  ctypes.byref(copt), counters.data_ptr(), _stream(tree.data.device))
    vals = counters.cpu().tolist()
    names = [f[0] for f in _abi.MarchStatsC._fields_]
    return {n: int(v) for n, v in zip(names, vals)}


def octree_kernels_serve(tree, opt):
    """True where the wavefront-per-tile kernels serve the render calls of `tree` under `opt` (forward, backward,
    se_grad, with or without density_softplus, any branching factor, any range of components), False where the
    one-ray-per-lane kernels do (fp64, other basis sizes and record shapes)."""
    spec = _pack_tree(tree)
    copt = opt._pack()
    rc = _abi.load_library().svox_octree_kernels_serve(ctypes.byref(spec), ctypes.byref(copt))
    if rc < 0:
        lib = _abi.load_library()
        raise RuntimeError(f"svox.octree_kernels_serve: {lib.svox_last_error().decode('utf-8', 'replace')}")
    return bool(rc)


def give_up_count():
    """How many wavefronts of the two-wavefront forward kernel have given up a bounded wait since the library was
    loaded (0 unless something is badly wrong; their pixels are NaN and their rays' notes say "march me").
    Waits for the device."""
    n = ctypes.c_int64(0)
    _call("svox_give_up_count", ctypes.byref(n))
    return int(n.value)


def set_debug_flags(flags):
    """Of the calling thread.  bit 0: route every call to the generic kernels; bit 1: small ray batches run like
    large ones; bit 2 / bit 3: forward renders never / always take the two-wavefront kernel; bit 4: the bounded
    waits of that kernel give up at the first look that finds nothing (tests of what a give-up leaves behind)"""
    _abi.load_library().svox_set_debug_flags(int(flags))
