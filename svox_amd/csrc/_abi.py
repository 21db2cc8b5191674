"""ctypes mirror of include/svox_hip.h and the loader of libsvox_hip.so.

The structures below must stay field-for-field identical to the C header; tests compare their
sizes and the exported symbol list against the header text.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsvox_hip.so")

SVOX_OK = 0
SVOX_F32, SVOX_F64 = 0, 1
FORMAT_RGBA, FORMAT_SH, FORMAT_SG, FORMAT_ASG = 0, 1, 2, 3
MAX_BASIS_DIM = 25
MAX_OUT_DIM = 16
STATIC_RAYS_MAX = 65536   # SVOX_STATIC_RAYS_MAX

c_void_p = ctypes.c_void_p
c_int32 = ctypes.c_int32
c_int64 = ctypes.c_int64
c_float = ctypes.c_float


ABI_VERSION = 3   # SVOX_ABI_VERSION of include/svox_hip.h: the struct layouts below


class TreeSpecC(ctypes.Structure):
    _fields_ = [
        ("data", c_void_p),
        ("child", c_void_p),
        ("parent_depth", c_void_p),
        ("extra_data", c_void_p),
        ("offset", c_void_p),
        ("scaling", c_void_p),
        ("weight_accum", c_void_p),
        ("capacity", c_int64),
        ("N", c_int32),
        ("data_dim", c_int32),
        ("extra_rows", c_int32),
        ("extra_cols", c_int32),
        ("weight_accum_max", c_int32),
        ("dtype", c_int32),
        ("child_marks", c_void_p),
        ("child_marks_thresh", c_float),
        ("child_marks_softplus", c_int32),
    ]


class RaysSpecC(ctypes.Structure):
    _fields_ = [
        ("origins", c_void_p),
        ("dirs", c_void_p),
        ("vdirs", c_void_p),
        ("n_rays", c_int64),
    ]


class CameraSpecC(ctypes.Structure):
    _fields_ = [
        ("c2w", c_void_p),
        ("fx", c_float),
        ("fy", c_float),
        ("width", c_int32),
        ("height", c_int32),
    ]


class RenderOptionsC(ctypes.Structure):
    _fields_ = [
        ("step_size", c_float),
        ("background_brightness", c_float),
        ("format", c_int32),
        ("basis_dim", c_int32),
        ("ndc_width", c_int32),
        ("ndc_height", c_int32),
        ("ndc_focal", c_float),
        ("min_comp", c_int32),
        ("max_comp", c_int32),
        ("sigma_thresh", c_float),
        ("stop_thresh", c_float),
        ("density_softplus", c_int32),
        ("rgb_padding", c_float),
    ]


class MarchStatsC(ctypes.Structure):
    _fields_ = [
        ("rays", ctypes.c_uint64),
        ("rays_hit", ctypes.c_uint64),
        ("samples", ctypes.c_uint64),
        ("samples_shaded", ctypes.c_uint64),
        ("samples_bwd", ctypes.c_uint64),
        ("samples_bwd_pos", ctypes.c_uint64),
        ("levels", ctypes.c_uint64),
        ("samples_tail", ctypes.c_uint64),
    ]

    def as_dict(self):
        return {name: int(getattr(self, name)) for name, _ in self._fields_}


P = ctypes.POINTER

# name -> (restype, argtypes); the entry points of include/svox_hip.h
SIGNATURES = {
    "svox_abi_version": (ctypes.c_int, []),
    "svox_last_error": (ctypes.c_char_p, []),
    "svox_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "svox_set_debug_flags": (None, [ctypes.c_int]),
    "svox_out_data_dim": (ctypes.c_int, [c_int32, c_int32, c_int32]),
    "svox_query_vertical": (ctypes.c_int, [P(TreeSpecC), c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "svox_query_vertical_backward": (
        ctypes.c_int, [P(TreeSpecC), c_void_p, c_int64, c_void_p, c_int32, c_void_p, c_int32, c_void_p]),
    "svox_assign_vertical": (ctypes.c_int, [P(TreeSpecC), c_void_p, c_int64, c_void_p, c_int32, c_void_p]),
    "svox_calc_corners": (ctypes.c_int, [P(TreeSpecC), c_void_p, c_int64, c_void_p, c_void_p]),
    "svox_volume_render": (ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p]),
    "svox_volume_render_image": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), P(RenderOptionsC), c_void_p, c_void_p]),
    "svox_volume_render_images": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), c_int32, c_int64, P(RenderOptionsC), c_void_p, c_void_p]),
    "svox_volume_render_images_backward": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), c_int32, c_int64, P(RenderOptionsC), c_void_p, c_void_p,
                       c_int32, c_void_p]),
    "svox_volume_render_backward": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_int32, c_void_p]),
    "svox_volume_render_backward_ws": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_int32, c_void_p, c_int64,
                       c_void_p]),
    "svox_volume_render_backward_static": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_int32, c_void_p]),
    "svox_volume_render_backward_workspace_bytes": (c_int64, [c_int64, c_int32]),
    "svox_notes_pool_info": (ctypes.c_int, [c_int64, c_int64, P(c_int64), P(c_int64)]),
    "svox_octree_kernels_serve": (ctypes.c_int, [P(TreeSpecC), P(RenderOptionsC)]),
    "svox_volume_render_noted": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_int64, c_void_p]),
    "svox_volume_render_backward_noted": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_int32, c_void_p, c_int64,
                       c_void_p]),
    "svox_volume_render_images_noted": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), c_int32, c_int64, P(RenderOptionsC), c_void_p, c_void_p, c_int64,
                       c_void_p]),
    "svox_volume_render_images_backward_noted": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), c_int32, c_int64, P(RenderOptionsC), c_void_p, c_void_p, c_int32,
                       c_void_p, c_int64, c_void_p]),
    "svox_volume_render_images_backward_ws": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), c_int32, c_int64, P(RenderOptionsC), c_void_p, c_void_p, c_int32,
                       c_void_p, c_int64, c_void_p]),
    "svox_volume_render_image_backward": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_int32, c_void_p]),
    "svox_se_grad": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_void_p, c_void_p,
                       c_void_p]),
    "svox_se_grad_image": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_void_p, c_void_p,
                       c_void_p]),
    "svox_se_grad_ws": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_void_p, c_void_p,
                       c_void_p, c_int64, c_void_p]),
    "svox_se_grad_image_ws": (
        ctypes.c_int, [P(TreeSpecC), P(CameraSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_void_p, c_void_p,
                       c_void_p, c_int64, c_void_p]),
    "svox_mark_empty_leaves": (ctypes.c_int, [P(TreeSpecC), c_void_p, c_void_p]),
    "svox_mark_leaves_below": (ctypes.c_int, [P(TreeSpecC), c_float, c_int32, c_void_p, c_void_p]),
    "svox_notes_serve": (ctypes.c_int, [P(TreeSpecC), P(RenderOptionsC)]),
    "svox_give_up_count": (ctypes.c_int, [P(c_int64)]),
    "svox_grid_weight_render": (
        ctypes.c_int, [c_void_p, c_int32, c_int32, P(CameraSpecC), P(RenderOptionsC), c_void_p, c_void_p, c_void_p,
                       c_void_p, c_void_p]),
    "svox_volume_render_stats": (
        ctypes.c_int, [P(TreeSpecC), P(RaysSpecC), P(CameraSpecC), P(RenderOptionsC), c_void_p, c_void_p]),
}

_lib = None


def load_library(path=None):
    """Load libsvox_hip.so (once) and bind the argument types.  Raises if it is not built.

    torch must already be imported: the library's libamdhip64 dependency then resolves to the HIP
    runtime torch has loaded, so both share one runtime and one set of device pointers.
    """
    global _lib
    if _lib is not None and path is None:
        return _lib
    import torch  # noqa: F401  (loads the HIP runtime the library binds to)

    lib_path = path or LIB_PATH
    if not os.path.exists(lib_path):
        raise RuntimeError(
            f"{lib_path} is missing: the HIP extension has not been built "
            "(run `python -m svox_amd.csrc.build`); there is no CPU fallback")
    lib = ctypes.CDLL(lib_path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            raise RuntimeError(f"{lib_path} does not export {name}: it was built from other sources, build it again")
        fn.restype = restype
        fn.argtypes = argtypes
    if path is None and lib.svox_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{lib_path} has ABI version {lib.svox_abi_version()}, this package expects "
                           f"{ABI_VERSION}: build it again")
    if path is None:
        _lib = lib
    return lib


def library_loaded():
    return _lib is not None
