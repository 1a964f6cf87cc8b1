"""ctypes mirror of include/vetrast.h and the loader of vet_amd/lib/libvetrast.so.

The library is never built implicitly and there is no fallback: if the shared object is missing, loading raises.
"""
import ctypes as C
import os

MAX_LAYERS = 5
MAX_CHANNELS = 4

OK = 0
ERR_INVALID_ARG = -1
ERR_WORKSPACE_SMALL = -2
ERR_HIP = -3
ERR_UNSUPPORTED = -4
ERR_BAD_INPUT_DATA = -5
ERR_TOO_LARGE = -6

CAMERA_PINHOLE_DISTORTION = 0
CAMERA_OCAM = 1
CAMERA_SPHERICAL = 2

RENDER_FULL_BLEND = 1
RENDER_FUZZY_BLEND = 2
RENDER_BILINEAR_BLEND = 3

SCOPE_NAMES = [
    "PREPARE", "PACK", "COUNT", "SCAN", "FILL", "BUILD", "BACKWARD_PREPARE", "BACKWARD_BLEND", "BACKWARD_GATHER", "BACKWARD_POST",
    "LIFT_ERROR",
]
SCOPE_COUNT = len(SCOPE_NAMES)


class View(C.Structure):
    _fields_ = [
        ("w", C.c_int32), ("h", C.c_int32),
        ("image_index", C.c_int32), ("camera_index", C.c_int32), ("camera_model_type", C.c_int32),
        ("crop_transform", C.c_float * 5),
        ("crop_rotation", C.c_float * 4),
    ]


class Params(C.Structure):
    _fields_ = [
        ("num_texture_channels", C.c_int32),
        ("num_layers", C.c_int32),
        ("debug_max_list_length", C.c_int32),
        ("use_environment_map", C.c_int32),
        ("need_point_gradient", C.c_int32),
        ("viewer_only", C.c_int32),
        ("stability_cutoff_value", C.c_float),
        ("drop_out_points_by_radius", C.c_int32),
        ("drop_out_radius_threshold", C.c_float),
        ("output_background_mask", C.c_int32),
        ("output_background_mask_value", C.c_float),
        ("check_normal", C.c_int32),
        ("quirk_background_confidence_leak", C.c_int32),
        ("point_gradient_normalization", C.c_int32),
        ("K_gradient_factor", C.c_float),
        ("camera_gradient_normalization", C.c_int32),
        ("render_mode", C.c_int32),
        ("confidence_activation", C.c_int32),
        ("confidence_scale", C.c_float),
        ("texture_abs", C.c_int32),
        ("depth_accept_blend", C.c_float),
        ("expected_fragments", C.c_float * MAX_LAYERS),
        ("allow_distortion", C.c_int32),
        ("distortion_gradient_factor", C.c_float),
    ]


class WorkspaceLayout(C.Structure):
    _fields_ = [
        ("layer_w", C.c_int32 * MAX_LAYERS),
        ("layer_h", C.c_int32 * MAX_LAYERS),
        ("layer_tiles_x", C.c_int32 * MAX_LAYERS),
        ("reserved0", C.c_int32),
        ("layer_tile_base", C.c_int64 * (MAX_LAYERS + 1)),
        ("layer_pixel_base", C.c_int64 * (MAX_LAYERS + 1)),
        ("fragment_capacity", C.c_int64),
        ("hits_per_layer", C.c_int32),
        ("reserved1", C.c_int32),
        ("total_bytes", C.c_size_t),
        ("offsets_base", C.c_size_t), ("offsets_stride", C.c_size_t),
        ("fragments_base", C.c_size_t), ("fragments_stride", C.c_size_t),
        ("transmittance_base", C.c_size_t), ("transmittance_stride", C.c_size_t),
        ("weight_base", C.c_size_t), ("weight_stride", C.c_size_t),
        ("kept_base", C.c_size_t), ("kept_stride", C.c_size_t),
        ("cut_flags_base", C.c_size_t), ("cut_flags_stride", C.c_size_t),
        ("packed_base", C.c_size_t),
        ("slots_base", C.c_size_t),
        ("views_base", C.c_size_t),
        ("scan_partials_base", C.c_size_t),
        ("num_bins", C.c_int64),
        ("bin_counts_base", C.c_size_t), ("bin_counts_stride", C.c_size_t),
        ("binned_base", C.c_size_t),
        ("flags_base", C.c_size_t),
        ("forward_only_bytes", C.c_size_t),
        ("partial_base", C.c_size_t),
        ("background_partial_base", C.c_size_t),
        ("camera_partial_base", C.c_size_t),
        ("primary_base", C.c_size_t), ("log_base", C.c_size_t), ("log_cursor_base", C.c_size_t),
        ("last_key_base", C.c_size_t), ("last_key_stride", C.c_size_t),
        ("projected_base", C.c_size_t), ("projected_stride", C.c_size_t),
        ("view_lanes", C.c_int32), ("reserved2", C.c_int32),
        ("binned_stride", C.c_size_t), ("primary_stride", C.c_size_t), ("scan_partials_stride", C.c_size_t),
        ("lane_scratch_stride", C.c_size_t),
    ]


class AdamArgs(C.Structure):
    _fields_ = [
        ("param", C.c_void_p), ("grad", C.c_void_p), ("exp_avg", C.c_void_p), ("exp_avg_sq", C.c_void_p),
        ("n", C.c_int64), ("step", C.c_int64),
        ("lr", C.c_double), ("beta1", C.c_double), ("beta2", C.c_double), ("eps", C.c_double),
        ("weight_decay", C.c_double),
        ("zero_grad", C.c_int32),
    ]


class PackArgs(C.Structure):
    _fields_ = [
        ("num_points", C.c_int32),
        ("texture", C.c_void_p), ("confidence", C.c_void_p),
        ("params", Params),
        ("packed", C.c_void_p),
    ]


LIFT_BORDER_PIXELS = 32
LIFT_FLAGS_OFFSET = 192
LIFT_QUEUE_LENGTH_OFFSET = 176
LIFT_STATIC_MAX_CELLS = 1 << 19


class LiftArgs(C.Structure):
    _fields_ = [
        ("num_cells", C.c_int64),
        ("cell_bb_min", C.c_void_p), ("cell_bb_length", C.c_void_p),
        ("cell_value", C.c_void_p), ("cell_access_count", C.c_void_p),
        ("num_poses", C.c_int32), ("num_cameras", C.c_int32),
        ("poses_se3", C.c_void_p), ("intrinsics", C.c_void_p),
        ("view", View),
        ("loss_image", C.c_void_p),
        ("channels", C.c_int32), ("height", C.c_int32), ("width", C.c_int32),
        ("border_pixels", C.c_int32),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
    ]


class ForwardArgs(C.Structure):
    _fields_ = [
        ("num_points", C.c_int32), ("num_views", C.c_int32), ("num_poses", C.c_int32), ("num_cameras", C.c_int32),
        ("position", C.c_void_p),
        ("index", C.c_void_p),
        ("texture", C.c_void_p),
        ("confidence", C.c_void_p),
        ("background", C.c_void_p),
        ("dropout", C.c_void_p),
        ("poses_se3", C.c_void_p),
        ("intrinsics", C.c_void_p),
        ("views", C.POINTER(View)),
        ("params", Params),
        ("save_for_backward", C.c_int32),
        ("out", C.c_void_p * MAX_LAYERS),
        ("out_mask", C.c_void_p * MAX_LAYERS),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_size_t),
        ("out_weight", C.c_void_p * MAX_LAYERS),
        ("point_order", C.c_void_p),
        ("packed_descriptors", C.c_void_p),
    ]


class BackwardArgs(C.Structure):
    _fields_ = [
        ("fwd", ForwardArgs),
        ("grad_out", C.c_void_p * MAX_LAYERS),
        ("grad_texture", C.c_void_p),
        ("grad_confidence", C.c_void_p),
        ("grad_background", C.c_void_p),
        ("grad_points", C.c_void_p),
        ("grad_point_count", C.c_void_p),
        ("grad_pose", C.c_void_p),
        ("grad_pose_count", C.c_void_p),
        ("grad_intrinsics", C.c_void_p),
        ("grad_intrinsics_count", C.c_void_p),
    ]


# Every symbol include/vetrast.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "vetrast_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "vetrast_destroy": (None, [C.c_void_p]),
    "vetrast_layer_sizes": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "vetrast_workspace_layout_for": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                               C.POINTER(WorkspaceLayout)]),
    "vetrast_workspace_layout_for_mode": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                                    C.POINTER(WorkspaceLayout)]),
    "vetrast_forward_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "vetrast_forward": (C.c_int, [C.c_void_p, C.POINTER(ForwardArgs), C.c_void_p]),
    "vetrast_backward": (C.c_int, [C.c_void_p, C.POINTER(BackwardArgs), C.c_void_p]),
    "vetrast_packed_descriptor_bytes": (C.c_size_t, [C.c_int32]),
    "vetrast_pack_descriptors": (C.c_int, [C.c_void_p, C.POINTER(PackArgs), C.c_void_p]),
    "vetrast_adam_step": (C.c_int, [C.c_void_p, C.POINTER(AdamArgs), C.c_void_p]),
    "vetrast_lift_workspace_bytes": (C.c_size_t, [C.c_int64]),
    "vetrast_lift_error": (C.c_int, [C.c_void_p, C.POINTER(LiftArgs), C.c_void_p]),
    "vetrast_lift_error_static": (C.c_int, [C.c_void_p, C.POINTER(LiftArgs), C.c_void_p]),
    "vetrast_query_device_flags": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(WorkspaceLayout), C.c_void_p]),
    "vetrast_set_profiling": (C.c_int, [C.c_void_p, C.c_int32]),
    "vetrast_reset_scope_times": (C.c_int, [C.c_void_p]),
    "vetrast_scope_times": (C.c_int, [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_int32)]),
    "vetrast_scope_name": (C.c_char_p, [C.c_int32]),
    "vetrast_status_string": (C.c_char_p, [C.c_int]),
    "vetrast_last_hip_error": (C.c_int, [C.c_void_p]),
}

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libvetrast.so")
_lib = None


def load_library(path=None):
    """Loads libvetrast.so and declares the prototypes. Raises OSError if the library has not been built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise OSError(f"{p} is missing: build it with `python -m vet_amd.build` (there is no CPU fallback)")
    lib = C.CDLL(p)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


class VetrastError(RuntimeError):
    def __init__(self, status, where=""):
        self.status = status
        try:
            msg = load_library().vetrast_status_string(status).decode()
        except Exception:  # pragma: no cover
            msg = "?"
        super().__init__(f"vetrast {where} failed: {status} ({msg})")


def check(status, where=""):
    if status != OK:
        raise VetrastError(status, where)
