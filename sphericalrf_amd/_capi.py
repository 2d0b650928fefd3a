"""ctypes view of libsrf_hip.so: structures and prototypes of include/srf_hip.h.

The library is loaded from sphericalrf_amd/lib/ (built in-tree by sphericalrf_amd.build).
There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# SRF_HIP_LIB names another build of the library (e.g. one compiled with different tuning constants)
LIB_PATH = os.environ.get("SRF_HIP_LIB") or os.path.join(_HERE, "lib", "libsrf_hip.so")

OK, ERR_INVALID, ERR_HIP, ERR_UNSUPPORTED = 0, -1, -2, -3
ACT_NONE, ACT_RELU, ACT_LOGISTIC, ACT_EXPONENTIAL = 0, 1, 2, 3
RENDER_AO, RENDER_SHADE, RENDER_NORMALS, RENDER_DEPTH, RENDER_DISTANCE, RENDER_COST = range(6)
COLOR_LINEAR, COLOR_SRGB, COLOR_VISPOSNEG = 0, 1, 2
WARP_NGP, WARP_MIPNERF360, WARP_DONERF, WARP_SIGMOID, WARP_ERP, WARP_SINUSOIDAL = range(6)
SAMPLING_ORIGINAL, SAMPLING_DISPARITY, SAMPLING_LOG = 0, 1, 2
GRID_WARPED_EXP, GRID_WARPED_RECIPROCAL, GRID_METRIC_EXP, GRID_METRIC_RECIPROCAL = range(4)
REG_NONE, REG_DISTORTION = 0, 1
LOSS_L2, LOSS_L1, LOSS_MAPE, LOSS_SMAPE, LOSS_SMOOTHL1, LOSS_LOGL1, LOSS_RELATIVEL2 = range(7)
DTYPE_F16, DTYPE_F32 = 0, 1

u32, i32, f32, u8, u16, u64 = C.c_uint32, C.c_int32, C.c_float, C.c_uint8, C.c_uint16, C.c_uint64
vp = C.c_void_p


class Pcg32(C.Structure):
    _fields_ = [("state", u64), ("inc", u64)]


class SamplerConfig(C.Structure):
    _fields_ = [
        ("warping_type", i32), ("aabb_scale", f32), ("use_grid", i32), ("init_grid_with_mask", i32),
        ("grid_size", u32 * 3), ("num_cascades", u32), ("ema_decay", f32), ("grid_distribution_type", i32),
        ("maximum_marching_steps", u32), ("cone_angle_constant", f32), ("min_cone_stepsize", f32), ("max_cone_stepsize", f32),
        ("near_distance", f32), ("far_distance", f32), ("sampling_type", i32),
        ("snap_to_pixel_centers_in_training", i32), ("snap_to_pixel_centers_in_rendering", i32), ("min_optical_thickness", f32),
    ]


class SamplerInfo(C.Structure):
    _fields_ = [
        ("warping_type", i32), ("aabb_scale", u32), ("aabb_min", f32 * 3), ("aabb_max", f32 * 3),
        ("use_grid", i32), ("init_grid_with_mask", i32), ("grid_size", u32 * 3),
        ("n_grid_elements", u32), ("n_cascades", u32), ("n_total_elements", u32), ("i_step", u32), ("ema_decay", f32),
        ("n_max_steps", u32), ("cone_angle_constant", f32), ("min_cone_stepsize", f32), ("max_cone_stepsize", f32),
        ("near_distance", f32), ("far_distance", f32), ("sampling_type", i32),
        ("snap_to_pixel_centers_in_training", i32), ("snap_to_pixel_centers_in_rendering", i32),
        ("min_optical_thickness", f32), ("griddist_type", i32),
        ("density_grid_current", vp), ("density_grid", vp), ("density_grid_mean", vp), ("density_grid_bitfield", vp),
        ("rng", Pcg32),
    ]


class Dataset(C.Structure):
    _fields_ = [
        ("n_images", u32), ("image_resolution", i32 * 2), ("focal_length", f32 * 2), ("principal_point", f32 * 2),
        ("xforms", vp), ("images", vp), ("sampling_probability", vp),
    ]


class MarcherConfig(C.Structure):
    _fields_ = [("train_with_random_bg_color", i32), ("train_in_linear_color", i32), ("transmittance_threshold", f32), ("regularization_type", i32)]


class LossArgs(C.Structure):
    _fields_ = [
        ("n_rays", u32), ("n_max_compacted_coords", u32), ("padded_output_width", i32),
        ("rgb_activation", i32), ("density_activation", i32), ("loss_type", i32), ("loss_scale", f32),
        ("min_optical_thickness", f32), ("use_grid", i32), ("background_color", f32 * 3), ("color_space", i32),
        ("rng", Pcg32), ("network_output_dtype", i32), ("dloss_dtype", i32), ("dt_stride", u32),
    ]


class RenderArgs(C.Structure):
    _fields_ = [
        ("n_rays", u32), ("n_steps", u32), ("i_steps_offset", u32), ("padded_output_width", u32),
        ("density_activation", i32), ("rgb_activation", i32), ("render_mode", i32),
        ("camera_matrix", f32 * 12), ("depth_scale", f32), ("network_output_dtype", i32),
    ]


class Field(C.Structure):
    _fields_ = [("table", vp), ("table_size", u32), ("seed", u32)]


class FrameArgs(C.Structure):
    _fields_ = [
        ("resolution", i32 * 2), ("focal_length", f32 * 2), ("principal_point", f32 * 2), ("camera_matrix", f32 * 12), ("spp", u32),
        ("render_mode", i32), ("density_activation", i32), ("rgb_activation", i32), ("depth_scale", f32),
        ("network_output_dtype", i32), ("padded_output_width", u32),
        ("input_gradient", vp), ("input_gradient_user", vp),
    ]


class FieldInferenceCtx(C.Structure):
    _fields_ = [("sampler", vp), ("field", C.POINTER(Field))]


# srf_inference_fn: (user, n_elements, coords, rgbsigma, dtype, padded_output_width, stream) -> int
INFERENCE_FN = C.CFUNCTYPE(C.c_int, vp, u32, vp, vp, i32, u32, vp)
# srf_input_gradient_fn: (user, n_elements, coords, stream) -> int
INPUT_GRADIENT_FN = C.CFUNCTYPE(C.c_int, vp, u32, vp, vp)
# the same with the element count in device memory: (user, n_elements_dev, max_elements, ...)
INFERENCE_COUNTED_FN = C.CFUNCTYPE(C.c_int, vp, vp, u32, vp, vp, i32, u32, vp)
INPUT_GRADIENT_COUNTED_FN = C.CFUNCTYPE(C.c_int, vp, vp, u32, vp, vp)


# every symbol include/srf_hip.h declares
SYMBOLS = [
    "srf_last_error", "srf_device_count",
    "srf_sampler_config_default", "srf_sampler_create", "srf_sampler_destroy", "srf_sampler_get_info", "srf_sampler_set_runtime",
    "srf_sampler_init", "srf_sampler_set_density_grid", "srf_sampler_load_density_grid", "srf_sampler_sample_positions_from_grid", "srf_sampler_update_grid",
    "srf_sampler_update_grid_bitfield", "srf_sampler_sample_coords_from_dataset", "srf_sampler_generate_rays_from_camera_matrix",
    "srf_sampler_generate_coords_from_rays", "srf_sampler_set_ray_sphere_bound", "srf_ray_sphere_bounds", "srf_sampler_set_grid_sample_order",
    "srf_marcher_config_default", "srf_marcher_create", "srf_marcher_destroy", "srf_marcher_get_config", "srf_marcher_set_config",
    "srf_marcher_volume_rendering_with_loss_and_gradient", "srf_marcher_volume_rendering_with_loss_and_gradient_noalloc", "srf_marcher_sync_check", "srf_marcher_volume_rendering",
    "srf_compact_rays", "srf_shade", "srf_fill_rollover", "srf_fill_rollover_and_rescale",
    "srf_render_frame", "srf_field_inference", "srf_field_input_gradient", "srf_render_frame_paced", "srf_field_inference_counted",
    "srf_field_input_gradient_counted", "srf_field_eval_counted", "srf_frame_accumulate", "srf_frame_tonemap",
    "srf_render_frame_fused", "srf_field_eval", "srf_debug_eval_elem", "srf_marcher_debug_set_lookback_spin_limit",
]


class SrfError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libsrf_hip error %d: %s" % (code, message))
        self.code = code
        self.message = message


_lib = None


def load():
    """Load libsrf_hip.so and set the prototypes.  Raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError("%s is missing: build it with `python -m sphericalrf_amd.build` (there is no CPU fallback)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    P = C.POINTER
    L.srf_last_error.restype = C.c_char_p
    L.srf_last_error.argtypes = []
    L.srf_device_count.restype = C.c_int
    L.srf_device_count.argtypes = []
    L.srf_sampler_config_default.restype = None
    L.srf_sampler_config_default.argtypes = [P(SamplerConfig)]
    L.srf_sampler_create.argtypes = [P(SamplerConfig), P(vp)]
    L.srf_sampler_destroy.restype = None
    L.srf_sampler_destroy.argtypes = [vp]
    L.srf_sampler_get_info.argtypes = [vp, P(SamplerInfo)]
    L.srf_sampler_set_runtime.argtypes = [vp, i32, i32, f32, f32]
    L.srf_sampler_init.argtypes = [vp, u32, P(i32 * 2), P(f32 * 2), P(f32 * 2), vp, P(Pcg32), vp]
    L.srf_sampler_set_density_grid.argtypes = [vp, vp, vp]
    L.srf_sampler_load_density_grid.argtypes = [vp, vp, u32, vp]
    L.srf_sampler_set_ray_sphere_bound.argtypes = [vp, P(f32 * 3), f32]
    L.srf_sampler_set_grid_sample_order.argtypes = [vp, i32]
    L.srf_ray_sphere_bounds.argtypes = [u32, vp, P(f32 * 3), f32, vp, vp, vp]
    L.srf_sampler_sample_positions_from_grid.argtypes = [vp, u32, u32, vp, vp, vp]
    L.srf_sampler_update_grid.argtypes = [vp, u32, u32, vp, i32, vp, i32, vp]
    L.srf_sampler_update_grid_bitfield.argtypes = [vp, vp]
    L.srf_sampler_sample_coords_from_dataset.argtypes = [vp, u32, u32, u32, P(Dataset), vp, vp, vp, vp, vp, vp, Pcg32, vp, vp, vp, vp]
    L.srf_sampler_generate_rays_from_camera_matrix.argtypes = [vp, P(i32 * 2), P(f32 * 2), P(f32 * 2), P(f32 * 12), vp, u32, vp]
    L.srf_sampler_generate_coords_from_rays.argtypes = [vp, u32, u32, vp, vp, vp]
    L.srf_marcher_config_default.restype = None
    L.srf_marcher_config_default.argtypes = [P(MarcherConfig)]
    L.srf_marcher_create.argtypes = [P(MarcherConfig), P(vp)]
    L.srf_marcher_destroy.restype = None
    L.srf_marcher_destroy.argtypes = [vp]
    L.srf_marcher_get_config.argtypes = [vp, P(MarcherConfig)]
    L.srf_marcher_set_config.argtypes = [vp, P(MarcherConfig)]
    L.srf_marcher_volume_rendering_with_loss_and_gradient.argtypes = [vp, P(LossArgs), vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    L.srf_marcher_volume_rendering_with_loss_and_gradient_noalloc.argtypes = L.srf_marcher_volume_rendering_with_loss_and_gradient.argtypes
    L.srf_marcher_sync_check.argtypes = [vp, vp]
    L.srf_marcher_volume_rendering.argtypes = [vp, vp, P(RenderArgs), vp, vp, vp, vp, vp]
    L.srf_compact_rays.argtypes = [vp, u32, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    L.srf_marcher_debug_set_lookback_spin_limit.argtypes = [vp, u32]
    L.srf_shade.argtypes = [u32, vp, vp, vp, i32, i32, vp]
    L.srf_fill_rollover.argtypes = [u32, u32, vp, vp, vp]
    L.srf_fill_rollover_and_rescale.argtypes = [u32, u32, vp, vp, i32, vp]
    L.srf_render_frame_fused.argtypes = [vp, vp, P(Field), P(i32 * 2), P(f32 * 2), P(f32 * 2), P(f32 * 12), u32, vp, vp, vp]
    L.srf_field_eval.argtypes = [vp, P(Field), u32, vp, vp, i32, u32, vp]
    L.srf_render_frame.argtypes = [vp, vp, P(FrameArgs), vp, vp, vp, P(u32), vp]
    L.srf_field_inference.argtypes = [vp, u32, vp, vp, i32, u32, vp]
    L.srf_field_input_gradient.argtypes = [vp, u32, vp, vp]
    L.srf_render_frame_paced.argtypes = [vp, vp, P(FrameArgs), vp, vp, vp, vp, vp, P(u32), vp]
    L.srf_field_inference_counted.argtypes = [vp, vp, u32, vp, vp, i32, u32, vp]
    L.srf_field_input_gradient_counted.argtypes = [vp, vp, u32, vp, vp]
    L.srf_field_eval_counted.argtypes = [vp, P(Field), vp, u32, vp, vp, i32, u32, vp]
    L.srf_frame_accumulate.argtypes = [P(i32 * 2), vp, vp, u32, i32, vp]
    L.srf_frame_tonemap.argtypes = [P(i32 * 2), f32, P(f32 * 4), vp, i32, i32, i32, vp, vp]
    L.srf_debug_eval_elem.argtypes = [i32, u32, vp, vp, vp, vp]
    for name in SYMBOLS:
        fn = getattr(L, name)
        if name not in ("srf_last_error", "srf_sampler_config_default", "srf_sampler_destroy", "srf_marcher_config_default", "srf_marcher_destroy"):
            fn.restype = C.c_int
    _lib = L
    return L


def check(code):
    if code != OK:
        raise SrfError(code, load().srf_last_error().decode("utf-8", "replace"))
    return code
