"""Host-side mirror of the reference's OccupancySampler / RayMarcher over libsrf_hip.so.

Method names and argument meaning follow internal/sampler/occupancy_sampler.h:13-135 and
internal/render/ray_marcher.h:13-81 of the reference; tcnn::GPUMemory<T> arguments become
torch CUDA tensors (used only as device memory), cudaStream_t becomes the current torch
stream.  Every method enqueues work and returns; errors raise SrfError (bad enum strings
raise with the reference's messages).
"""
import ctypes as C

import torch

from . import _capi as K
from ._capi import (ACT_EXPONENTIAL, ACT_LOGISTIC, ACT_NONE, ACT_RELU, COLOR_LINEAR, COLOR_SRGB, DTYPE_F16, DTYPE_F32,  # noqa: F401
                    ERR_HIP, ERR_INVALID, ERR_UNSUPPORTED, LOSS_L2, LOSS_SMOOTHL1, RENDER_AO, RENDER_COST, RENDER_DEPTH, RENDER_DISTANCE,
                    RENDER_NORMALS, RENDER_SHADE, SrfError)

_WARP = {"ngp": K.WARP_NGP, "mipnerf360": K.WARP_MIPNERF360, "donerf": K.WARP_DONERF, "sigmoid": K.WARP_SIGMOID,
         "erp": K.WARP_ERP, "sinusoidalprojection": K.WARP_SINUSOIDAL}
_SAMPLING = {"original": K.SAMPLING_ORIGINAL, "disparity": K.SAMPLING_DISPARITY, "log": K.SAMPLING_LOG}
_GRIDDIST = {"warpedspace_exp": K.GRID_WARPED_EXP, "warpedspace_reciprocal": K.GRID_WARPED_RECIPROCAL,
             "metricspace_exp": K.GRID_METRIC_EXP, "metricspace_reciprocal": K.GRID_METRIC_RECIPROCAL}
_REG = {"none": K.REG_NONE, "distortion": K.REG_DISTORTION}
_LOSS = {"l2": K.LOSS_L2, "relativel2": K.LOSS_RELATIVEL2, "l1": K.LOSS_L1, "mape": K.LOSS_MAPE, "smape": K.LOSS_SMAPE,
         "smoothl1": K.LOSS_SMOOTHL1, "logl1": K.LOSS_LOGL1}


def _lookup(table, s, message):
    """case-insensitive enum parsing with the reference's error text (occupancy_sampler.cu:865-907)"""
    if isinstance(s, int):
        return s
    try:
        return table[str(s).lower()]
    except KeyError:
        raise RuntimeError(message) from None


def string_to_warping_type(s):
    return _lookup(_WARP, s, "Unknown warping type.")


def string_to_sampling_type(s):
    return _lookup(_SAMPLING, s, "Unknown sampling type.")


def string_to_griddist_type(s):
    return _lookup(_GRIDDIST, s, "Unknown grid distribution type.")


def string_to_regularization_type(s):
    return _lookup(_REG, s, "Unknown regularization type.")


def string_to_loss_type(s):
    return _lookup(_LOSS, s, "Unknown loss type.")


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, dtype=None, min_numel=None, name="tensor", allow_none=False):
    """device pointer of a contiguous CUDA tensor, with the checks the C side cannot make"""
    if t is None:
        if allow_none:
            return None
        raise ValueError("%s is required" % name)
    if not t.is_cuda:
        raise ValueError("%s must live on the GPU" % name)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if dtype is not None and t.dtype != dtype:
        raise ValueError("%s: dtype %s expected, got %s" % (name, dtype, t.dtype))
    if min_numel is not None and t.numel() < min_numel:
        raise ValueError("%s: %d elements needed, has %d" % (name, min_numel, t.numel()))
    return C.c_void_p(t.data_ptr())


def _net_dtype(t):
    if t.dtype == torch.float16:
        return K.DTYPE_F16
    if t.dtype == torch.float32:
        return K.DTYPE_F32
    raise ValueError("network tensors must be float16 or float32")


class Pcg32:
    """tcnn::pcg32 held on the host, as Testbed::m_rng (internal/testbed.h:92-93)."""
    MULT = 0x5851f42d4c957f2d
    MASK = (1 << 64) - 1

    def __init__(self, initstate=None, initseq=1):
        if initstate is None:
            self.state, self.inc = 0x853c49e6748fea9b, 0xda3e39cb94b95bdb
        else:
            self.state = 0
            self.inc = ((initseq << 1) | 1) & self.MASK
            self.next_uint()
            self.state = (self.state + initstate) & self.MASK
            self.next_uint()

    def next_uint(self):
        old = self.state
        self.state = (old * self.MULT + self.inc) & self.MASK
        xs = (((old >> 18) ^ old) >> 27) & 0xffffffff
        rot = old >> 59
        return ((xs >> rot) | (xs << ((-rot) & 31))) & 0xffffffff

    def advance(self, delta=1 << 32):
        cur_mult, cur_plus, acc_mult, acc_plus = self.MULT, self.inc, 1, 0
        delta &= self.MASK
        while delta > 0:
            if delta & 1:
                acc_mult = (acc_mult * cur_mult) & self.MASK
                acc_plus = (acc_plus * cur_mult + cur_plus) & self.MASK
            cur_plus = ((cur_mult + 1) * cur_plus) & self.MASK
            cur_mult = (cur_mult * cur_mult) & self.MASK
            delta >>= 1
        self.state = (acc_mult * self.state + acc_plus) & self.MASK

    def as_c(self):
        return K.Pcg32(self.state, self.inc)


class Dataset:
    """The Dataset fields the sampler reads (internal/dataset/dataset.h:19-39)."""

    def __init__(self, xforms, image_resolution, focal_length, principal_point, images=None, sampling_probability=None):
        self.xforms = xforms.contiguous()
        if self.xforms.dtype != torch.float32 or self.xforms.numel() % 12:
            raise ValueError("xforms: float32 tensor of n_images x 12 (column-major 3x4) expected")
        self.n_images = self.xforms.numel() // 12
        self.image_resolution = tuple(int(v) for v in image_resolution)
        self.focal_length = tuple(float(v) for v in focal_length)
        self.principal_point = tuple(float(v) for v in principal_point)
        self.images = images
        self.sampling_probability = sampling_probability

    def as_c(self):
        n_px = self.n_images * self.image_resolution[0] * self.image_resolution[1]
        d = K.Dataset()
        d.n_images = self.n_images
        d.image_resolution = (K.i32 * 2)(*self.image_resolution)
        d.focal_length = (K.f32 * 2)(*self.focal_length)
        d.principal_point = (K.f32 * 2)(*self.principal_point)
        d.xforms = _dev(self.xforms, torch.float32, self.n_images * 12, "xforms")
        d.images = _dev(self.images, torch.float16, n_px * 4, "images", allow_none=True)
        d.sampling_probability = _dev(self.sampling_probability, torch.float16, n_px, "sampling_probability", allow_none=True)
        return d


def sampler_config_from_dict(config):
    """the "samlper" JSON block (a dict) as srf_sampler_config: the reference's keys and defaults, occupancy_sampler.cu:911-943"""
    L = K.load()
    cfg = K.SamplerConfig()
    L.srf_sampler_config_default(C.byref(cfg))
    cfg.warping_type = string_to_warping_type(config.get("warping_type", "NGP"))
    cfg.aabb_scale = float(config.get("aabb_scale", 1))
    cfg.use_grid = int(bool(config.get("use_grid", True)))
    cfg.init_grid_with_mask = int(bool(config.get("init_grid_with_mask", True)))
    gs = config.get("grid_size", 128)
    gs = (gs, gs, gs) if isinstance(gs, int) else tuple(gs)
    cfg.grid_size = (K.u32 * 3)(*gs)
    cfg.num_cascades = int(config.get("num_cascades", 1))
    cfg.ema_decay = float(config.get("ema_decay", 0.95))
    if cfg.use_grid:
        # the reference parses this key only when use_grid is set, and its default "Exp" is not a valid name
        cfg.grid_distribution_type = string_to_griddist_type(config.get("grid_distribution_type", "Exp"))
    cfg.maximum_marching_steps = int(config.get("maximum_marching_steps", 1024))
    cfg.cone_angle_constant = float(config.get("cone_angle_constant", 0.0))
    cfg.min_cone_stepsize = float(config.get("min_cone_stepsize", -1.0))
    cfg.max_cone_stepsize = float(config.get("max_cone_stepsize", -1.0))
    cfg.near_distance = float(config.get("near_distance", 0.2))
    cfg.far_distance = float(config.get("far_distance", 100.0))
    cfg.sampling_type = string_to_sampling_type(config.get("sampling_type", "Original"))
    cfg.snap_to_pixel_centers_in_training = int(bool(config.get("snap_to_pixel_centers_in_training", True)))
    cfg.snap_to_pixel_centers_in_rendering = int(bool(config.get("snap_to_pixel_centers_in_rendering", True)))
    cfg.min_optical_thickness = float(config.get("min_optical_thickness", 0.01))
    return cfg


class OccupancySampler:
    """internal/sampler/occupancy_sampler.h:13-135.  `config` is the "samlper" JSON block as a dict."""

    def __init__(self, config):
        self._h = None
        L = K.load()
        cfg = sampler_config_from_dict(config)
        h = C.c_void_p()
        K.check(L.srf_sampler_create(C.byref(cfg), C.byref(h)))
        self._h = h
        self._L = L

    def __del__(self):
        if getattr(self, "_h", None):
            self._L.srf_sampler_destroy(self._h)
            self._h = None

    # ---- public members ---------------------------------------------------------
    @property
    def info(self):
        out = K.SamplerInfo()
        K.check(self._L.srf_sampler_get_info(self._h, C.byref(out)))
        return out

    def __getattr__(self, name):
        # the reference's public data members: warping_type, aabb_scale, n_grid_size ... (occupancy_sampler.h:88-134)
        if name.startswith("_"):
            raise AttributeError(name)
        info = self.info
        if name == "n_grid_size":
            return int(info.grid_size[0])
        if name in ("density_grid", "density_grid_current", "density_grid_mean", "density_grid_bitfield"):
            return self._view(name, info)
        if hasattr(info, name):
            v = getattr(info, name)
            return list(v) if hasattr(v, "__len__") else v
        raise AttributeError(name)

    def _view(self, name, info):
        """a torch tensor aliasing one of the sampler-owned device buffers (no copy)"""
        ptr = getattr(info, name)
        if not ptr:
            return None
        if name == "density_grid_bitfield":
            n, dt, item = info.n_total_elements // 8, torch.uint8, 1
        elif name == "density_grid_mean":
            n, dt, item = 1, torch.float32, 4
        else:
            n, dt, item = info.n_total_elements, torch.float32, 4

        class _Holder:
            pass
        holder = _Holder()
        holder.__cuda_array_interface__ = {"shape": (n,), "typestr": "|u1" if item == 1 else "<f4", "data": (int(ptr), False), "version": 2}
        holder._owner = self
        return torch.as_tensor(holder, device="cuda")

    def set_runtime(self, snap_to_pixel_centers_in_training=None, snap_to_pixel_centers_in_rendering=None, near_distance=None, far_distance=None):
        i = self.info
        K.check(self._L.srf_sampler_set_runtime(
            self._h,
            int(i.snap_to_pixel_centers_in_training if snap_to_pixel_centers_in_training is None else snap_to_pixel_centers_in_training),
            int(i.snap_to_pixel_centers_in_rendering if snap_to_pixel_centers_in_rendering is None else snap_to_pixel_centers_in_rendering),
            float(i.near_distance if near_distance is None else near_distance),
            float(i.far_distance if far_distance is None else far_distance)))

    # ---- methods ----------------------------------------------------------------
    def init(self, n_images, image_resolution, focal_length, principal_point, camera_matrices, images, rng):
        """occupancy_sampler.cu:946-978; `rng` is the caller's Pcg32 and is advanced by one draw."""
        r = rng.as_c()
        K.check(self._L.srf_sampler_init(self._h, int(n_images), C.byref((K.i32 * 2)(*image_resolution)), C.byref((K.f32 * 2)(*focal_length)),
                                         C.byref((K.f32 * 2)(*principal_point)), _dev(camera_matrices, allow_none=True), C.byref(r), _stream()))
        rng.state, rng.inc = r.state, r.inc

    def set_ray_sphere_bound(self, center, radius):
        """bounds the marches by a sphere as well (no counterpart in the reference; radius <= 0 removes the bound): exactly those
        samples of the unbounded march remain whose t lies within the ray's stretch inside the sphere"""
        K.check(self._L.srf_sampler_set_ray_sphere_bound(self._h, C.byref((K.f32 * 3)(*[float(v) for v in center])), float(radius)))

    def set_grid_sample_order(self, cell_order):
        """cell_order=True: sample_positions_from_grid leaves the uniform points of whole multiples of the cell count sorted by
        cell, and likewise those of the non-uniform draw (no counterpart in the reference; see grid_sample_entry_points for
        which point an entry holds); update_grid, given densities and indices in that order, splats the uniform ones without
        sorting; the resulting grid is the same"""
        K.check(self._L.srf_sampler_set_grid_sample_order(self._h, 1 if cell_order else 0))

    def grid_sample_entry_points(self, n_uniform, n_nonuniform=0, step=None):
        """which point of the reference's order (uniform draw, then non-uniform draw) each entry of sample_positions_from_grid's
        outputs holds in cell order (numpy int64 array of n_uniform + n_nonuniform entries); step: the number of update_grid
        calls before the draw (default: so far)"""
        import numpy as np
        nc = int(self.info.n_grid_elements)
        step = self.i_step if step is None else int(step)
        inv = pow(56924617, -1, 1 << 32)
        parts = []
        for first, n in ((0, int(n_uniform)), (int(n_uniform), int(n_nonuniform))):
            n_dealt = n // nc * nc if nc >= 2048 and nc & (nc - 1) == 0 else 0
            t = np.arange(n_dealt, dtype=np.int64)
            u = ((t & (nc - 1)) * inv) & (nc - 1)
            parts.append(first + ((u - step * n) & (nc - 1)) + (t // nc) * nc)
            parts.append(first + np.arange(n_dealt, n, dtype=np.int64))
        return np.concatenate(parts)

    def set_density_grid(self, grid):
        K.check(self._L.srf_sampler_set_density_grid(self._h, _dev(grid, torch.float32, self.info.n_total_elements, "grid"), _stream()))

    def sample_positions_from_grid(self, n_uniform_positions, n_nonuniform_positions, grid_positions, grid_indices):
        n = n_uniform_positions + n_nonuniform_positions
        K.check(self._L.srf_sampler_sample_positions_from_grid(self._h, n_uniform_positions, n_nonuniform_positions,
                                                               _dev(grid_positions, torch.float32, 3 * n, "grid_positions"),
                                                               _dev(grid_indices, torch.int32, n, "grid_indices"), _stream()))

    def update_grid(self, n_total_positions, padded_output_width, grid_densities, grid_indices, density_activation):
        K.check(self._L.srf_sampler_update_grid(self._h, n_total_positions, padded_output_width,
                                                _dev(grid_densities, None, n_total_positions * padded_output_width, "grid_densities"),
                                                _net_dtype(grid_densities), _dev(grid_indices, torch.int32, n_total_positions, "grid_indices"),
                                                int(density_activation), _stream()))

    def update_grid_bitfield(self):
        K.check(self._L.srf_sampler_update_grid_bitfield(self._h, _stream()))

    def sample_coords_from_dataset(self, n_rays, n_rays_shift, n_coords, dataset, rays, rays_rgba, n_rays_counter, ray_coord_indices,
                                   coords, n_coords_counter, rng, sample_t=None, sample_dt=None, sample_cell=None):
        d = dataset.as_c()
        for t, need, nm in ((coords, 7 * n_coords, "coords"), (sample_t, n_coords, "sample_t"), (sample_dt, n_coords, "sample_dt")):
            if t is not None and (t.dtype != torch.float32 or t.numel() < need):
                raise ValueError("%s: float32 tensor of at least %d elements expected" % (nm, need))
        K.check(self._L.srf_sampler_sample_coords_from_dataset(
            self._h, n_rays, n_rays_shift, n_coords, C.byref(d),
            _dev(rays, torch.float32, 6 * n_rays, "rays"), _dev(rays_rgba, torch.float32, 4 * n_rays, "rays_rgba"),
            _dev(n_rays_counter, torch.int32, 1, "n_rays_counter"), _dev(ray_coord_indices, torch.int32, 2 * n_rays, "ray_coord_indices"),
            _dev(coords, torch.float32, None, "coords", allow_none=True), _dev(n_coords_counter, torch.int32, 1, "n_coords_counter"),
            rng.as_c(), _dev(sample_t, torch.float32, None, "sample_t", allow_none=True), _dev(sample_dt, torch.float32, None, "sample_dt", allow_none=True),
            _dev(sample_cell, torch.int32, n_coords, "sample_cell", allow_none=True), _stream()))

    def generate_rays_from_camera_matrix(self, resolution, focal_length, principal_point, camera_matrix, payload, spp=0):
        n = resolution[0] * resolution[1]
        K.check(self._L.srf_sampler_generate_rays_from_camera_matrix(
            self._h, C.byref((K.i32 * 2)(*resolution)), C.byref((K.f32 * 2)(*focal_length)), C.byref((K.f32 * 2)(*principal_point)),
            C.byref((K.f32 * 12)(*[float(v) for v in camera_matrix])), _dev(payload, torch.uint8, 40 * n, "payload"), int(spp), _stream()))

    def generate_coords_from_rays(self, n_rays, n_steps, payloads, coords):
        K.check(self._L.srf_sampler_generate_coords_from_rays(self._h, n_rays, n_steps, _dev(payloads, torch.uint8, 40 * n_rays, "payloads"),
                                                              _dev(coords, torch.float32, 7 * n_rays * n_steps, "coords"), _stream()))

    def field_eval(self, field, n_coords, coords, rgbsigma, padded_output_width=4):
        K.check(self._L.srf_field_eval(self._h, C.byref(field.as_c()), n_coords, _dev(coords, torch.float32, 7 * n_coords, "coords"),
                                       _dev(rgbsigma, None, n_coords * padded_output_width, "rgbsigma"), _net_dtype(rgbsigma),
                                       padded_output_width, _stream()))

    def render_frame_fused(self, marcher, field, resolution, focal_length, principal_point, camera_matrix, frame_buffer, n_samples=None, spp=0):
        n = resolution[0] * resolution[1]
        K.check(self._L.srf_render_frame_fused(
            self._h, marcher._h, C.byref(field.as_c()), C.byref((K.i32 * 2)(*resolution)), C.byref((K.f32 * 2)(*focal_length)),
            C.byref((K.f32 * 2)(*principal_point)), C.byref((K.f32 * 12)(*[float(v) for v in camera_matrix])), int(spp),
            _dev(frame_buffer, torch.float32, 4 * n, "frame_buffer"), _dev(n_samples, torch.int32, n, "n_samples", allow_none=True), _stream()))


    def render_frame(self, marcher, inference, resolution, focal_length, principal_point, camera_matrix, frame_buffer, spp=0,
                     render_mode=K.RENDER_SHADE, density_activation=K.ACT_EXPONENTIAL, rgb_activation=K.ACT_LOGISTIC, depth_scale=1.0,
                     network_output_dtype=K.DTYPE_F16, padded_output_width=4, input_gradient=None, paced=False):
        """Testbed::render_frame up to shade (internal/testbed.cu:479-611).  `inference` is a Field (the stand-in network) or a callable
        (n_elements, coords_ptr, rgbsigma_ptr, dtype, padded_output_width, stream_ptr) -> int that enqueues the network on the stream.
        Normals mode needs `input_gradient` (testbed.cu:558-560): True with a Field (the stand-in's gradient), else a callable
        (n_elements, coords_ptr, stream_ptr) -> int that overwrites each record's position with the density's gradient.
        An exception raised by a callable ends the frame and is raised again here.  Returns the number of rounds.
        paced=True runs the loop paced by the device (srf_render_frame_paced): the callables then get the element count as a device
        pointer followed by an upper limit, (n_elements_ptr, max_elements, coords_ptr, ...), and must not need it on the host."""
        a = K.FrameArgs()
        a.resolution, a.focal_length, a.principal_point = (K.i32 * 2)(*resolution), (K.f32 * 2)(*focal_length), (K.f32 * 2)(*principal_point)
        a.camera_matrix = (K.f32 * 12)(*[float(v) for v in camera_matrix])
        a.spp, a.render_mode, a.density_activation, a.rgb_activation = int(spp), int(render_mode), int(density_activation), int(rgb_activation)
        a.depth_scale, a.network_output_dtype, a.padded_output_width = float(depth_scale), int(network_output_dtype), int(padded_output_width)
        iters = K.u32(0)
        n = resolution[0] * resolution[1]
        raised = []

        def guarded(fn, *args):
            # ctypes prints and drops an exception that leaves a callback, and the frame would go on with stale buffers
            try:
                return int(fn(*args) or 0)
            except BaseException as e:      # noqa: B902 - handed back to the caller below
                raised.append(e)
                return K.ERR_INVALID

        keep = []
        if isinstance(inference, Field):
            f = inference.as_c()
            ctx = K.FieldInferenceCtx(self._h, C.pointer(f))
            fn = C.cast(self._L.srf_field_inference_counted if paced else self._L.srf_field_inference, C.c_void_p)
            user = C.cast(C.pointer(ctx), C.c_void_p)
            keep += [f, ctx]
            if input_gradient is True:
                gfn, guser = C.cast(self._L.srf_field_input_gradient_counted if paced else self._L.srf_field_input_gradient, C.c_void_p), user
                input_gradient = None
            else:
                gfn, guser = None, None
        else:
            if paced:
                cb = K.INFERENCE_COUNTED_FN(lambda user, n_dev, n_max, coords, out, dtype, width, stream: guarded(inference, n_dev, n_max, coords, out, dtype, width, stream))
            else:
                cb = K.INFERENCE_FN(lambda user, n_el, coords, out, dtype, width, stream: guarded(inference, n_el, coords, out, dtype, width, stream))
            fn, user, gfn, guser = C.cast(cb, C.c_void_p), None, None, None
            keep.append(cb)
        if input_gradient is True:
            raise ValueError("input_gradient=True needs a Field as the inference")
        if input_gradient is not None:
            if paced:
                gcb = K.INPUT_GRADIENT_COUNTED_FN(lambda user, n_dev, n_max, coords, stream: guarded(input_gradient, n_dev, n_max, coords, stream))
            else:
                gcb = K.INPUT_GRADIENT_FN(lambda user, n_el, coords, stream: guarded(input_gradient, n_el, coords, stream))
            gfn = C.cast(gcb, C.c_void_p)
            keep.append(gcb)
        fb = _dev(frame_buffer, torch.float32, 4 * n, "frame_buffer")
        if paced:
            rc = self._L.srf_render_frame_paced(self._h, marcher._h, C.byref(a), fn, user, gfn, guser, fb, C.byref(iters), _stream())
        else:
            a.input_gradient, a.input_gradient_user = gfn, guser
            rc = self._L.srf_render_frame(self._h, marcher._h, C.byref(a), fn, user, fb, C.byref(iters), _stream())
        del keep
        if raised:
            raise raised[0]
        K.check(rc)
        return int(iters.value)


def ray_sphere_bounds(rays, center, radius, t_near, t_far):
    """the stretch t_near <= t <= t_far of every ray (origin, direction: 6 floats) inside a sphere; (+inf, -inf) for a miss"""
    n = rays.numel() // 6
    K.check(K.load().srf_ray_sphere_bounds(n, _dev(rays, torch.float32, 6 * n, "rays"), C.byref((K.f32 * 3)(*[float(v) for v in center])), float(radius),
                                           _dev(t_near, torch.float32, n, "t_near"), _dev(t_far, torch.float32, n, "t_far"), _stream()))


def frame_accumulate(resolution, frame_buffer, accumulate_buffer, spp, color_space=K.COLOR_LINEAR):
    """CudaRenderBuffer::accumulate (internal/utils/render_buffer.cu:46-85, :211-227); spp = frames already accumulated"""
    n = resolution[0] * resolution[1]
    K.check(K.load().srf_frame_accumulate(C.byref((K.i32 * 2)(*resolution)), _dev(frame_buffer, torch.float32, 4 * n, "frame_buffer"),
                                          _dev(accumulate_buffer, torch.float32, 4 * n, "accumulate_buffer"), int(spp), int(color_space), _stream()))


TONEMAP_IDENTITY, TONEMAP_ACES, TONEMAP_HABLE, TONEMAP_REINHARD = 0, 1, 2, 3


def frame_tonemap(resolution, exposure, background_color, accumulate_buffer, out_rgba, color_space=K.COLOR_LINEAR, output_color_space=K.COLOR_SRGB,
                  tonemap_curve=TONEMAP_IDENTITY):
    """CudaRenderBuffer::tonemap (internal/utils/render_buffer.cu:87-178, :229-235)"""
    n = resolution[0] * resolution[1]
    K.check(K.load().srf_frame_tonemap(C.byref((K.i32 * 2)(*resolution)), float(exposure), C.byref((K.f32 * 4)(*background_color)),
                                       _dev(accumulate_buffer, torch.float32, 4 * n, "accumulate_buffer"), int(color_space), int(output_color_space),
                                       int(tonemap_curve), _dev(out_rgba, torch.float32, 4 * n, "out_rgba"), _stream()))


class Field:
    """Table-lookup stand-in for the network (not in the reference): table is (size, 4) float32 on the GPU, size a power of two."""

    def __init__(self, table, seed):
        if table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != 4 or table.shape[0] & (table.shape[0] - 1):
            raise ValueError("table: (2^k, 4) float32 expected")
        self.table = table.contiguous()
        self.seed = int(seed)

    def as_c(self):
        return K.Field(_dev(self.table, torch.float32, None, "table"), self.table.shape[0], self.seed)


class RayMarcher:
    """internal/render/ray_marcher.h:13-81.  `config` is the "render" JSON block as a dict."""

    def __init__(self, config):
        self._h = None
        L = K.load()
        cfg = K.MarcherConfig()
        L.srf_marcher_config_default(C.byref(cfg))
        cfg.train_with_random_bg_color = int(bool(config.get("train_with_random_bg_color", True)))
        cfg.train_in_linear_color = int(bool(config.get("train_in_linear_color", False)))
        cfg.transmittance_threshold = float(config.get("transmittance_threshold", 0.0001))
        cfg.regularization_type = string_to_regularization_type(config.get("regularization_type", "None"))
        h = C.c_void_p()
        K.check(L.srf_marcher_create(C.byref(cfg), C.byref(h)))
        self._h = h
        self._L = L

    def __del__(self):
        if getattr(self, "_h", None):
            self._L.srf_marcher_destroy(self._h)
            self._h = None

    @property
    def config(self):
        out = K.MarcherConfig()
        K.check(self._L.srf_marcher_get_config(self._h, C.byref(out)))
        return out

    def __getattr__(self, name):
        if name.startswith("_"):
            raise AttributeError(name)
        cfg = self.config
        if hasattr(cfg, name):
            return getattr(cfg, name)
        raise AttributeError(name)

    def volume_rendering_with_loss_and_gradient(self, n_rays, n_max_compacted_coords, rays_rgba, n_rays_counter, ray_coord_indices,
                                                 dt, network_output, dloss_doutput, n_compacted_coords_counter, padded_output_width=4,
                                                 rgb_activation=K.ACT_LOGISTIC, density_activation=K.ACT_EXPONENTIAL, loss_output=None,
                                                 loss_type=K.LOSS_L2, loss_scale=128.0, density_grid_mean=None, min_optical_thickness=0.01,
                                                 use_grid=True, background_color=(0.0, 0.0, 0.0), color_space=K.COLOR_LINEAR, rng=None,
                                                 coords=None, compacted_coords=None, dt_stride=1, rgb_ray_out=None, no_alloc=False):
        """no_alloc: go through the entry point that allocates no device memory (n_rays <= NOALLOC_MAX_RAYS)"""
        a = K.LossArgs()
        a.n_rays, a.n_max_compacted_coords, a.padded_output_width = n_rays, n_max_compacted_coords, padded_output_width
        a.rgb_activation, a.density_activation = int(rgb_activation), int(density_activation)
        a.loss_type, a.loss_scale = string_to_loss_type(loss_type), float(loss_scale)
        a.min_optical_thickness, a.use_grid = float(min_optical_thickness), int(bool(use_grid))
        a.background_color = (K.f32 * 3)(*background_color)
        a.color_space = int(color_space)
        a.rng = (rng or Pcg32()).as_c()
        a.network_output_dtype, a.dloss_dtype = _net_dtype(network_output), _net_dtype(dloss_doutput)
        a.dt_stride = int(dt_stride)
        entry = self._L.srf_marcher_volume_rendering_with_loss_and_gradient_noalloc if no_alloc else self._L.srf_marcher_volume_rendering_with_loss_and_gradient
        K.check(entry(
            self._h, C.byref(a), _dev(rays_rgba, torch.float32, 4 * n_rays, "rays_rgba"), _dev(n_rays_counter, torch.int32, 1, "n_rays_counter"),
            _dev(ray_coord_indices, torch.int32, 2 * n_rays, "ray_coord_indices"), _dev(dt, torch.float32, None, "dt"),
            _dev(coords, torch.float32, None, "coords", allow_none=True), _dev(compacted_coords, torch.float32, None, "compacted_coords", allow_none=True),
            _dev(n_compacted_coords_counter, torch.int32, 1, "n_compacted_coords_counter"), _dev(network_output, None, None, "network_output"),
            _dev(dloss_doutput, None, n_max_compacted_coords * padded_output_width, "dloss_doutput"),
            _dev(loss_output, torch.float32, n_rays, "loss_output", allow_none=True),
            _dev(density_grid_mean, torch.float32, 1, "density_grid_mean", allow_none=True),
            _dev(rgb_ray_out, torch.float32, 3 * n_rays, "rgb_ray_out", allow_none=True), _stream()))

    def sync_check(self):
        """wait for the current stream and raise if a training compositing call could not order its offsets"""
        K.check(self._L.srf_marcher_sync_check(self._h, _stream()))

    def debug_set_lookback_spin_limit(self, polls):
        """test hook: polls a workgroup of the streaming kernel makes before it gives up waiting for its predecessors"""
        K.check(self._L.srf_marcher_debug_set_lookback_spin_limit(self._h, int(polls)))

    def volume_rendering(self, sampler, n_rays, n_steps, i_steps_offset, payloads, rgba, coords, rgbsigma, padded_output_width=4,
                         density_activation=K.ACT_EXPONENTIAL, rgb_activation=K.ACT_LOGISTIC, render_mode=K.RENDER_SHADE,
                         camera_matrix=None, depth_scale=1.0):
        a = K.RenderArgs()
        a.n_rays, a.n_steps, a.i_steps_offset, a.padded_output_width = n_rays, n_steps, i_steps_offset, padded_output_width
        a.density_activation, a.rgb_activation, a.render_mode = int(density_activation), int(rgb_activation), int(render_mode)
        a.camera_matrix = (K.f32 * 12)(*[float(v) for v in (camera_matrix if camera_matrix is not None else [0.0] * 12)])
        a.depth_scale = float(depth_scale)
        a.network_output_dtype = _net_dtype(rgbsigma)
        K.check(self._L.srf_marcher_volume_rendering(self._h, sampler._h, C.byref(a), _dev(payloads, torch.uint8, 40 * n_rays, "payloads"),
                                                     _dev(rgba, torch.float32, 4 * n_rays, "rgba"), _dev(coords, torch.float32, 7 * n_rays * n_steps, "coords"),
                                                     _dev(rgbsigma, None, n_rays * n_steps * padded_output_width, "rgbsigma"), _stream()))


NOALLOC_MAX_RAYS = 262144   # SRF_NOALLOC_MAX_RAYS


# ---- orchestrator kernels (internal/testbed.cu:398-404, 423-477) ---------------------------------
def compact_rays(marcher, n_elements, src_payloads, src_rgba, dst_payloads, dst_rgba, final_payloads, final_rgba, n_alive_counter, n_final_counter):
    """compact_rays_kernel (internal/testbed.cu:423-446); `marcher` (a RayMarcher) owns the scratch of the ordered compaction"""
    K.check(K.load().srf_compact_rays(marcher._h, n_elements, _dev(src_payloads, torch.uint8, 40 * n_elements), _dev(src_rgba, torch.float32, 4 * n_elements),
                                      _dev(dst_payloads, torch.uint8, 40 * n_elements), _dev(dst_rgba, torch.float32, 4 * n_elements),
                                      _dev(final_payloads, torch.uint8, 40 * n_elements), _dev(final_rgba, torch.float32, 4 * n_elements),
                                      _dev(n_alive_counter, torch.int32, 1), _dev(n_final_counter, torch.int32, 1), _stream()))


def shade(n_rays, rgba, payloads, frame_buffer, render_mode=K.RENDER_SHADE, train_in_linear_colors=False):
    K.check(K.load().srf_shade(n_rays, _dev(rgba, torch.float32, 4 * n_rays), _dev(payloads, torch.uint8, 40 * n_rays),
                               _dev(frame_buffer, torch.float32), int(render_mode), int(bool(train_in_linear_colors)), _stream()))


def fill_rollover(n_elements, n_input_elements, inout):
    stride_bytes = inout.element_size() * (inout.numel() // n_elements)
    K.check(K.load().srf_fill_rollover(n_elements, stride_bytes, _dev(n_input_elements, torch.int32, 1), _dev(inout), _stream()))


def fill_rollover_and_rescale(n_elements, stride, n_input_elements, inout):
    K.check(K.load().srf_fill_rollover_and_rescale(n_elements, stride, _dev(n_input_elements, torch.int32, 1),
                                                   _dev(inout, None, n_elements * stride), _net_dtype(inout), _stream()))


def debug_eval_elem(which, a, b=None):
    out = torch.empty_like(a)
    K.check(K.load().srf_debug_eval_elem(which, a.numel(), _dev(a, torch.float32), _dev(b, torch.float32, a.numel(), allow_none=True), _dev(out), _stream()))
    return out
