"""ctypes binding of the CPU oracle (liboracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark import this
module.  Arrays are numpy, C-contiguous; every wrapper checks dtype and size
before handing a pointer to C.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

ACT_NONE, ACT_RELU, ACT_LOGISTIC, ACT_EXPONENTIAL = 0, 1, 2, 3
RENDER_AO, RENDER_SHADE, RENDER_NORMALS, RENDER_DEPTH, RENDER_DISTANCE, RENDER_COST = range(6)
COLOR_LINEAR, COLOR_SRGB, COLOR_VISPOSNEG = 0, 1, 2
WARP_NGP, WARP_MIPNERF360, WARP_DONERF, WARP_SIGMOID, WARP_ERP, WARP_SINUSOIDAL = range(6)
SAMPLING_ORIGINAL, SAMPLING_DISPARITY, SAMPLING_LOG = 0, 1, 2
GRID_WARPED_EXP, GRID_WARPED_RECIPROCAL, GRID_METRIC_EXP, GRID_METRIC_RECIPROCAL = range(4)
REG_NONE, REG_DISTORTION = 0, 1
LOSS_L2, LOSS_L1, LOSS_MAPE, LOSS_SMAPE, LOSS_SMOOTHL1, LOSS_LOGL1, LOSS_RELATIVEL2 = range(7)
DTYPE_F16, DTYPE_F32 = 0, 1

u32, i32, f32, u8, u16, u64, i64 = C.c_uint32, C.c_int32, C.c_float, C.c_uint8, C.c_uint16, C.c_uint64, C.c_int64
vp = C.c_void_p


class Params(C.Structure):
    _fields_ = [
        ("warping_type", i32), ("griddist_type", i32), ("sampling_type", i32), ("use_grid", i32),
        ("aabb_min", f32 * 3), ("aabb_max", f32 * 3), ("aabb_scale", u32),
        ("grid_size", u32 * 3), ("n_cascades", u32), ("n_max_steps", u32),
        ("cone_angle_constant", f32), ("min_cone_stepsize", f32), ("max_cone_stepsize", f32),
        ("near_distance", f32), ("far_distance", f32),
        ("snap_to_pixel_centers_in_training", i32), ("snap_to_pixel_centers_in_rendering", i32),
        ("min_optical_thickness", f32), ("ema_decay", f32),
    ]

    @property
    def n_cells(self):
        return int(self.grid_size[0]) * int(self.grid_size[1]) * int(self.grid_size[2])

    @property
    def n_total(self):
        return self.n_cells * int(self.n_cascades)


class Pcg32(C.Structure):
    _fields_ = [("state", u64), ("inc", u64)]


class Dataset(C.Structure):
    _fields_ = [
        ("n_images", u32), ("resolution", i32 * 2), ("focal_length", f32 * 2), ("principal_point", f32 * 2),
        ("xforms", vp), ("images", vp), ("sampling_probability", vp),
    ]


class LossArgs(C.Structure):
    _fields_ = [
        ("n_rays", u32), ("n_max_compacted_coords", u32), ("padded_output_width", i32),
        ("rgb_activation", i32), ("density_activation", i32), ("loss_type", i32), ("loss_scale", f32),
        ("regularization_type", i32), ("mean_density", f32), ("min_optical_thickness", f32), ("use_grid", i32),
        ("background_color", f32 * 3), ("color_space", i32), ("train_with_random_bg_color", i32),
        ("train_in_linear_color", i32), ("transmittance_threshold", f32), ("rng", Pcg32),
        ("network_output_dtype", i32), ("dloss_dtype", i32), ("dt_stride", u32),
    ]


class RenderArgs(C.Structure):
    _fields_ = [
        ("n_rays", u32), ("n_steps", u32), ("n_steps_offset", u32), ("padded_output_width", u32),
        ("density_activation", i32), ("rgb_activation", i32), ("render_mode", i32),
        ("camera", f32 * 12), ("depth_scale", f32), ("transmittance_threshold", f32), ("network_output_dtype", i32),
    ]


class Field(C.Structure):
    _fields_ = [("table", vp), ("table_size", u32), ("seed", u32)]


PAYLOAD_DTYPE = np.dtype([("alive", np.uint8), ("pad_", np.uint8, (3,)), ("o", np.float32, (3,)), ("d", np.float32, (3,)),
                          ("idx", np.uint32), ("t", np.float32), ("n_steps", np.uint32)])
assert PAYLOAD_DTYPE.itemsize == 40


def build(force=False):
    """Compile liboracle.so / liboracle_libm.so with the Makefile beside this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)


def _ptr(a, dtype=None, min_size=None, allow_none=False):
    if a is None:
        if allow_none:
            return None
        raise ValueError("array required")
    if not isinstance(a, np.ndarray) or not a.flags["C_CONTIGUOUS"]:
        raise ValueError("need a C-contiguous numpy array")
    if dtype is not None and a.dtype != np.dtype(dtype):
        raise ValueError("dtype %s expected, got %s" % (np.dtype(dtype), a.dtype))
    if min_size is not None and a.size < min_size:
        raise ValueError("array too small: %d < %d" % (a.size, min_size))
    return a.ctypes.data_as(vp)


def _f3(x):
    return (f32 * 3)(*[float(v) for v in x])


class Oracle:
    """One loaded oracle library (shared-definition build by default, glibc build with libm=True)."""

    def __init__(self, libm=False, path=None):
        """path: a library built elsewhere from a (deliberately altered) copy of srf_oracle.cpp; the mutation tests use it"""
        if path is None:
            name = "liboracle_libm.so" if libm else "liboracle.so"
            path = os.path.join(_HERE, name)
            if not os.path.exists(path):
                build()
        self.lib = L = C.CDLL(path)
        L.orc_max_threads.restype = C.c_int
        L.orc_uses_libm.restype = C.c_int
        L.orc_morton3d.restype = u32
        L.orc_morton3d.argtypes = [u32, u32, u32]
        L.orc_morton3d_invert.restype = u32
        L.orc_morton3d_invert.argtypes = [u32]
        L.orc_pcg32_seed.argtypes = [C.POINTER(Pcg32), u64, u64]
        L.orc_pcg32_default.argtypes = [C.POINTER(Pcg32)]
        L.orc_pcg32_next_uint.restype = u32
        L.orc_pcg32_next_uint.argtypes = [C.POINTER(Pcg32)]
        L.orc_pcg32_next_float.restype = f32
        L.orc_pcg32_next_float.argtypes = [C.POINTER(Pcg32)]
        L.orc_pcg32_advance.argtypes = [C.POINTER(Pcg32), i64]
        L.orc_sobol.restype = u32
        L.orc_sobol.argtypes = [u32, u32]
        L.orc_ld_random_val.restype = f32
        L.orc_ld_random_val.argtypes = [u32, u32, u32]
        L.orc_ld_random_pixel_offset.argtypes = [u32, C.POINTER(f32 * 2)]
        L.orc_half_to_float.restype = f32
        L.orc_half_to_float.argtypes = [u16]
        L.orc_float_to_half.restype = u16
        L.orc_float_to_half.argtypes = [f32]
        L.orc_elem.restype = f32
        L.orc_elem.argtypes = [C.c_int, f32, f32]
        L.orc_params_default.argtypes = [C.POINTER(Params)]
        L.orc_params_finalize.argtypes = [C.POINTER(Params), f32, C.c_int, C.c_int]
        L.orc_calc_dt.restype = f32
        L.orc_calc_dt.argtypes = [C.POINTER(Params), f32, f32]
        L.orc_level_from_pos.restype = C.c_int
        L.orc_cascaded_grid_idx_at.restype = u32
        L.orc_occupied_at.restype = C.c_int
        L.orc_aabb_contains.restype = C.c_int
        for n in ("orc_network_to_rgb", "orc_network_to_rgb_derivative", "orc_network_to_density", "orc_network_to_density_derivative"):
            getattr(L, n).restype = f32
            getattr(L, n).argtypes = [f32, C.c_int]
        for n in ("orc_srgb_to_linear", "orc_linear_to_srgb"):
            getattr(L, n).restype = f32
            getattr(L, n).argtypes = [f32]
        L.orc_grid_mean.restype = f32
        L.orc_grid_mean.argtypes = [vp, u32]
        L.orc_update_grid_bitfield.restype = f32
        L.orc_render_frame.restype = u32
        L.orc_render_frame_mode.restype = u32

    # ---- primitives -------------------------------------------------------------
    def max_threads(self):
        return int(self.lib.orc_max_threads())

    def set_threads(self, n):
        self.lib.orc_set_threads(C.c_int(int(n)))

    def morton3d(self, x, y, z):
        return int(self.lib.orc_morton3d(x, y, z))

    def morton3d_invert(self, x):
        return int(self.lib.orc_morton3d_invert(x))

    def pcg32(self, initstate=None, initseq=1):
        r = Pcg32()
        if initstate is None:
            self.lib.orc_pcg32_default(C.byref(r))
        else:
            self.lib.orc_pcg32_seed(C.byref(r), int(initstate), int(initseq))
        return r

    def next_uint(self, r):
        return int(self.lib.orc_pcg32_next_uint(C.byref(r)))

    def next_float(self, r):
        return float(self.lib.orc_pcg32_next_float(C.byref(r)))

    def advance(self, r, delta=1 << 32):
        self.lib.orc_pcg32_advance(C.byref(r), int(delta))

    def sobol(self, index, dim):
        return int(self.lib.orc_sobol(index, dim))

    def ld_random_val(self, index, seed, dim=0):
        return float(self.lib.orc_ld_random_val(index, seed, dim))

    def ld_random_pixel_offset(self, spp):
        out = (f32 * 2)()
        self.lib.orc_ld_random_pixel_offset(spp, C.byref(out))
        return np.array(out[:], dtype=np.float32)

    def elem(self, which, a, b=0.0):
        return np.float32(self.lib.orc_elem(which, float(a), float(b)))

    def elem_array(self, which, a, b=None):
        a = np.asarray(a, dtype=np.float32)
        b = np.zeros_like(a) if b is None else np.asarray(b, dtype=np.float32)
        out = np.empty_like(a)
        fn = self.lib.orc_elem
        af, bf, of = a.ravel(), b.ravel(), out.ravel()
        for i in range(af.size):
            of[i] = fn(which, float(af[i]), float(bf[i]))
        return out

    # ---- parameters --------------------------------------------------------------
    def params(self, aabb_scale=1.0, min_cone_stepsize=None, max_cone_stepsize=None, grid_size=None, **kw):
        p = Params()
        self.lib.orc_params_default(C.byref(p))
        if grid_size is not None:
            gs = (grid_size,) * 3 if np.isscalar(grid_size) else tuple(grid_size)
            p.grid_size = (u32 * 3)(*gs)
        for k, v in kw.items():
            if not hasattr(p, k):
                raise AttributeError(k)
            setattr(p, k, v)
        if min_cone_stepsize is not None:
            p.min_cone_stepsize = min_cone_stepsize
        if max_cone_stepsize is not None:
            p.max_cone_stepsize = max_cone_stepsize
        self.lib.orc_params_finalize(C.byref(p), float(aabb_scale), int(min_cone_stepsize is not None), int(max_cone_stepsize is not None))
        return p

    # ---- scalar helpers ----------------------------------------------------------
    def ray_intersect(self, p, o, d):
        out = (f32 * 2)()
        self.lib.orc_aabb_ray_intersect(p.aabb_min, p.aabb_max, _f3(o), _f3(d), out)
        return np.array(out[:], dtype=np.float32)

    def contains(self, p, pos):
        return bool(self.lib.orc_aabb_contains(p.aabb_min, p.aabb_max, _f3(pos)))

    def calc_dt(self, p, t, cone_angle=0.0):
        return np.float32(self.lib.orc_calc_dt(C.byref(p), float(t), float(cone_angle)))

    def warp_position(self, p, pos):
        out = (f32 * 3)()
        self.lib.orc_warp_position(C.byref(p), _f3(pos), out)
        return np.array(out[:], dtype=np.float32)

    def unwarp_position(self, p, wpos):
        out = (f32 * 3)()
        self.lib.orc_unwarp_position(C.byref(p), _f3(wpos), out)
        return np.array(out[:], dtype=np.float32)

    def level_from_pos(self, p, pos, wpos):
        return int(self.lib.orc_level_from_pos(C.byref(p), _f3(pos), _f3(wpos)))

    def cascaded_grid_idx_at(self, p, pos, wpos, level):
        return int(self.lib.orc_cascaded_grid_idx_at(C.byref(p), _f3(pos), _f3(wpos), u32(level)))

    def occupied_at(self, p, bitfield, pos, wpos, level):
        return bool(self.lib.orc_occupied_at(C.byref(p), _ptr(bitfield, np.uint8, p.n_total // 8), _f3(pos), _f3(wpos), u32(level)))

    def pixel_to_ray(self, pixel, res, focal, pp, cam, spp=0, snap=True):
        out = (f32 * 6)()
        cam = np.ascontiguousarray(cam, dtype=np.float32).ravel()
        self.lib.orc_pixel_to_ray((i32 * 2)(*pixel), (i32 * 2)(*res), (f32 * 2)(*focal), (f32 * 2)(*pp), _ptr(cam, np.float32, 12), u32(spp), int(snap), out)
        return np.array(out[:], dtype=np.float32)

    def loss_and_gradient(self, loss_type, target, pred):
        l, g = (f32 * 3)(), (f32 * 3)()
        self.lib.orc_loss_and_gradient(int(loss_type), _f3(target), _f3(pred), l, g)
        return np.array(l[:], dtype=np.float32), np.array(g[:], dtype=np.float32)

    # ---- grid maintenance --------------------------------------------------------
    def generate_grid_samples(self, p, n_elements, rng, step, grid_in, thresh):
        pos = np.empty((n_elements, 3), np.float32)
        idx = np.empty(n_elements, np.uint32)
        self.lib.orc_generate_grid_samples(C.byref(p), u32(n_elements), rng, u32(step), _ptr(grid_in, np.float32, p.n_total), f32(thresh), _ptr(pos), _ptr(idx))
        return pos, idx

    def mark_untrained_density_grid(self, p, resolution, focal_length, xforms):
        xforms = np.ascontiguousarray(xforms, dtype=np.float32).reshape(-1, 12)
        grid = np.empty(p.n_total, np.float32)
        self.lib.orc_mark_untrained_density_grid(C.byref(p), u32(xforms.shape[0]), (i32 * 2)(*resolution), (f32 * 2)(*focal_length),
                                                 _ptr(xforms, np.float32, allow_none=True), _ptr(grid))
        return grid

    def splat_grid_samples(self, p, indices, padded_output_width, network_output, density_activation, grid_current):
        dtype = DTYPE_F16 if network_output.dtype == np.float16 else DTYPE_F32
        n = indices.size
        self.lib.orc_splat_grid_samples(C.byref(p), u32(n), _ptr(indices, np.uint32), u32(padded_output_width),
                                        _ptr(network_output, None, n * padded_output_width if n else 0), int(dtype), int(density_activation),
                                        _ptr(grid_current, np.float32, p.n_total))

    def ema_grid(self, grid_current, decay, grid):
        self.lib.orc_ema_grid(u32(grid.size), _ptr(grid_current, np.float32, grid.size), f32(decay), _ptr(grid, np.float32))

    def grid_mean(self, grid, n_elements):
        return np.float32(self.lib.orc_grid_mean(_ptr(grid, np.float32, n_elements), u32(n_elements)))

    def grid_to_bitfield(self, grid, mean, min_optical_thickness):
        bf = np.empty(grid.size // 8, np.uint8)
        self.lib.orc_grid_to_bitfield(u32(bf.size), _ptr(grid, np.float32), _ptr(bf), f32(mean), f32(min_optical_thickness))
        return bf

    def bitfield_max_pool(self, p, prev_level, next_level):
        self.lib.orc_bitfield_max_pool(C.byref(p), _ptr(prev_level, np.uint8, p.n_cells // 8), _ptr(next_level, np.uint8, p.n_cells // 8))

    def update_grid_bitfield(self, p, grid):
        bf = np.zeros(p.n_total // 8, np.uint8)
        mean = self.lib.orc_update_grid_bitfield(C.byref(p), _ptr(grid, np.float32, p.n_total), _ptr(bf))
        return bf, np.float32(mean)

    # ---- training sampler --------------------------------------------------------
    def make_dataset(self, xforms, resolution, focal, pp, images=None, sampling_probability=None):
        xforms = np.ascontiguousarray(xforms, dtype=np.float32).reshape(-1, 12)
        ds = Dataset()
        ds.n_images = xforms.shape[0]
        ds.resolution = (i32 * 2)(*resolution)
        ds.focal_length = (f32 * 2)(*focal)
        ds.principal_point = (f32 * 2)(*pp)
        ds.xforms = _ptr(xforms, np.float32)
        n_px = xforms.shape[0] * resolution[0] * resolution[1]
        ds.images = _ptr(images, np.float16, n_px * 4, allow_none=True)
        ds.sampling_probability = _ptr(sampling_probability, np.float16, n_px, allow_none=True)
        ds._keep = (xforms, images, sampling_probability)
        return ds

    def generate_training_samples(self, p, n_rays, n_rays_shift, n_coords, ds, bitfield, rng, ray_counter=0, numsteps_counter=0,
                                  want_coords=True, coords_capacity=None):
        cap = int(n_coords if coords_capacity is None else coords_capacity)
        rc = np.array([ray_counter], np.uint32)
        nc = np.array([numsteps_counter], np.uint32)
        rays = np.zeros((n_rays, 6), np.float32)
        rgba = np.zeros((n_rays, 4), np.float32)
        numsteps = np.zeros((n_rays, 2), np.uint32)
        coords = np.zeros((cap, 7), np.float32) if want_coords else None
        t_dt = np.zeros((cap, 2), np.float32)
        cell = np.zeros(cap, np.uint32)
        src = np.zeros(n_rays, np.uint32)
        self.lib.orc_generate_training_samples(C.byref(p), u32(n_rays), u32(n_rays_shift), u32(n_coords), C.byref(ds),
                                               _ptr(bitfield, np.uint8, p.n_total // 8, allow_none=not p.use_grid), rng,
                                               _ptr(rc), _ptr(nc), _ptr(rays), _ptr(rgba), _ptr(numsteps),
                                               _ptr(coords, allow_none=True), _ptr(t_dt), _ptr(cell), _ptr(src))
        return dict(ray_counter=int(rc[0]), numsteps_counter=int(nc[0]), rays=rays, rays_rgba=rgba, numsteps=numsteps,
                    coords=coords, t_dt=t_dt, cell=cell, src=src)

    # ---- rendering sampler -------------------------------------------------------
    def init_rays_with_payload(self, p, res, focal, pp, cam, spp=0):
        n = res[0] * res[1]
        pay = np.zeros(n, PAYLOAD_DTYPE)
        cam = np.ascontiguousarray(cam, dtype=np.float32).ravel()
        self.lib.orc_init_rays_with_payload(C.byref(p), (i32 * 2)(*res), (f32 * 2)(*focal), (f32 * 2)(*pp), _ptr(cam, np.float32, 12), u32(spp), _ptr(pay))
        return pay

    def advance_pos(self, p, payloads, bitfield, spp=0):
        self.lib.orc_advance_pos(C.byref(p), u32(payloads.size), u32(spp), _ptr(payloads, PAYLOAD_DTYPE), _ptr(bitfield, np.uint8, allow_none=True))

    def generate_coords_from_rays(self, p, n_rays, n_steps, bitfield, payloads, coords):
        self.lib.orc_generate_coords_from_rays(C.byref(p), u32(n_rays), u32(n_steps), _ptr(bitfield, np.uint8, allow_none=True),
                                               _ptr(payloads, PAYLOAD_DTYPE, n_rays), _ptr(coords, np.float32, n_rays * n_steps * 7))

    # ---- compositing -------------------------------------------------------------
    def volume_rendering_with_loss_and_gradient(self, args, rays_rgba, n_rays_counter, ray_coord_indices, dt, network_output, dloss,
                                                 n_compacted_counter=0, coords=None, compacted_coords=None, loss_output=None,
                                                 reg_buffer=None, rgb_ray_out=None):
        nrc = np.array([n_rays_counter], np.uint32)
        ncc = np.array([n_compacted_counter], np.uint32)
        self.lib.orc_volume_rendering_with_loss_and_gradient(
            C.byref(args), _ptr(rays_rgba, np.float32), _ptr(nrc), _ptr(ray_coord_indices, np.uint32), _ptr(dt, np.float32),
            _ptr(coords, np.float32, allow_none=True), _ptr(compacted_coords, np.float32, allow_none=True), _ptr(ncc),
            _ptr(network_output), _ptr(dloss), _ptr(loss_output, np.float32, allow_none=True),
            _ptr(reg_buffer, np.float32, allow_none=True), _ptr(rgb_ray_out, np.float32, allow_none=True))
        return int(ncc[0])

    def volume_rendering(self, p, args, payloads, rgba, coords, network_output):
        self.lib.orc_volume_rendering(C.byref(p), C.byref(args), _ptr(payloads, PAYLOAD_DTYPE), _ptr(rgba, np.float32),
                                      _ptr(coords, np.float32), _ptr(network_output))

    # ---- orchestrator kernels ----------------------------------------------------
    def compact_rays(self, n, src_pay, src_rgba, dst_pay, dst_rgba, fin_pay, fin_rgba, n_alive=0, n_final=0):
        na = np.array([n_alive], np.uint32)
        nf = np.array([n_final], np.uint32)
        self.lib.orc_compact_rays(u32(n), _ptr(src_pay, PAYLOAD_DTYPE), _ptr(src_rgba, np.float32), _ptr(dst_pay, PAYLOAD_DTYPE), _ptr(dst_rgba, np.float32),
                                  _ptr(fin_pay, PAYLOAD_DTYPE), _ptr(fin_rgba, np.float32), _ptr(na), _ptr(nf))
        return int(na[0]), int(nf[0])

    def shade(self, n, rgba, payloads, frame, render_mode=RENDER_SHADE, train_in_linear_colors=True):
        self.lib.orc_shade(u32(n), _ptr(rgba, np.float32), _ptr(payloads, PAYLOAD_DTYPE), _ptr(frame, np.float32), int(render_mode), int(train_in_linear_colors))

    def fill_rollover(self, n_out, n_in, buf):
        width_bytes = buf.itemsize * (buf.size // n_out)
        self.lib.orc_fill_rollover(u32(n_out), u32(width_bytes), u32(n_in), _ptr(buf))

    def fill_rollover_and_rescale(self, n_out, width, n_in, buf):
        dtype = DTYPE_F16 if buf.dtype == np.float16 else DTYPE_F32
        self.lib.orc_fill_rollover_and_rescale(u32(n_out), u32(width), u32(n_in), _ptr(buf, None, n_out * width), int(dtype))

    # ---- whole frame ---------------------------------------------------------------
    def make_field(self, table, seed):
        table = np.ascontiguousarray(table, dtype=np.float32).reshape(-1, 4)
        assert table.shape[0] & (table.shape[0] - 1) == 0
        f = Field()
        f.table = _ptr(table)
        f.table_size = table.shape[0]
        f.seed = seed
        f._keep = table
        return f

    def field_eval(self, p, field, wpos):
        out = (f32 * 4)()
        self.lib.orc_field_eval(C.byref(p), C.byref(field), _f3(wpos), out)
        return np.array(out[:], dtype=np.float32)

    def accumulate(self, frame, acc, sample_count, color_space):
        """render_buffer.cu:46-85 in place on `acc` (float32 [n, 4])"""
        self.lib.orc_accumulate(u32(frame.shape[0]), _ptr(frame, np.float32), _ptr(acc, np.float32), f32(sample_count), int(color_space))

    def tonemap(self, acc, exposure, background_color, color_space, output_color_space, curve):
        out = np.empty_like(acc)
        self.lib.orc_tonemap(u32(acc.shape[0]), f32(exposure), (f32 * 4)(*background_color), _ptr(acc, np.float32), int(color_space), int(output_color_space),
                             int(curve), _ptr(out))
        return out

    def render_frame(self, p, field, bitfield, res, focal, pp, cam, spp=0, transmittance_threshold=1e-4, train_in_linear_colors=True, render_mode=RENDER_SHADE):
        n = res[0] * res[1]
        frame = np.zeros((res[1], res[0], 4), np.float32)
        nsamp = np.zeros(n, np.uint32)
        cam = np.ascontiguousarray(cam, dtype=np.float32).ravel()
        iters = self.lib.orc_render_frame_mode(C.byref(p), C.byref(field), _ptr(bitfield, np.uint8, allow_none=not p.use_grid),
                                               (i32 * 2)(*res), (f32 * 2)(*focal), (f32 * 2)(*pp), _ptr(cam, np.float32, 12), u32(spp),
                                               f32(transmittance_threshold), int(train_in_linear_colors), int(render_mode), _ptr(frame), _ptr(nsamp))
        return frame, nsamp.reshape(res[1], res[0]), int(iters)


_cache = {}


def get(libm=False):
    if libm not in _cache:
        _cache[libm] = Oracle(libm=libm)
    return _cache[libm]
