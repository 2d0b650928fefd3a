"""Pins of the oracle's batch functions that take nothing from the function under test: every expectation below is rebuilt in the
test from separately pinned scalars (pcg32, calc_dt, the slab test) or from float64 formulas written from the reference's lines.

Each pin is a plain function of an oracle object, so that tests/test_oracle_mutations.py can run it against a deliberately wrong
build of the oracle and require it to fail."""
import numpy as np

from oracle import oracle as O
from oracle.support import loss_args
from sphericalrf_amd import scene

U32 = 0xffffffff


def _f32(x):
    return np.float32(x)


# ------------------------------------------------------------------------------------------------------------
# training rays: internal/sampler/occupancy_sampler.cu:556-590,646 and internal/utils/common_device.h:191-213
# ------------------------------------------------------------------------------------------------------------
def _training_case(orc, aabb_scale, cam_radius, near, n_images=3, res=(7, 5), snap=1):
    p = orc.params(aabb_scale=aabb_scale, grid_size=(8, 8, 8), n_cascades=1, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_EXP,
                   sampling_type=O.SAMPLING_DISPARITY, n_max_steps=32, near_distance=near, far_distance=20.0,
                   snap_to_pixel_centers_in_training=snap)
    rng = np.random.default_rng(5)
    cams = np.zeros((n_images, 12), np.float32)
    for k in range(n_images):
        v = rng.normal(size=3)
        v /= np.linalg.norm(v)
        pos = 0.5 + cam_radius * v
        cams[k] = scene.look_at(pos, -v + 0.1 * rng.normal(size=3))
    focal = (9.0, 6.5)                      # non-square pixels
    pp = (0.4, 0.65)                        # principal point off the centre
    images = rng.random((n_images * res[0] * res[1], 4)).astype(np.float16)
    return p, cams, res, focal, pp, images


def _expected_training_ray(orc, p, cams, res, focal, pp, seed, i, n_rays, shift, snap):
    """one ray of generate_training_samples_nerf written from occupancy_sampler.cu:556-590; float32 step by step"""
    n_images = cams.shape[0]
    img = ((((shift + i) * n_images) & U32) // n_rays) % n_images                     # :556 (u32 wrap)
    rng = orc.pcg32(seed)
    orc.advance(rng, (i * 8) & U32)                                                   # :563
    xy = [_f32(orc.next_float(rng)), _f32(orc.next_float(rng))]                       # :564 random_val_2d: x first
    if snap:                                                                          # :565-567
        xy = [_f32((_f32(min(max(int(_f32(xy[a] * _f32(res[a]))), 0), res[a] - 1)) + _f32(0.5)) / _f32(res[a])) for a in range(2)]
    px = [min(max(int(_f32(xy[a] * _f32(res[a]))), 0), res[a] - 1) for a in range(2)]  # common_device.h:191-193 image_pos
    pixel_index = px[0] + px[1] * res[0] + img * res[0] * res[1]                      # common_device.h:195-197
    m = cams[img]
    o = m[9:12]
    dl = np.array([(np.float64(xy[0]) - pp[0]) * res[0] / focal[0], (np.float64(xy[1]) - pp[1]) * res[1] / focal[1], 1.0])   # :577-581
    d = m[0:3].astype(np.float64) * dl[0] + m[3:6].astype(np.float64) * dl[1] + m[6:9].astype(np.float64) * dl[2]
    d = d / np.linalg.norm(d)
    return dict(img=img, rng=rng, o=o, d=d, pixel_index=pixel_index, xy=xy)


def pin_training_rays(orc, aabb_scale=64, cam_radius=0.5, near=0.3):
    """origins, directions, the start of the march and the target pixel of every ray of a small batch, with a principal point
    off the centre, non-square pixels and image, three cameras, a shift, and the camera inside the box (start = near plane)"""
    p, cams, res, focal, pp, images = _training_case(orc, aabb_scale, cam_radius, near)
    ds = orc.make_dataset(cams, res, focal, pp, images=images)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    n_rays, shift, seed = 23, 11, 77
    out = orc.generate_training_samples(p, n_rays, shift, 1 << 16, ds, bf, orc.pcg32(seed))
    assert out["ray_counter"] == n_rays            # every bit is set: every ray has samples, kept ray r is ray r
    flat = images.astype(np.float32)
    n_jittered = 0
    for i in range(n_rays):
        e = _expected_training_ray(orc, p, cams, res, focal, pp, seed, i, n_rays, shift, snap=1)
        assert np.array_equal(out["rays"][i, :3], e["o"]), i
        assert np.allclose(out["rays"][i, 3:], e["d"], rtol=0, atol=2e-6), (i, out["rays"][i, 3:], e["d"])
        assert np.array_equal(out["rays_rgba"][i], flat[e["pixel_index"]]), i        # :646 read_rgba
        # :585-590: t0 = max(tmin, near), start = t0 + calc_dt(t0) * third draw; with every bit set the first sample is the start
        d32 = out["rays"][i, 3:]
        tmin = orc.ray_intersect(p, e["o"], d32)[0]
        t0 = _f32(max(tmin, _f32(p.near_distance)))
        jitter = _f32(orc.next_float(e["rng"]))
        start = _f32(t0 + _f32(orc.calc_dt(p, t0) * jitter))
        first = out["t_dt"][int(out["numsteps"][i, 1]), 0]
        assert first == start, (i, first, start, t0, jitter)
        n_jittered += jitter != _f32(0.5)
    assert n_jittered > n_rays // 2


def pin_training_rays_entering_the_box(orc):
    """the camera outside a unit box: the slab entry lies beyond the near plane and is where the march starts"""
    p, cams, res, focal, pp, images = _training_case(orc, 1, 2.5, 1.0)
    ds = orc.make_dataset(cams, res, focal, pp, images=images)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    n_rays, seed = 40, 3
    out = orc.generate_training_samples(p, n_rays, 0, 1 << 16, ds, bf, orc.pcg32(seed))
    n_checked = 0
    for r in range(out["ray_counter"]):
        i = int(out["src"][r])
        e = _expected_training_ray(orc, p, cams, res, focal, pp, seed, i, n_rays, 0, snap=1)
        assert np.array_equal(out["rays"][r, :3], e["o"])
        d32 = out["rays"][r, 3:]
        assert np.allclose(d32, e["d"], rtol=0, atol=2e-6)
        tmin = orc.ray_intersect(p, e["o"], d32)[0]
        assert 1.0 < tmin < 1e4                                    # a real entry point, beyond the near plane at 1.0
        start = _f32(tmin + _f32(orc.calc_dt(p, tmin) * _f32(orc.next_float(e["rng"]))))
        assert out["t_dt"][int(out["numsteps"][r, 1]), 0] == start
        n_checked += 1
    assert n_checked >= 5


def pin_training_rays_without_snapping(orc):
    """snap_to_pixel_centers off: the two draws are the image position as they are"""
    p, cams, res, focal, pp, images = _training_case(orc, 64, 0.5, 0.3, snap=0)
    ds = orc.make_dataset(cams, res, focal, pp, images=images)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    n_rays, seed = 9, 12
    out = orc.generate_training_samples(p, n_rays, 0, 1 << 16, ds, bf, orc.pcg32(seed))
    flat = images.astype(np.float32)
    for i in range(n_rays):
        e = _expected_training_ray(orc, p, cams, res, focal, pp, seed, i, n_rays, 0, snap=0)
        assert np.allclose(out["rays"][i, 3:], e["d"], rtol=0, atol=2e-6)
        assert np.array_equal(out["rays_rgba"][i], flat[e["pixel_index"]])


def pin_sampling_probability_pixel(orc):
    """a ray is skipped exactly when the probability AT ITS OWN PIXEL (x + y*W + img*W*H) is <= 0 (:569-570); a negative one skips
    it too, and a NaN, which is not <= 0, keeps it"""
    p, cams, res, focal, pp, images = _training_case(orc, 64, 0.5, 0.3)
    n_rays, seed = 60, 21
    expected = [_expected_training_ray(orc, p, cams, res, focal, pp, seed, i, n_rays, 0, snap=1) for i in range(n_rays)]
    hit = sorted({e["pixel_index"] for e in expected})
    zeroed = set(hit[::2])                                          # every second pixel that some ray lands on
    prob = np.ones(cams.shape[0] * res[0] * res[1], np.float16)
    prob[list(zeroed)] = 0
    prob[hit[2]] = -0.5
    prob[hit[1]] = np.nan
    ds = orc.make_dataset(cams, res, focal, pp, images=images, sampling_probability=prob)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    out = orc.generate_training_samples(p, n_rays, 0, 1 << 16, ds, bf, orc.pcg32(seed))
    kept = [i for i, e in enumerate(expected) if e["pixel_index"] not in zeroed]
    assert any(e["pixel_index"] == hit[1] for e in expected)
    assert 0 < len(kept) < n_rays
    assert out["ray_counter"] == len(kept)
    assert np.array_equal(out["src"][:len(kept)], np.uint32(kept))


# ------------------------------------------------------------------------------------------------------------
# grid samples: internal/sampler/occupancy_sampler.cu:121-147
# ------------------------------------------------------------------------------------------------------------
def _invert_morton(idx):
    x = y = z = 0
    for b in range(10):
        x |= ((idx >> (3 * b)) & 1) << b
        y |= ((idx >> (3 * b + 1)) & 1) << b
        z |= ((idx >> (3 * b + 2)) & 1) << b
    return x, y, z


def pin_grid_sample_draws(orc):
    """level = uint(f0 * C) % C and position = (cell corner + (f1, f2, f3)) / N - 0.5, scaled by 2^-(C-level-1), + 0.5, with f0..f3
    the four draws after advance(4 i); uniform draw (every cell passes at the first try)"""
    N, Cn = (8, 4, 4), 3
    p = orc.params(aabb_scale=4, grid_size=N, n_cascades=Cn, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_EXP)
    grid = np.zeros(p.n_total, np.float32)
    n, step, seed = 50, 3, 19
    pos, idx = orc.generate_grid_samples(p, n, orc.pcg32(seed), step, grid, -0.01)
    levels = set()
    for i in range(n):
        rng = orc.pcg32(seed)
        orc.advance(rng, (4 * i) & U32)
        f = [_f32(orc.next_float(rng)) for _ in range(4)]
        level = int(_f32(f[0] * _f32(Cn))) % Cn
        cell = (((i + step * n) * 56924617 + 96925573) & U32) % p.n_cells
        assert idx[i] == cell + level * p.n_cells, (i, idx[i], cell, level)
        xyz = _invert_morton(cell)
        scale = 2.0 ** -(Cn - level - 1)
        want = [((xyz[a] + np.float64(f[1 + a])) / N[a] - 0.5) * scale + 0.5 for a in range(3)]
        assert np.allclose(pos[i], want, rtol=0, atol=1e-6), (i, pos[i], want)
        levels.add(level)
    assert levels == {0, 1, 2}


def pin_grid_sample_retries(orc):
    """non-uniform draw: the first of the ten candidate cells ((i + step n) A + j B + C) mod n_cells whose value in the point's own
    cascade exceeds the threshold; the last candidate when none does"""
    N, Cn = (4, 4, 4), 2
    p = orc.params(aabb_scale=2, grid_size=N, n_cascades=Cn, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_EXP)
    g = np.random.default_rng(1)
    grid = (g.random(p.n_total) < 0.2).astype(np.float32)          # sparse: several tries fail
    n, step, seed, thresh = 80, 1, 4, 0.5
    pos, idx = orc.generate_grid_samples(p, n, orc.pcg32(seed), step, grid, thresh)
    n_late = n_none = 0
    for i in range(n):
        rng = orc.pcg32(seed)
        orc.advance(rng, (4 * i) & U32)
        level = int(_f32(_f32(orc.next_float(rng)) * _f32(Cn))) % Cn
        chosen = None
        for j in range(10):
            chosen = ((((i + step * n) * 56924617) + j * 19349663 + 96925573) & U32) % p.n_cells + level * p.n_cells
            if grid[chosen] > thresh:
                break
        else:
            n_none += 1
        n_late += j > 0
        assert idx[i] == chosen, (i, idx[i], chosen)
    assert n_late > 10 and n_none > 0


# ------------------------------------------------------------------------------------------------------------
# compositing: internal/render/ray_marcher.cu:57-135
# ------------------------------------------------------------------------------------------------------------
def _srgb_to_linear(v):
    v = np.asarray(v, np.float64)
    return np.where(v <= 0.04045, v / 12.92, ((v + 0.055) / 1.055) ** 2.4)


def _linear_to_srgb(v):
    v = np.asarray(v, np.float64)
    return np.where(v < 0.0031308, 12.92 * v, 1.055 * np.maximum(v, 0) ** 0.41666 - 0.055)


def _composite(orc, a, counts, net, dt, targets):
    n_rays = len(counts)
    idx = np.zeros((n_rays, 2), np.uint32)
    idx[:, 0] = counts
    idx[:, 1] = np.concatenate([[0], np.cumsum(counts)[:-1]])
    dloss = np.zeros((int(np.sum(counts)), 4), np.float32)
    loss = np.full(n_rays, -1, np.float32)
    rgb = np.zeros((n_rays, 3), np.float32)
    orc.volume_rendering_with_loss_and_gradient(a, targets, n_rays, idx, dt, net, dloss, loss_output=loss, rgb_ray_out=rgb)
    return idx, dloss, loss, rgb


def pin_background_only_behind_unterminated_rays(orc):
    """ray 0 falls below the transmittance threshold half way (T = 4^-3 < 0.05 before its fourth sample): no background, although
    its T is still large enough to show; ray 1 runs through all its samples: T * bg is added (:106-109).  Linear training, so
    bg = srgb_to_linear(background_color)."""
    bg = (0.8, 0.4, 0.2)
    c = np.float32([0.25, 0.5, 0.75])
    n = 6
    net = np.zeros((2 * n, 4), np.float32)
    net[:, :3] = c
    net[:n, 3] = np.log(4.0)   # alpha = 3/4 per sample
    net[n:, 3] = 0.1
    dt = np.ones(2 * n, np.float32)
    a = loss_args(2, 100, background_color=(O.f32 * 3)(*bg), transmittance_threshold=0.05)
    idx, dloss, loss, rgb = _composite(orc, a, [n, n], net, dt, np.float32([[0, 0, 0, 1], [0, 0, 0, 1]]))
    assert idx[0, 0] == 3 and idx[1, 0] == n
    assert np.allclose(rgb[0], c * (1 - 4.0 ** -3), rtol=2e-6)                        # terminated: colour only
    T = np.exp(-0.1 * n)
    assert np.allclose(rgb[1], c * (1 - T) + T * _srgb_to_linear(bg), rtol=2e-6)      # open: colour + T bg


def _target_from_gradient(orc, a, tex, n_rays=1):
    """the target colour the kernel formed for texel `tex`, recovered from the L2 gradient of one half-transparent sample:
    dL/dc = loss_scale / n_rays * w * 2 (pred - target)"""
    net = np.float32([[0.3, 0.6, 0.9, np.log(2.0)]])
    dt = np.ones(1, np.float32)
    targets = np.zeros((n_rays, 4), np.float32)
    targets[0] = tex
    counts = [1] + [0] * (n_rays - 1)
    idx, dloss, loss, rgb = _composite(orc, a, counts, net, dt, targets)
    w = 0.5
    pred = rgb[0].astype(np.float64)
    return pred - dloss[0, :3].astype(np.float64) * n_rays / (a.loss_scale * 2 * w), pred, loss


def pin_srgb_target_unpremultiplies(orc):
    """colour space sRGB, training in sRGB: target = linear_to_srgb(rgb / a) * a + (1 - a) * bg_srgb for a > 0, bg_srgb for a = 0
    (:97-104); the linear colour space instead converts rgb + (1 - a) bg as a whole (:91-96)"""
    bg = (0.2, 0.5, 0.9)
    bg_srgb = _linear_to_srgb(_srgb_to_linear(bg))
    tex = np.float32([0.1, 0.2, 0.3, 0.5])
    a = loss_args(1, 10, background_color=(O.f32 * 3)(*bg), color_space=O.COLOR_SRGB, train_in_linear_color=0)
    got, _, _ = _target_from_gradient(orc, a, tex)
    want = _linear_to_srgb(tex[:3].astype(np.float64) / 0.5) * 0.5 + 0.5 * bg_srgb
    assert np.allclose(got, want, rtol=0, atol=2e-6), (got, want)
    got0, _, _ = _target_from_gradient(orc, a, np.float32([0.1, 0.2, 0.3, 0.0]))
    assert np.allclose(got0, bg_srgb, rtol=0, atol=2e-6)
    a_lin = loss_args(1, 10, background_color=(O.f32 * 3)(*bg), color_space=O.COLOR_LINEAR, train_in_linear_color=0)
    got_lin, _, _ = _target_from_gradient(orc, a_lin, tex)
    want_lin = _linear_to_srgb(tex[:3].astype(np.float64) + 0.5 * _srgb_to_linear(bg))
    assert np.allclose(got_lin, want_lin, rtol=0, atol=2e-6), (got_lin, want_lin)
    assert not np.allclose(want, want_lin, atol=1e-3)


def pin_loss_output_is_divided_by_n_rays(orc):
    """loss_output[i] = mean over channels of the loss / n_rays (:131), and the gradients carry loss_scale / n_rays (:133)"""
    n_rays = 5
    a = loss_args(n_rays, 10)
    target, pred, loss = _target_from_gradient(orc, a, np.float32([0.9, 0.1, 0.4, 1.0]), n_rays=n_rays)
    assert np.allclose(target, [0.9, 0.1, 0.4], atol=2e-6)          # which also pins the 1 / n_rays of the gradient
    assert np.isclose(loss[0] * n_rays, np.mean((pred - [0.9, 0.1, 0.4]) ** 2), rtol=1e-5)
    assert (loss[1:] == -1).all()                                    # rays without samples write no loss


def pin_exponential_rgb_regulariser(orc):
    """Exponential rgb activation: dL/draw = ls * (w g exp(raw) + max(0, 1e-4 raw)) (:135,183-185); with the target equal to the
    prediction g vanishes and only the regulariser is left — for positive raw values, nothing for negative ones"""
    raw = np.float32([[0.5, -0.7, 1.25, np.log(2.0)]])
    dt = np.ones(1, np.float32)
    a = loss_args(1, 10, rgb_activation=O.ACT_EXPONENTIAL)
    _, _, _, rgb = _composite(orc, a, [1], raw, dt, np.float32([[0, 0, 0, 1]]))
    assert np.allclose(rgb[0], 0.5 * np.exp(raw[0, :3].astype(np.float64)), rtol=2e-6)
    tgt = np.float32([[rgb[0, 0], rgb[0, 1], rgb[0, 2], 1.0]])       # prediction == target: g = 0 exactly
    _, dloss, _, _ = _composite(orc, a, [1], raw, dt, tgt)
    want = a.loss_scale * np.maximum(0.0, 1e-4 * raw[0, :3].astype(np.float64))
    assert np.allclose(dloss[0, :3], want, rtol=1e-5, atol=0), (dloss[0, :3], want)
    assert dloss[0, 1] == 0 and dloss[0, 0] > 0
    # the other activations carry no such term
    a2 = loss_args(1, 10, rgb_activation=O.ACT_NONE)
    _, _, _, rgb2 = _composite(orc, a2, [1], raw, dt, np.float32([[0, 0, 0, 1]]))
    _, dloss2, _, _ = _composite(orc, a2, [1], raw, dt, np.float32([[rgb2[0, 0], rgb2[0, 1], rgb2[0, 2], 1.0]]))
    assert (dloss2[0, :3] == 0).all()


# ------------------------------------------------------------------------------------------------------------
# bitfield threshold: internal/sampler/occupancy_sampler.cu:1063-1088
# ------------------------------------------------------------------------------------------------------------
def pin_bitfield_mean_is_cascade_zero_only(orc):
    """the threshold is min(min_optical_thickness, mean of max(v, 0) over cascade 0); cascades 1.. hold much larger values here, so a
    mean over everything would clear most of cascade 0's bits"""
    N, Cn = (8, 8, 8), 3
    p = orc.params(aabb_scale=4, grid_size=N, n_cascades=Cn, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_RECIPROCAL,
                   min_optical_thickness=0.5)
    g = np.random.default_rng(2)
    grid = np.empty(p.n_total, np.float32)
    grid[:p.n_cells] = g.random(p.n_cells) * 1e-3
    grid[:p.n_cells:7] = -1.0                                        # masked cells count as 0 in the mean
    grid[p.n_cells:] = 0.2 + g.random(p.n_total - p.n_cells) * 0.2
    bf, mean = orc.update_grid_bitfield(p, grid)
    want_mean = np.maximum(grid[:p.n_cells].astype(np.float64), 0).sum() / p.n_cells
    assert np.isclose(mean, want_mean, rtol=1e-5), (mean, want_mean)
    bits = np.unpackbits(bf, bitorder="little")
    assert np.array_equal(bits, (grid > np.float32(mean)).astype(np.uint8))      # Reciprocal grid: no pooling on top
    assert 0.3 < bits[:p.n_cells].mean() < 0.7 and bits[p.n_cells:].all()


PINS = [pin_training_rays, pin_training_rays_entering_the_box, pin_training_rays_without_snapping, pin_sampling_probability_pixel,
        pin_grid_sample_draws, pin_grid_sample_retries, pin_background_only_behind_unterminated_rays, pin_srgb_target_unpremultiplies,
        pin_loss_output_is_divided_by_n_rays, pin_exponential_rgb_regulariser, pin_bitfield_mean_is_cascade_zero_only]


def test_training_rays(orc):
    pin_training_rays(orc)


def test_training_rays_entering_the_box(orc):
    pin_training_rays_entering_the_box(orc)


def test_training_rays_without_snapping(orc):
    pin_training_rays_without_snapping(orc)


def test_sampling_probability_pixel(orc):
    pin_sampling_probability_pixel(orc)


def test_grid_sample_draws(orc):
    pin_grid_sample_draws(orc)


def test_grid_sample_retries(orc):
    pin_grid_sample_retries(orc)


def test_background_only_behind_unterminated_rays(orc):
    pin_background_only_behind_unterminated_rays(orc)


def test_srgb_target_unpremultiplies(orc):
    pin_srgb_target_unpremultiplies(orc)


def test_loss_output_is_divided_by_n_rays(orc):
    pin_loss_output_is_divided_by_n_rays(orc)


def test_exponential_rgb_regulariser(orc):
    pin_exponential_rgb_regulariser(orc)


def test_bitfield_mean_is_cascade_zero_only(orc):
    pin_bitfield_mean_is_cascade_zero_only(orc)
