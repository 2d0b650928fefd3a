"""Closed forms, float64 finite differences and bookkeeping checks that pin the oracle's compositing kernels."""
import math

import numpy as np
import pytest

from oracle import oracle as O
from sphericalrf_amd import scene
from oracle.support import loss_args  # noqa: F401  (other test modules import it from here)
from tests import helpers


def run(orc, a, counts, net, dt, targets, n_active=None, counter0=0):
    n_rays = len(counts)
    idx = np.zeros((n_rays, 2), np.uint32)
    idx[:, 0] = counts
    idx[:, 1] = np.concatenate([[0], np.cumsum(counts)[:-1]])
    dloss_dt = np.float16 if a.dloss_dtype == O.DTYPE_F16 else np.float32
    dloss = np.full((max(1, a.n_max_compacted_coords), 4), 7, dloss_dt)
    loss = np.full(n_rays, -1, np.float32)
    rgb = np.zeros((n_rays, 3), np.float32)
    total = orc.volume_rendering_with_loss_and_gradient(a, targets, n_rays if n_active is None else n_active, idx, dt, net, dloss,
                                                        n_compacted_counter=counter0, loss_output=loss, rgb_ray_out=rgb)
    return idx, dloss, loss, rgb, total


def test_constant_density_closed_form(orc):
    n, sigma, dt_v = 40, 3.0, 0.05
    c = np.float32([0.2, 0.5, 0.9])
    net = np.tile(np.float32([c[0], c[1], c[2], sigma]), (n, 1))
    dt = np.full(n, dt_v, np.float32)
    tgt = np.float32([[0, 0, 0, 1]])
    bg = (0.3, 0.6, 0.1)
    a = loss_args(1, 1000, background_color=(O.f32 * 3)(*bg), transmittance_threshold=0.0)
    idx, dloss, loss, rgb, total = run(orc, a, [n], net, dt, tgt)
    T_N = math.exp(-sigma * dt_v * n)
    bg_lin = [v / 12.92 if v <= 0.04045 else ((v + 0.055) / 1.055) ** 2.4 for v in bg]   # the background passes through srgb_to_linear
    want = c * (1 - T_N) + T_N * np.float32(bg_lin)
    assert np.allclose(rgb[0], want, rtol=2e-6)
    assert total == n and idx[0, 0] == n and idx[0, 1] == 0
    # loss: mean over channels of (rgb - target)^2, divided by n_rays
    assert abs(loss[0] - np.mean((want - 0) ** 2)) < 1e-6


def test_early_termination_count(orc):
    # alpha ~ 1/2 per sample: T_k ~ 2^-k, and 2^-14 < 1e-4 < 2^-13, so exactly 14 samples are used
    n = 40
    net = np.tile(np.float32([1, 1, 1, math.log(2.0)]), (n, 1))
    dt = np.ones(n, np.float32)
    tgt = np.float32([[0.5, 0.5, 0.5, 1]])
    idx, dloss, loss, rgb, total = run(orc, loss_args(1, 1000), [n], net, dt, tgt)
    assert total == 14 and idx[0, 0] == 14
    assert np.allclose(rgb[0], 1 - 2.0 ** -14, rtol=1e-6)     # terminated: no background added
    assert (dloss[14:] == 7).all() and (dloss[:14] != 7).all()
    # opaque first sample: one sample; empty space: all samples, colour = background
    net2 = np.tile(np.float32([1, 1, 1, 1000.0]), (n, 1))
    assert run(orc, loss_args(1, 1000), [n], net2, dt, tgt)[4] == 1    # T becomes 0 after sample 0, which stops the loop before sample 1
    net3 = np.tile(np.float32([1, 1, 1, 0.0]), (n, 1))
    idx, dloss, loss, rgb, total = run(orc, loss_args(1, 1000, background_color=(O.f32 * 3)(1, 1, 1)), [n], net3, dt, tgt)
    assert total == n and np.allclose(rgb[0], 1.0)


def reference_forward_f64(net, dt, counts, targets, bg, rgb_act, den_act):
    """independent float64 forward: L = sum over rays and channels of (C - target)^2"""
    def act(v, kind):
        if kind == O.ACT_NONE:
            return v
        if kind == O.ACT_RELU:
            return np.maximum(v, 0)
        if kind == O.ACT_LOGISTIC:
            return 1 / (1 + np.exp(-v))
        return np.exp(v)
    L = 0.0
    s = 0
    for r, n in enumerate(counts):
        T = 1.0
        C = np.zeros(3)
        for k in range(n):
            sig = act(net[s + k, 3], den_act)
            c = act(net[s + k, :3], rgb_act)
            alpha = 1 - math.exp(-sig * dt[s + k])
            C += alpha * T * c
            T *= 1 - alpha
        C += T * bg
        t = targets[r, :3] + (1 - targets[r, 3]) * bg
        L += ((C - t) ** 2).sum()
        s += n
    return L


@pytest.mark.parametrize("rgb_act,den_act", [(O.ACT_NONE, O.ACT_NONE), (O.ACT_LOGISTIC, O.ACT_EXPONENTIAL), (O.ACT_RELU, O.ACT_RELU)])
def test_gradients_against_float64_finite_differences(orc, rgb_act, den_act):
    rng = np.random.default_rng(7)
    counts = [5, 1, 9, 3]
    n = sum(counts)
    net = np.empty((n, 4), np.float32)
    net[:, :3] = rng.random((n, 3)) * 2 - 0.5
    net[:, 3] = rng.random(n) * 2 + (0.1 if den_act != O.ACT_EXPONENTIAL else -1.0)
    dt = (rng.random(n) * 0.3 + 0.05).astype(np.float32)
    tgt = np.concatenate([rng.random((4, 3)), rng.random((4, 1))], axis=1).astype(np.float32)
    a = loss_args(4, 100, rgb_activation=rgb_act, density_activation=den_act, loss_scale=4.0, transmittance_threshold=0.0,
                  use_grid=0)
    idx, dloss, loss, rgb, total = run(orc, a, counts, net, dt, tgt)
    assert total == n
    bg = np.zeros(3)
    scale = 4.0 / 4          # loss_scale / n_rays
    net64, dt64, tgt64 = net.astype(np.float64), dt.astype(np.float64), tgt.astype(np.float64)
    eps = 1e-6
    for s in range(n):
        for c in range(4):
            hi, lo = net64.copy(), net64.copy()
            hi[s, c] += eps
            lo[s, c] -= eps
            fd = (reference_forward_f64(hi, dt64, counts, tgt64, bg, rgb_act, den_act) - reference_forward_f64(lo, dt64, counts, tgt64, bg, rgb_act, den_act)) / (2 * eps)
            assert abs(dloss[s, c] - scale * fd) <= 2e-5 * max(1.0, abs(scale * fd)), (s, c)
    # the L2 regulariser on rgb only exists for the exponential activation, the L1 on density only with use_grid and a sparse grid
    a2 = loss_args(4, 100, rgb_activation=rgb_act, density_activation=den_act, loss_scale=4.0, transmittance_threshold=0.0, use_grid=1, mean_density=0.001)
    net_neg = net.copy()
    net_neg[:, 3] = -np.abs(net_neg[:, 3]) if den_act != O.ACT_NONE else net_neg[:, 3]
    d1 = run(orc, a2, counts, net_neg, dt, tgt)[1]
    d0 = run(orc, loss_args(4, 100, rgb_activation=rgb_act, density_activation=den_act, loss_scale=4.0, transmittance_threshold=0.0, use_grid=0), counts, net_neg, dt, tgt)[1]
    neg = net_neg[:, 3] < 0
    assert np.allclose(d1[:n, 3][neg], d0[:n, 3][neg] - 1e-4, atol=1e-7)
    assert np.array_equal(d1[:n, 3][~neg], d0[:n, 3][~neg])


def test_compaction_offsets_truncation_and_counters(orc):
    rng = np.random.default_rng(3)
    counts = rng.integers(0, 12, 30)
    n = int(counts.sum())
    net = helpers.random_network_output(rng, n)
    net[:, 3] *= 8      # some rays terminate early
    dt = (rng.random(n) * 0.5 + 0.1).astype(np.float32)
    tgt = rng.random((30, 4)).astype(np.float32)
    idx, dloss, loss, rgb, total = run(orc, loss_args(30, 10000), counts, net, dt, tgt)
    used = idx[:, 0]
    assert (used <= counts).all() and (used < counts).any()
    assert np.array_equal(idx[:, 1], np.concatenate([[0], np.cumsum(used)[:-1]]))
    assert total == used.sum()
    assert (loss[used > 0] >= 0).all() and (loss[used == 0] == -1).all()
    # a starting counter shifts every offset
    idx2 = run(orc, loss_args(30, 10000), counts, net, dt, tgt, counter0=100)[0]
    assert np.array_equal(idx2[:, 1], idx[:, 1] + 100)
    # a small capacity truncates: min(cap - min(cap, base), n); the counter still runs to the full total
    cap = int(used[:10].sum() + 2)
    idx3, dloss3, _, _, total3 = run(orc, loss_args(30, cap), counts, net, dt, tgt)
    want = np.minimum(cap - np.minimum(cap, idx[:, 1]), used)
    assert np.array_equal(idx3[:, 0], want) and np.array_equal(idx3[:, 1], idx[:, 1]) and total3 == total
    assert np.array_equal(dloss3[:cap], dloss[:cap])
    # only the first n_active rays take part
    idx4, _, loss4, _, total4 = run(orc, loss_args(30, 10000), counts, net, dt, tgt, n_active=7)
    assert total4 == used[:7].sum() and np.array_equal(idx4[7:, 0], counts[7:]) and (loss4[7:] == -1).all()


def test_half_precision_io_rounds_like_numpy(orc):
    rng = np.random.default_rng(5)
    counts = [6, 4, 7]
    n = sum(counts)
    net16 = helpers.random_network_output(rng, n, np.float16)
    dt = (rng.random(n) * 0.5 + 0.1).astype(np.float32)
    tgt = rng.random((3, 4)).astype(np.float32)
    a32 = loss_args(3, 100, transmittance_threshold=0.0)
    d32 = run(orc, a32, counts, net16.astype(np.float32), dt, tgt)[1]
    a16 = loss_args(3, 100, transmittance_threshold=0.0, network_output_dtype=O.DTYPE_F16, dloss_dtype=O.DTYPE_F16)
    d16 = run(orc, a16, counts, net16, dt, tgt)[1]
    assert np.array_equal(d16[:n].view(np.uint16), d32[:n].astype(np.float16).view(np.uint16))


def test_random_background_is_shared_by_all_rays(orc):
    counts = [2, 2]
    net = np.zeros((4, 4), np.float32)     # empty space: colour = background
    dt = np.ones(4, np.float32)
    tgt = np.zeros((2, 4), np.float32)
    r = orc.pcg32(77)
    a = loss_args(2, 10, train_with_random_bg_color=1, rng=r)
    rgb = run(orc, a, counts, net, dt, tgt)[3]
    r2 = orc.pcg32(77)
    draw = [orc.next_float(r2) for _ in range(3)]
    lin = [v / 12.92 if v <= 0.04045 else ((v + 0.055) / 1.055) ** 2.4 for v in draw]
    assert np.allclose(rgb[0], lin, rtol=1e-5) and np.array_equal(rgb[0], rgb[1])


def test_inference_compositing_matches_training_forward(orc):
    """volume_rendering over chunks accumulates what the training forward pass computes in one go"""
    rng = np.random.default_rng(9)
    p = orc.params(aabb_scale=4, warping_type=O.WARP_ERP)
    n_rays, n_steps, n_chunks = 5, 4, 3
    net = helpers.random_network_output(rng, n_rays * n_steps * n_chunks).reshape(n_chunks, n_rays, n_steps, 4)
    net[..., 3] *= 0.7
    coords = np.zeros((n_chunks, n_rays, n_steps, 7), np.float32)
    coords[..., 3] = rng.random((n_chunks, n_rays, n_steps)) * 0.4 + 0.05
    pay = np.zeros(n_rays, O.PAYLOAD_DTYPE)
    pay["alive"] = 1
    rgba = np.zeros((n_rays, 4), np.float32)
    for c in range(n_chunks):
        pay["n_steps"][pay["alive"] == 1] = n_steps
        a = O.RenderArgs()
        a.n_rays, a.n_steps, a.n_steps_offset, a.padded_output_width = n_rays, n_steps, 1 + c * n_steps, 4
        a.density_activation, a.rgb_activation, a.render_mode = O.ACT_NONE, O.ACT_NONE, O.RENDER_SHADE
        a.depth_scale, a.transmittance_threshold, a.network_output_dtype = 1.0, 1e-4, O.DTYPE_F32
        orc.volume_rendering(p, a, pay, rgba, np.ascontiguousarray(coords[c]), np.ascontiguousarray(net[c]))
    for r in range(n_rays):
        T, C = 1.0, np.zeros(3)
        for c in range(n_chunks):
            for j in range(n_steps):
                alpha = 1 - math.exp(-float(net[c, r, j, 3]) * float(coords[c, r, j, 3]))
                C += alpha * T * net[c, r, j, :3].astype(np.float64)
                T *= 1 - alpha
        assert np.allclose(rgba[r, :3], C, rtol=1e-5) and abs(rgba[r, 3] - (1 - T)) < 1e-5


def test_rollover_fill(orc):
    buf = np.arange(40, dtype=np.float32).reshape(10, 4)
    orc.fill_rollover(10, 3, buf)
    assert np.array_equal(buf[3:], np.arange(12, dtype=np.float32).reshape(3, 4)[[0, 1, 2, 0, 1, 2, 0]])
    g = np.arange(20, dtype=np.float32).reshape(10, 2) + 1
    keep = g[:4].copy()
    orc.fill_rollover_and_rescale(10, 2, 4, g)
    assert np.array_equal(g[:4], keep)
    assert np.allclose(g[4:], keep[[0, 1, 2, 3, 0, 1]] * 4 / 10)
    h = g.copy()
    orc.fill_rollover_and_rescale(10, 2, 0, h)      # nothing valid: untouched
    assert np.array_equal(h, g)


def test_compact_and_shade(orc):
    n = 12
    pay = np.zeros(n, O.PAYLOAD_DTYPE)
    pay["idx"] = np.arange(n)[::-1]
    pay["alive"] = [1, 0, 0, 1, 1, 0, 0, 0, 1, 0, 1, 0]
    rgba = np.zeros((n, 4), np.float32)
    rgba[:, 3] = [0, 0.5, 0.0005, 0, 0.2, 0.9, 0.001, 0.0011, 0, 0, 0, 1]
    rgba[:, 0] = np.arange(n)
    dp, dc = np.zeros(n, O.PAYLOAD_DTYPE), np.zeros((n, 4), np.float32)
    fp, fc = np.zeros(n, O.PAYLOAD_DTYPE), np.zeros((n, 4), np.float32)
    na, nf = orc.compact_rays(n, pay, rgba, dp, dc, fp, fc, 0, 2)
    assert na == 5 and nf == 2 + 4
    assert list(dc[:na, 0]) == [0, 3, 4, 8, 10]          # survivors in order
    assert list(fc[2:nf, 0]) == [1, 5, 7, 11]            # finished rays with alpha > 0.001, appended after the 2 already there
    frame = np.full((n, 4), 0.5, np.float32)
    orc.shade(nf - 2, np.ascontiguousarray(fc[2:nf]), np.ascontiguousarray(fp[2:nf]), frame, O.RENDER_SHADE, True)
    for k, src in enumerate([1, 5, 7, 11]):
        px = int(pay["idx"][src])
        assert np.allclose(frame[px], rgba[src] + 0.5 * (1 - rgba[src, 3]))


def _unwarp_sinusoidal64(w):
    """common_device.h:508-520 in float64: inverse of the effective ("ERP" falls through to sinusoidal) warp"""
    phi = (w[1] - 0.5) * math.pi
    theta = (w[0] - 0.5) * 2 * math.pi / math.cos(phi)
    rho = 2 * w[2]
    rho = rho if rho <= 1 else 1 / (2 - rho)
    return np.array([rho * math.cos(phi) * math.cos(theta) + 0.5, rho * math.cos(phi) * math.sin(theta) + 0.5, rho * math.sin(phi) + 0.5])


@pytest.mark.parametrize("mode", [O.RENDER_AO, O.RENDER_DEPTH, O.RENDER_DISTANCE, O.RENDER_NORMALS, O.RENDER_SHADE])
def test_inference_render_modes_against_float64_formulas(orc, mode):
    """ray_marcher.cu:233-281 per render mode: what replaces the colour (alpha for AO, forward distance for Depth, Euclidean
    distance for Distance, the unit vector along -sigma' * warped_pos for Normals), early stop at alpha sum > 1 - thr, the ray
    killed with n_steps = j + offset when it consumed fewer than n_steps samples, and the un-normalised accumulator stored"""
    rng = np.random.default_rng(21 + mode)
    p = orc.params(aabb_scale=8, warping_type=O.WARP_ERP)
    n_rays, n_steps = 7, 6
    net = helpers.random_network_output(rng, n_rays * n_steps).reshape(n_rays, n_steps, 4)
    net[2, :, 3] *= 40          # ray 2 saturates early
    coords = np.zeros((n_rays, n_steps, 7), np.float32)
    coords[..., 0:3] = (rng.random((n_rays, n_steps, 3)) * 0.6 + 0.2).astype(np.float32)
    coords[..., 3] = (rng.random((n_rays, n_steps)) * 0.3 + 0.05).astype(np.float32)
    pay = np.zeros(n_rays, O.PAYLOAD_DTYPE)
    pay["alive"] = 1
    pay["alive"][5] = 0                                   # a dead ray is left alone
    pay["n_steps"] = [6, 6, 6, 4, 6, 6, 0]                # ray 3 got only 4 samples, ray 6 none
    pay["o"] = (rng.random((n_rays, 3)) * 0.2 + 0.4).astype(np.float32)
    rgba = (rng.random((n_rays, 4)) * 0.1).astype(np.float32)     # accumulators carried in from earlier chunks
    rgba0 = rgba.copy()
    cam = scene.look_at(np.array([0.4, 0.5, 0.6]), np.array([0.3, -0.5, 0.2]))
    a = O.RenderArgs()
    a.n_rays, a.n_steps, a.n_steps_offset, a.padded_output_width = n_rays, n_steps, 9, 4
    a.density_activation, a.rgb_activation, a.render_mode = O.ACT_EXPONENTIAL, O.ACT_LOGISTIC, mode
    a.camera = (O.f32 * 12)(*cam)
    a.depth_scale, a.transmittance_threshold, a.network_output_dtype = 0.7, 1e-2, O.DTYPE_F32
    net[..., 3] = np.log(net[..., 3])                     # exponential activation brings the densities back
    orc.volume_rendering(p, a, pay, rgba, coords, np.ascontiguousarray(net))
    fwd = cam[6:9].astype(np.float64)
    for r in range(n_rays):
        if r == 5:
            assert np.array_equal(rgba[r], rgba0[r]) and pay["n_steps"][r] == 6 and not pay["alive"][r]
            continue
        acc = rgba0[r].astype(np.float64)
        n_in = [6, 6, 6, 4, 6, 6, 0][r]
        j = 0
        while j < n_in:
            sigma = math.exp(float(net[r, j, 3]))
            dt = float(coords[r, j, 3])
            alpha = 1 - math.exp(-sigma * dt)
            w = alpha * (1 - acc[3])
            wp = coords[r, j, :3].astype(np.float64)
            if mode == O.RENDER_SHADE:
                c = 1 / (1 + np.exp(-net[r, j, :3].astype(np.float64)))
            elif mode == O.RENDER_AO:
                c = np.full(3, alpha)
            elif mode == O.RENDER_NORMALS:
                v = -math.exp(min(15.0, max(-15.0, float(net[r, j, 3])))) * wp
                c = v / np.linalg.norm(v)
            else:
                rel = _unwarp_sinusoidal64(wp) - pay["o"][r].astype(np.float64)
                z = (fwd @ rel if mode == O.RENDER_DEPTH else np.linalg.norm(rel)) * 0.7
                c = np.full(3, z)
            acc[:3] += c * w
            acc[3] += w
            if acc[3] > 1 - 1e-2:
                break
            j += 1
        assert np.allclose(rgba[r], acc, rtol=2e-5, atol=1e-6), (mode, r)
        if j < n_steps:
            assert not pay["alive"][r] and pay["n_steps"][r] == j + 9
        else:
            assert pay["alive"][r] and pay["n_steps"][r] == 6
    assert not pay["alive"][2] and pay["n_steps"][2] < 6 + 9         # the saturated ray stopped early
    assert not pay["alive"][3] and pay["n_steps"][3] == 4 + 9        # ran out of samples
    assert not pay["alive"][6] and pay["n_steps"][6] == 0 + 9


def test_shade_modes_against_float64_formulas(orc):
    """testbed.cu:448-477: Normals maps the normalised accumulated vector to 0.5 n + 0.5 times alpha, Cost shows n_steps / 128
    with alpha 1, Shade converts sRGB to linear unless training is in linear colours; then tmp + frame * (1 - tmp.w)"""
    rng = np.random.default_rng(33)
    n = 9
    pay = np.zeros(n, O.PAYLOAD_DTYPE)
    pay["idx"] = rng.permutation(n)
    pay["n_steps"] = rng.integers(0, 400, n)
    rgba = rng.random((n, 4)).astype(np.float32)
    rgba[0, :3] = [0.001, 0.03, 0.5]            # both branches of srgb_to_linear
    frame0 = rng.random((n, 4)).astype(np.float32)

    def srgb_to_linear(v):
        return v / 12.92 if v <= 0.04045 else ((v + 0.055) / 1.055) ** 2.4

    for mode, linear in ((O.RENDER_NORMALS, True), (O.RENDER_COST, False), (O.RENDER_SHADE, False), (O.RENDER_SHADE, True), (O.RENDER_DEPTH, False)):
        frame = frame0.copy()
        orc.shade(n, rgba, pay, frame, mode, linear)
        for i in range(n):
            tmp = rgba[i].astype(np.float64)
            if mode == O.RENDER_NORMALS:
                v = tmp[:3] / np.linalg.norm(tmp[:3])
                tmp[:3] = (0.5 * v + 0.5) * tmp[3]
            elif mode == O.RENDER_COST:
                tmp = np.array([pay["n_steps"][i] / 128.0] * 3 + [1.0])
            if not linear and mode == O.RENDER_SHADE:
                tmp[:3] = [srgb_to_linear(v) for v in tmp[:3]]
            want = tmp + frame0[pay["idx"][i]].astype(np.float64) * (1 - tmp[3])
            assert np.allclose(frame[pay["idx"][i]], want, rtol=1e-5, atol=1e-7), (mode, linear, i)


def test_distortion_side_buffer_holds_running_sums_with_unit_transmittance(orc):
    """ray_marcher.cu:142-166: per compacted sample the running sum of alpha (T stays 1 in that loop) and of alpha (j+1)/n"""
    rng = np.random.default_rng(17)
    counts = [5, 3, 6]
    n = sum(counts)
    net = helpers.random_network_output(rng, n)
    dt = (rng.random(n) * 0.3 + 0.05).astype(np.float32)
    tgt = rng.random((3, 4)).astype(np.float32)
    a = loss_args(3, 100, transmittance_threshold=0.0, regularization_type=O.REG_DISTORTION)
    idx = np.zeros((3, 2), np.uint32)
    idx[:, 0] = counts
    idx[:, 1] = np.concatenate([[0], np.cumsum(counts)[:-1]])
    reg = np.zeros((100, 2), np.float32)
    dloss = np.zeros((100, 4), np.float32)
    orc.volume_rendering_with_loss_and_gradient(a, tgt, 3, idx, dt, net, dloss, reg_buffer=reg)
    k = 0
    for c in counts:
        sw = swp = 0.0
        for j in range(c):
            alpha = 1 - math.exp(-float(net[k, 3]) * float(dt[k]))
            sw += alpha
            swp += alpha * (j + 1) / c
            assert abs(reg[k, 0] - sw) < 1e-5 and abs(reg[k, 1] - swp) < 1e-5
            k += 1
