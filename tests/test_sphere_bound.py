"""The optional sphere bound of the marches.  The reference bounds rays by the box alone (bounding_box.h:145-180), so this has no
counterpart there and the oracle has none either; what pins it: the closed form of the quadratic (in float64), and the contract
that the bounded march keeps exactly those samples of the unbounded march -- which other tests hold to the oracle -- whose t
lies within the ray's stretch inside the sphere, without moving any of them.  Host build of the kernel bodies (tests/hostsim)."""
import ctypes as C

import numpy as np
import pytest

from tests import helpers
from tests.helpers import ptr
from oracle import oracle as O


def _spans(hostsim, rays, sphere):
    n = rays.shape[0]
    t0, t1, hit = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint8)
    hostsim.lib.hs_sphere_spans(n, ptr(np.ascontiguousarray(rays, np.float32)), ptr(np.asarray(sphere, np.float32)), ptr(t0), ptr(t1), ptr(hit))
    return t0, t1, hit.astype(bool)


def test_stretch_inside_the_sphere_is_the_quadratics_root_interval(hostsim):
    rng = np.random.default_rng(11)
    n = 20000
    o = rng.uniform(-1.5, 2.5, (n, 3))
    d = rng.normal(size=(n, 3))
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    d *= rng.uniform(0.5, 2.0, (n, 1))                 # directions need not be of unit length
    rays = np.concatenate([o, d], axis=1).astype(np.float32)
    sphere = np.array([0.5, 0.4, 0.6, 0.9], np.float32)
    t0, t1, hit = _spans(hostsim, rays, sphere)
    o64, d64 = rays[:, :3].astype(np.float64), rays[:, 3:].astype(np.float64)
    m = o64 - sphere[:3].astype(np.float64)
    a, b, c = (d64 * d64).sum(1), (m * d64).sum(1), (m * m).sum(1) - float(sphere[3]) ** 2
    disc = b * b - a * c
    clear = np.abs(disc) > 1e-3 * (b * b + a * abs(float(sphere[3]) ** 2))      # away from tangency, where float32 decides either way
    assert np.array_equal(hit[clear], disc[clear] > 0) and hit.sum() > 2000 and (~hit).sum() > 2000
    ok = hit & clear
    w0, w1 = (-b - np.sqrt(np.abs(disc))) / a, (-b + np.sqrt(np.abs(disc))) / a
    tol = 2e-5 * (np.abs(b / a) + np.sqrt(np.abs(disc)) / a + 1.0)
    assert np.all(np.abs(t0[ok] - w0[ok]) <= tol[ok]) and np.all(np.abs(t1[ok] - w1[ok]) <= tol[ok])
    # the end points lie on the sphere, the middle inside
    for t in (t0, t1):
        q = o64[ok] + t[ok, None].astype(np.float64) * d64[ok] - sphere[:3]
        assert np.all(np.abs(np.linalg.norm(q, axis=1) - float(sphere[3])) < 1e-4)
    mid = o64[ok] + (0.5 * (t0[ok].astype(np.float64) + t1[ok])).reshape(-1, 1) * d64[ok] - sphere[:3]
    assert np.all(np.linalg.norm(mid, axis=1) < float(sphere[3]))
    # a direction of length zero has no stretch
    z = np.zeros((1, 6), np.float32)
    assert not _spans(hostsim, z, sphere)[2][0]


def _train(hostsim, orc, p, ds, bf, n_rays, cap, table, wave, budget, log_words=0xffffffff):
    rc, nc = np.array([0], np.uint32), np.array([0], np.uint32)
    rays, rgba = np.zeros((n_rays, 6), np.float32), np.zeros((n_rays, 4), np.float32)
    ns = np.zeros((n_rays, 2), np.uint32)
    coords, ts, dts, cell = np.zeros((cap, 7), np.float32), np.zeros(cap, np.float32), np.zeros(cap, np.float32), np.zeros(cap, np.uint32)
    hostsim.lib.hs_generate_training_samples(C.byref(p), n_rays, 5, cap, C.byref(ds), ptr(bf), orc.pcg32(99), ptr(rc), ptr(nc),
                                             ptr(rays), ptr(rgba), ptr(ns), ptr(coords), ptr(ts), ptr(dts), ptr(cell), C.c_uint32(log_words),
                                             None if table is None else ptr(table), C.c_uint32(wave), C.c_uint32(budget))
    k = int(rc[0])
    return dict(rays=rays[:k], rgba=rgba[:k], ns=ns[:k], coords=coords, t=ts, dt=dts, cell=cell, total=int(nc[0]))


@pytest.mark.parametrize("mode", ["alone", "wavefronts", "parked", "no_log"])
@pytest.mark.parametrize("sphere", [(0.5, 0.5, 0.5, 8.0), (6.0, 0.4, 0.5, 5.0), (0.5, 0.5, 0.5, 200.0)])
def test_bounded_training_march_keeps_the_samples_inside_and_moves_none(orc, hostsim, sphere, mode):
    from tests.test_empty_space_skipping import _table
    w, p, grid, bf, mean = helpers.build_scene(orc, 3, 1 / 8)
    nb, dist = _table(orc, hostsim, p, bf)
    rng = np.random.default_rng(3)
    res = w["resolution"]
    images = rng.random((w["cameras"].shape[0] * res[0] * res[1], 4)).astype(np.float16)
    ds = orc.make_dataset(w["cameras"], res, w["focal"], (0.5, 0.5), images=images)
    n_rays, cap = 900, 1 << 20
    table, wave, budget, log_words = {"alone": (None, 0, 0, 0xffffffff), "wavefronts": (dist, 64, 0, 0xffffffff),
                                      "parked": (dist, 64, 6, 0xffffffff), "no_log": (dist, 64, 0, 0)}[mode]
    hostsim.lib.hs_set_sphere(None)
    free = _train(hostsim, orc, p, ds, bf, n_rays, cap, None, 0, 0)
    hostsim.lib.hs_set_sphere(ptr(np.asarray(sphere, np.float32)))
    try:
        got = _train(hostsim, orc, p, ds, bf, n_rays, cap, table, wave, budget, log_words)
    finally:
        hostsim.lib.hs_set_sphere(None)
    t0, t1, hit = _spans(hostsim, free["rays"], sphere)
    keep_rays, rows = [], []
    for r in range(free["rays"].shape[0]):
        n, base = free["ns"][r]
        t = free["t"][base:base + n]
        inside = hit[r] & (t >= t0[r]) & (t <= t1[r])
        if inside.any():
            keep_rays.append(r)
            rows.append(base + np.nonzero(inside)[0])
    assert len(keep_rays) == got["rays"].shape[0]
    assert np.array_equal(got["rays"].view(np.uint32), free["rays"][keep_rays].view(np.uint32))
    assert np.array_equal(got["rgba"].view(np.uint32), free["rgba"][keep_rays].view(np.uint32))
    sel = np.concatenate(rows)
    assert got["total"] == sel.size
    assert np.array_equal(got["ns"][:, 0], [len(q) for q in rows]) and np.array_equal(got["ns"][:, 1], np.cumsum([0] + [len(q) for q in rows])[:-1])
    for key in ("t", "dt", "cell", "coords"):
        assert np.array_equal(got[key][:sel.size].view(np.uint32), free[key][sel].view(np.uint32)), key
    if sphere[3] > 100:
        assert sel.size == free["total"] > 1000          # a sphere around the whole box changes nothing
    else:
        assert 200 < sel.size < free["total"]


def test_bounded_render_marches(orc, hostsim):
    """fused frame and the stepwise pair under a sphere: nothing changes when the sphere holds the box; with a small one a ray's
    coordinates are a contiguous run of its unbounded ones, rays that miss the sphere get none, and the fused frame counts the
    same samples per pixel as the stepwise march emits"""
    from sphericalrf_amd import scene
    from tests.test_empty_space_skipping import _table
    w, p, grid, bf, mean = helpers.build_scene(orc, 3, 1 / 8)
    nb, dist = _table(orc, hostsim, p, bf)
    res, f = (40, 24), (scene.focal_from_fov(40, 70.0),) * 2
    cam = np.ascontiguousarray(w["cameras"][2], dtype=np.float32)
    n, n_steps = res[0] * res[1], 96
    table = scene.field_table(1024, 5)
    table[:, 3] = 0                                        # transparent: a ray is never ended by its transmittance
    field = orc.make_field(table, 77)

    def run(sphere):
        hostsim.lib.hs_set_sphere(None if sphere is None else ptr(np.asarray(sphere, np.float32)))
        pay = np.zeros(n, O.PAYLOAD_DTYPE)
        hostsim.lib.hs_generate_rays(C.byref(p), (C.c_int32 * 2)(*res), (C.c_float * 2)(*f), (C.c_float * 2)(0.5, 0.5), ptr(cam), 0, ptr(bf), ptr(pay))
        first = pay.copy()
        coords = np.zeros((n, n_steps, 7), np.float32)
        hostsim.lib.hs_generate_coords(C.byref(p), n, n_steps, ptr(bf), ptr(pay), ptr(coords))
        frame, ns = np.zeros((res[1], res[0], 4), np.float32), np.zeros(n, np.uint32)
        hostsim.lib.hs_render_fused(C.byref(p), C.byref(field), ptr(bf), (C.c_int32 * 2)(*res), (C.c_float * 2)(*f), (C.c_float * 2)(0.5, 0.5), ptr(cam), 0,
                                    C.c_float(1e-4), 1, ptr(frame), ptr(ns))
        return first, pay, coords, frame, ns

    hostsim.lib.hs_set_render_skip_table(ptr(dist))
    try:
        free = run(None)
        big = run((0.5, 0.5, 0.5, 500.0))
        # a sphere ahead of the camera and off to one side: part of the frame's rays miss it
        fwd = free[0]["d"].mean(0) / np.linalg.norm(free[0]["d"].mean(0))
        side = free[0]["d"][res[0] - 1] - free[0]["d"][0]
        small_sphere = tuple(free[0]["o"][0] + 7.0 * fwd + 2.5 * side / np.linalg.norm(side)) + (3.0,)
        small = run(small_sphere)
    finally:
        hostsim.lib.hs_set_render_skip_table(None)
        hostsim.lib.hs_set_sphere(None)
    for a, b in zip(free, big):
        assert a.tobytes() == b.tobytes()
    first, pay, coords, frame, ns = small
    rays = np.concatenate([free[0]["o"], free[0]["d"]], axis=1)
    t0, t1, hit = _spans(hostsim, rays, small_sphere)
    started = free[0]["alive"] == 1
    count = np.where(pay["alive"] == 1, pay["n_steps"], 0)
    free_count = np.where(free[1]["alive"] == 1, free[1]["n_steps"], 0)
    assert (count[started & ~hit] == 0).all() and (ns[~hit] == 0).all() and hit.sum() > 50 and (~hit & started).sum() > 50
    assert (count <= free_count).all() and count.sum() < free_count.sum() and count.sum() > 100
    checked = 0
    for i in np.nonzero(count > 0)[0]:
        if free_count[i] >= n_steps:
            continue                                         # the unbounded ray filled its chunk: its later samples are not at hand
        mine, theirs = coords[i, :count[i]], free[2][i, :free_count[i]]
        at = [k for k in range(free_count[i] - count[i] + 1) if np.array_equal(theirs[k], mine[0])]
        assert any(np.array_equal(theirs[k:k + count[i]], mine) for k in at)
        assert first["t"][i] >= t0[i]
        checked += 1
    assert checked > 30
    # the fused frame's per-pixel sample count is the stepwise march's (no ray fills the chunk of 96 under this sphere)
    assert count.max() < n_steps and np.array_equal(ns, count)


# ---- on the GPU, through the C ABI ------------------------------------------------------------------------------------------

def _u32(t):
    return t.cpu().numpy().view(np.uint32)


@pytest.mark.gpu
def test_stretches_from_the_library_are_the_host_builds(gpu, hostsim):
    torch = gpu
    from sphericalrf_amd import api
    rng = np.random.default_rng(5)
    n = 100003
    rays = np.concatenate([rng.uniform(-3, 4, (n, 3)), rng.normal(size=(n, 3))], axis=1).astype(np.float32)
    sphere = (0.4, 0.7, 0.5, 1.3)
    t0, t1, hit = _spans(hostsim, rays, sphere)
    near, far = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    api.ray_sphere_bounds(torch.from_numpy(rays).cuda(), sphere[:3], sphere[3], near, far)
    near, far = near.cpu().numpy(), far.cpu().numpy()
    assert 0.1 < hit.mean() < 0.9
    assert np.array_equal(near[hit].view(np.uint32), t0[hit].view(np.uint32)) and np.array_equal(far[hit].view(np.uint32), t1[hit].view(np.uint32))
    assert np.all(near[~hit] == np.inf) and np.all(far[~hit] == -np.inf)
    with pytest.raises(api.SrfError, match="positive radius"):
        api.ray_sphere_bounds(torch.from_numpy(rays).cuda(), sphere[:3], 0.0, torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"))


@pytest.mark.gpu
@pytest.mark.parametrize("budget", [None, "1"])
def test_bounded_marches_on_the_gpu(gpu, orc, hostsim, budget, monkeypatch):
    """a training batch and a frame with the sphere set: the training samples are exactly the unbounded (oracle's) ones inside the
    ray's stretch, the frame and its per-pixel counts equal the host build's; taking the sphere away restores the oracle's output"""
    torch = gpu
    if budget is not None:
        monkeypatch.setenv("SRF_COUNT_PROBE_BUDGET", budget)      # every ray parked at its first lookup: the wide march under the bound
        monkeypatch.setenv("SRF_COUNT_PARK_LANES", "64")
    from sphericalrf_amd import api, scene
    from tests.test_gpu_parity import make_sampler
    w, p, grid, bf, mean = helpers.build_scene(orc, 3, 1 / 8)
    s = make_sampler(torch, api, w, grid)
    res = w["resolution"]
    o_ds = orc.make_dataset(w["cameras"], res, w["focal"], (0.5, 0.5))
    g_ds = api.Dataset(torch.from_numpy(w["cameras"]).cuda(), res, w["focal"], (0.5, 0.5))
    n_rays, cap = 6000, 1 << 22
    want = orc.generate_training_samples(p, n_rays, 3, cap, o_ds, bf, orc.pcg32(99), coords_capacity=cap)

    def sample():
        rays, rgba = torch.zeros((n_rays, 6), device="cuda"), torch.zeros((n_rays, 4), device="cuda")
        ns = torch.zeros((n_rays, 2), dtype=torch.int32, device="cuda")
        coords = torch.zeros((cap, 7), device="cuda")
        ts, dts, cell = torch.zeros(cap, device="cuda"), torch.zeros(cap, device="cuda"), torch.zeros(cap, dtype=torch.int32, device="cuda")
        rc, nc = torch.zeros(1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
        s.sample_coords_from_dataset(n_rays, 3, cap, g_ds, rays, rgba, rc, ns, coords, nc, api.Pcg32(99), ts, dts, cell)
        torch.cuda.synchronize()
        k = int(rc.item())
        return dict(rays=rays.cpu().numpy()[:k], ns=_u32(ns)[:k], coords=coords.cpu().numpy(), t=ts.cpu().numpy(), dt=dts.cpu().numpy(), cell=_u32(cell),
                    total=int(_u32(nc)[0]))

    sphere = (0.5, 0.5, 0.5, 8.0)
    s.set_ray_sphere_bound(sphere[:3], sphere[3])
    got = sample()
    k = want["ray_counter"]
    t0, t1, hit = _spans(hostsim, want["rays"][:k], sphere)
    keep_rays, rows = [], []
    for r in range(k):
        n, base = want["numsteps"][r]
        t = want["t_dt"][base:base + n, 0]
        inside = hit[r] & (t >= t0[r]) & (t <= t1[r])
        if inside.any():
            keep_rays.append(r)
            rows.append(base + np.nonzero(inside)[0])
    sel = np.concatenate(rows)
    assert 1000 < sel.size < want["numsteps_counter"] and got["total"] == sel.size
    assert np.array_equal(got["rays"].view(np.uint32), want["rays"][keep_rays].view(np.uint32))
    assert np.array_equal(got["ns"][:, 0], [len(q) for q in rows]) and np.array_equal(got["ns"][:, 1], np.cumsum([0] + [len(q) for q in rows])[:-1])
    assert np.array_equal(got["t"][:sel.size].view(np.uint32), want["t_dt"][sel, 0].view(np.uint32))
    assert np.array_equal(got["dt"][:sel.size].view(np.uint32), want["t_dt"][sel, 1].view(np.uint32))
    assert np.array_equal(got["cell"][:sel.size], want["cell"][sel])
    assert np.array_equal(got["coords"][:sel.size].view(np.uint32), want["coords"][sel].view(np.uint32))

    # a frame under a sphere that part of the rays miss, against the host build of the same march
    from tests.test_empty_space_skipping import _table
    nb, dist = _table(orc, hostsim, p, bf)
    fres, f = (64, 40), (scene.focal_from_fov(64, 70.0),) * 2
    cam = np.ascontiguousarray(w["cameras"][2], dtype=np.float32)
    n = fres[0] * fres[1]
    o_pay = orc.init_rays_with_payload(p, fres, f, (0.5, 0.5), cam)
    fwd = o_pay["d"].mean(0) / np.linalg.norm(o_pay["d"].mean(0))
    side = o_pay["d"][fres[0] - 1] - o_pay["d"][0]
    fsphere = tuple(float(v) for v in o_pay["o"][0] + 7.0 * fwd + 2.5 * side / np.linalg.norm(side)) + (3.0,)
    table = scene.field_table(1024, 5)
    table[:, 3] *= 0.3
    field = orc.make_field(table, 77)
    wf, wn = np.zeros((fres[1], fres[0], 4), np.float32), np.zeros(n, np.uint32)
    w_pay, w_coords = np.zeros(n, O.PAYLOAD_DTYPE), np.zeros((n, 8, 7), np.float32)
    hostsim.lib.hs_set_sphere(ptr(np.asarray(fsphere, np.float32)))
    hostsim.lib.hs_set_render_skip_table(ptr(dist))
    try:
        hostsim.lib.hs_render_fused(C.byref(p), C.byref(field), ptr(bf), (C.c_int32 * 2)(*fres), (C.c_float * 2)(*f), (C.c_float * 2)(0.5, 0.5), ptr(cam), 0,
                                    C.c_float(1e-4), 0, ptr(wf), ptr(wn))
        hostsim.lib.hs_generate_rays(C.byref(p), (C.c_int32 * 2)(*fres), (C.c_float * 2)(*f), (C.c_float * 2)(0.5, 0.5), ptr(cam), 0, ptr(bf), ptr(w_pay))
        hostsim.lib.hs_generate_coords(C.byref(p), n, 8, ptr(bf), ptr(w_pay), ptr(w_coords))
    finally:
        hostsim.lib.hs_set_sphere(None)
        hostsim.lib.hs_set_render_skip_table(None)
    m = api.RayMarcher(dict(train_in_linear_color=True, transmittance_threshold=1e-4))
    s.set_ray_sphere_bound(fsphere[:3], fsphere[3])
    frame, fns = torch.ones((fres[1], fres[0], 4), device="cuda"), torch.zeros(n, dtype=torch.int32, device="cuda")
    s.render_frame_fused(m, api.Field(torch.from_numpy(table).cuda(), 77), fres, f, (0.5, 0.5), cam, frame, fns)
    pay = torch.zeros(n * 40, dtype=torch.uint8, device="cuda")
    s.generate_rays_from_camera_matrix(fres, f, (0.5, 0.5), cam, pay)
    g_coords = torch.zeros((n, 8, 7), device="cuda")
    s.generate_coords_from_rays(n, 8, pay, g_coords)
    torch.cuda.synchronize()
    assert (wn > 0).mean() > 0.05 and (wn == 0).mean() > 0.05 and (wf[..., 3] > 0).any()
    assert np.array_equal(frame.cpu().numpy().view(np.uint32), wf.view(np.uint32)) and np.array_equal(_u32(fns), wn)
    g_pay = pay.cpu().numpy().view(O.PAYLOAD_DTYPE)
    alive = w_pay["alive"] == 1
    assert np.array_equal(g_pay["alive"], w_pay["alive"]) and np.array_equal(g_pay["t"][alive], w_pay["t"][alive]) and np.array_equal(g_pay["n_steps"][alive], w_pay["n_steps"][alive])
    assert np.array_equal(g_coords.cpu().numpy().view(np.uint32), w_coords.view(np.uint32))

    # without the sphere again: the oracle's batch
    s.set_ray_sphere_bound((0, 0, 0), 0.0)
    back = sample()
    assert back["total"] == want["numsteps_counter"] and np.array_equal(back["ns"], want["numsteps"][:k])
    assert np.array_equal(back["coords"][:back["total"]].view(np.uint32), want["coords"][:back["total"]].view(np.uint32))
