"""Closed-form counts, invariants and overflow semantics that pin the oracle's marching kernels."""
import numpy as np
import pytest

from oracle import oracle as O
from sphericalrf_amd import scene
from tests import helpers


def small_setup(orc, N=16, C=2, n_max_steps=64, res=(12, 10), n_cams=3, **kw):
    p = orc.params(aabb_scale=64, grid_size=(N, N, N), n_cascades=C, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_EXP,
                   sampling_type=O.SAMPLING_DISPARITY, n_max_steps=n_max_steps, near_distance=0.05, far_distance=20.0, **kw)
    cams = scene.ring_cameras(n_cams, 0.5, 15.0, 1)
    f = scene.focal_from_fov(res[0], 60.0)
    ds = orc.make_dataset(cams, res, (f, f), (0.5, 0.5))
    return p, ds, cams, res, f


def count_steps_inside(orc, p, o, d, start):
    """number of marching steps a ray takes before it leaves the box or the step collapses"""
    t = np.float32(start)
    n = 0
    while n < 100000:
        pos = (o + t * d).astype(np.float32)
        if not orc.contains(p, pos):
            break
        dt = orc.calc_dt(p, t)
        n += 1
        t = np.float32(t + dt)
        if dt == 0:
            break
    return n


def test_all_zero_bitfield_gives_no_samples(orc):
    p, ds, *_ = small_setup(orc)
    bf = np.zeros(p.n_total // 8, np.uint8)
    out = orc.generate_training_samples(p, 200, 0, 10000, ds, bf, orc.pcg32(5))
    assert out["ray_counter"] == 0 and out["numsteps_counter"] == 0


def test_all_ones_bitfield_counts_every_step_up_to_the_cap(orc):
    p, ds, *_ = small_setup(orc, n_max_steps=64)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    n_rays = 64
    out = orc.generate_training_samples(p, n_rays, 0, 1 << 20, ds, bf, orc.pcg32(5))
    assert out["ray_counter"] == n_rays
    counts = out["numsteps"][:, 0]
    assert counts.max() <= 64
    # every ray starts inside the box at t>=near and walks towards far=20 < box half-size: the number of steps is the
    # number of disparity steps from the jittered start, capped at n_max_steps
    for r in range(0, n_rays, 7):
        o, d = out["rays"][r, :3], out["rays"][r, 3:]
        b, n = int(out["numsteps"][r, 1]), int(out["numsteps"][r, 0])
        start = out["t_dt"][b, 0]
        assert n == min(64, count_steps_inside(orc, p, o, d, start))
        # consecutive samples are consecutive steps: t[k+1] = t[k] + dt[k]
        t, dt = out["t_dt"][b:b + n, 0], out["t_dt"][b:b + n, 1]
        assert np.array_equal(t[1:], (t[:-1] + dt[:-1]).astype(np.float32))
        # coords carry the warped position, dt and the warped direction
        c = out["coords"][b:b + n]
        assert np.array_equal(c[:, 3], dt)
        assert np.allclose(c[:, 4:], (d + 1) * 0.5, atol=1e-7)
        pos0 = (o + t[0] * d).astype(np.float32)
        assert np.array_equal(c[0, :3], orc.warp_position(p, pos0))


def test_without_grid_every_step_is_a_sample(orc):
    p, ds, *_ = small_setup(orc, use_grid=0)
    out = orc.generate_training_samples(p, 32, 0, 1 << 20, ds, None, orc.pcg32(5))
    assert out["ray_counter"] == 32
    assert (out["numsteps"][:, 0] == 64).all()


def test_offsets_are_the_exclusive_scan_of_counts_and_bits_are_set(orc):
    p, ds, *_ = small_setup(orc, N=16, C=2)
    rng = np.random.default_rng(0)
    bf = (rng.random(p.n_total // 8) < 0.3).astype(np.uint8) * rng.integers(1, 256, p.n_total // 8).astype(np.uint8)
    n_rays = 300
    out = orc.generate_training_samples(p, n_rays, 17, 1 << 20, ds, bf, orc.pcg32(9), ray_counter=0, numsteps_counter=0)
    nr = out["ray_counter"]
    assert 0 < nr <= n_rays
    counts, base = out["numsteps"][:nr, 0], out["numsteps"][:nr, 1]
    assert (counts > 0).all() and (counts <= p.n_max_steps).all()
    assert np.array_equal(base, np.concatenate([[0], np.cumsum(counts)[:-1]]))
    assert out["numsteps_counter"] == counts.sum()
    # source indices increase: kept rays stay in ray order
    assert (np.diff(out["src"][:nr].astype(np.int64)) > 0).all()
    # every emitted cell has its bit set
    cells = out["cell"][:out["numsteps_counter"]]
    bits = np.unpackbits(bf, bitorder="little")
    assert bits[cells].all()
    # counters continue from their starting values
    out2 = orc.generate_training_samples(p, n_rays, 17, 1 << 20, ds, bf, orc.pcg32(9), ray_counter=5, numsteps_counter=1000)
    assert out2["ray_counter"] == nr + 5 and out2["numsteps_counter"] == counts.sum() + 1000
    assert np.array_equal(out2["numsteps"][5:5 + nr, 1], base + 1000)


def test_no_occupied_step_is_missed(orc):
    """walk a ray by hand, test every step position against the bitfield, compare with what the sampler emitted"""
    p, ds, *_ = small_setup(orc, N=8, C=2, n_max_steps=48)
    rng = np.random.default_rng(3)
    bf = rng.integers(0, 256, p.n_total // 8).astype(np.uint8) & rng.integers(0, 256, p.n_total // 8).astype(np.uint8)
    out = orc.generate_training_samples(p, 40, 0, 1 << 20, ds, bf, orc.pcg32(2))
    for r in range(0, out["ray_counter"], 5):
        o, d = out["rays"][r, :3], out["rays"][r, 3:]
        b, n = int(out["numsteps"][r, 1]), int(out["numsteps"][r, 0])
        t = out["t_dt"][b, 0]
        # the first emitted sample is the first occupied step at or after the start; replay from there
        emitted = []
        while len(emitted) < n:
            pos = (o + t * d).astype(np.float32)
            if not orc.contains(p, pos):
                break
            w = orc.warp_position(p, pos)
            lvl = orc.level_from_pos(p, pos, w)
            if orc.occupied_at(p, bf, pos, w, lvl):
                emitted.append((t, orc.cascaded_grid_idx_at(p, pos, w, lvl) + lvl * p.n_cells))
            dt = orc.calc_dt(p, t)
            t = np.float32(t + dt)
            if dt == 0:
                break
        assert len(emitted) == n
        assert np.array_equal(np.float32([e[0] for e in emitted]), out["t_dt"][b:b + n, 0])
        assert np.array_equal(np.uint32([e[1] for e in emitted]), out["cell"][b:b + n])


def test_overflowing_rays_are_dropped_but_still_counted(orc):
    p, ds, *_ = small_setup(orc)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    n_rays = 50
    full = orc.generate_training_samples(p, n_rays, 0, 1 << 20, ds, bf, orc.pcg32(5))
    counts = full["numsteps"][:, 0]
    cap = int(counts[:20].sum() + counts[20] // 2)     # ray 20 does not fit
    out = orc.generate_training_samples(p, n_rays, 0, cap, ds, bf, orc.pcg32(5), coords_capacity=1 << 20)
    assert out["numsteps_counter"] == counts.sum()       # the counter keeps running past the cap
    assert out["ray_counter"] == 20                      # ray 20 and everything after it is dropped
    assert np.array_equal(out["numsteps"][:20], full["numsteps"][:20])


def test_camera_is_stratified_by_ray_index(orc):
    p, ds, cams, *_ = small_setup(orc, n_cams=4)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    n_rays = 40
    out = orc.generate_training_samples(p, n_rays, 0, 1 << 20, ds, bf, orc.pcg32(5))
    origins = out["rays"][:, :3]
    for i in range(n_rays):
        img = ((0 + i) * 4 // n_rays) % 4
        assert np.array_equal(origins[i], cams[img, 9:12])
    out = orc.generate_training_samples(p, n_rays, 23, 1 << 20, ds, bf, orc.pcg32(5))
    for i in range(n_rays):
        img = ((23 + i) * 4 // n_rays) % 4
        assert np.array_equal(out["rays"][i, :3], cams[img, 9:12])


def test_sampling_probability_zero_skips_the_ray(orc):
    p, ds, cams, res, f = small_setup(orc)
    prob = np.ones(3 * res[0] * res[1], np.float16)
    prob[: res[0] * res[1]] = 0      # camera 0 contributes nothing
    img = (np.random.default_rng(0).random((3 * res[0] * res[1], 4))).astype(np.float16)
    ds2 = orc.make_dataset(cams, res, (f, f), (0.5, 0.5), images=img, sampling_probability=prob)
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    out = orc.generate_training_samples(p, 30, 0, 1 << 20, ds2, bf, orc.pcg32(5))
    assert out["ray_counter"] == 20
    assert not any(np.array_equal(o, cams[0, 9:12]) for o in out["rays"][:20, :3])
    # targets are the pixels under the (snapped) sample positions
    r = 3
    o, d = out["rays"][r, :3], out["rays"][r, 3:]
    assert (out["rays_rgba"][r] >= 0).all() and (out["rays_rgba"][r] <= 1).all()
    flat = img.astype(np.float32)
    assert any(np.array_equal(out["rays_rgba"][r], row) for row in flat)


def test_render_rays_match_one_uninterrupted_march(orc):
    """payload init + advance + chunked generation visits the same samples whatever the chunk size"""
    p, ds, cams, res, f = small_setup(orc, N=16, C=2, n_max_steps=64)
    rng = np.random.default_rng(8)
    bf = (rng.random(p.n_total // 8) < 0.15).astype(np.uint8) * 0xff
    seqs = []
    for n_steps in (1, 3, 8):
        pay = orc.init_rays_with_payload(p, res, (f, f), (0.5, 0.5), cams[0])
        assert pay["alive"].all()
        t0 = pay["t"].copy()
        assert np.allclose(t0, np.float32(0.05) + np.float32(1e-6))
        orc.advance_pos(p, pay, bf)
        n = pay.size
        per_ray = [[] for _ in range(n)]
        for _ in range(200):
            if not pay["alive"].any():
                break
            coords = np.zeros((n, n_steps, 7), np.float32)
            orc.generate_coords_from_rays(p, n, n_steps, bf, pay, coords)
            for i in range(n):
                if pay["alive"][i]:
                    k = int(pay["n_steps"][i])
                    per_ray[i].extend(map(tuple, coords[i, :k, :4]))
                    if k < n_steps:
                        pay["alive"][i] = 0
        seqs.append(per_ray)
    # a ray that reaches the far plane inside an occupied cell is re-emitted with dt == 0 for ever: compare up to there
    def until_stuck(seq):
        out = []
        for smp in seq:
            if smp[3] == 0:
                break
            out.append(smp)
        return out
    a, b, c = ([until_stuck(r) for r in s] for s in seqs)
    assert a == b == c
    assert sum(len(r) for r in a) > 0


def _hand_walk_until_occupied(orc, p, bf, o, d, t):
    """occupancy_sampler.cu:773-794 / :827-853 by hand with the oracle's scalar helpers: returns (t, state, dt) where state
    is "occupied" (stopped at an occupied step, t not advanced), "outside" (left the box) or "stuck" (dt == 0 after t += dt)"""
    for _ in range(100000):
        pos = (o + t * d).astype(np.float32)
        if not orc.contains(p, pos):
            return t, "outside", np.float32(0)
        dt = orc.calc_dt(p, t)
        w = orc.warp_position(p, pos)
        lvl = orc.level_from_pos(p, pos, w)
        if orc.occupied_at(p, bf, pos, w, lvl):
            return t, "occupied", dt
        t = np.float32(t + dt)
        if dt == 0:
            return t, "stuck", dt
    raise AssertionError("walk did not end")


def test_render_rays_walked_by_hand(orc):
    """advance_pos and generate_coords_from_rays against a step-by-step walk written from occupancy_sampler.cu:691-863:
    start t = max(tmin, 0.05) + 1e-6, jitter ld_random_val(spp, i * 786433) * calc_dt(t0), stop AT the first occupied
    step, alive flag cleared when the ray leaves the box or the step collapses at the far plane, then n_steps samples
    per call, each {warp(pos), dt, (d + 1) / 2}, with t stored only when all n_steps were emitted."""
    res = (6, 5)
    p, ds, cams, _, _ = small_setup(orc, N=8, C=2, n_max_steps=48, res=res)
    f = scene.focal_from_fov(res[0], 60.0)
    rng = np.random.default_rng(11)
    bf = rng.integers(0, 256, p.n_total // 8).astype(np.uint8) & rng.integers(0, 256, p.n_total // 8).astype(np.uint8) & rng.integers(0, 256, p.n_total // 8).astype(np.uint8)
    for spp in (0, 3):
        pay = orc.init_rays_with_payload(p, res, (f, f), (0.5, 0.5), cams[1], spp=spp)
        n = pay.size
        assert n == 30 and pay["alive"].all()
        o_all, d_all, t0_all = pay["o"].copy(), pay["d"].copy(), pay["t"].copy()
        for i in range(n):
            tmin = orc.ray_intersect(p, o_all[i], d_all[i])[0]
            assert t0_all[i] == np.float32(np.float32(max(tmin, np.float32(0.05))) + np.float32(1e-6))
            assert pay["idx"][i] == i and pay["n_steps"][i] == 0
        orc.advance_pos(p, pay, bf, spp=spp)
        walked = []
        for i in range(n):
            t0 = t0_all[i]
            start = np.float32(t0 + np.float32(np.float32(orc.ld_random_val(spp, (i * 786433) & 0xffffffff)) * orc.calc_dt(p, t0)))
            t, state, dt = _hand_walk_until_occupied(orc, p, bf, o_all[i], d_all[i], start)
            walked.append((t, state))
            assert pay["t"][i] == t, (i, pay["t"][i], t)
            assert bool(pay["alive"][i]) == (state == "occupied")
        assert any(s == "occupied" for _, s in walked) and any(s != "occupied" for _, s in walked)
        # the jitter really is there: some start differs from t0
        assert any(np.float32(orc.ld_random_val(spp, (i * 786433) & 0xffffffff)) != 0 for i in range(n))

        n_steps = 3
        coords = np.full((n, n_steps, 7), np.nan, np.float32)
        before = pay.copy()
        orc.generate_coords_from_rays(p, n, n_steps, bf, pay, coords)
        n_checked = 0
        for i in range(n):
            if not before["alive"][i]:
                assert pay["t"][i] == before["t"][i] and np.isnan(coords[i]).all()
                continue
            t = before["t"][i]
            emitted, ended = [], False
            for j in range(n_steps):
                t, state, dt = _hand_walk_until_occupied(orc, p, bf, o_all[i], d_all[i], t)
                if state != "occupied":
                    ended = True
                    break
                pos = (o_all[i] + t * d_all[i]).astype(np.float32)
                emitted.append(np.concatenate([orc.warp_position(p, pos), [dt], ((d_all[i] + np.float32(1)) * np.float32(0.5)).astype(np.float32)]).astype(np.float32))
                t = np.float32(t + dt)
            k = len(emitted)
            assert pay["n_steps"][i] == k
            assert np.array_equal(coords[i, :k], np.array(emitted, np.float32).reshape(k, 7))
            assert np.isnan(coords[i, k:]).all()              # nothing is written past the last sample
            if ended:
                assert pay["t"][i] == before["t"][i]          # the kernel returns without storing t
                assert k < n_steps
            else:
                assert pay["t"][i] == t
            assert pay["alive"][i]                            # this kernel never clears the flag (volume_rendering does)
            n_checked += k
        assert n_checked > 10


def test_render_ray_that_starts_outside_the_box_is_dead(orc):
    """a camera outside the box looking away: ray_intersect gives {1e5, 1e5}-like misses and o + t d is not contained"""
    res = (4, 4)
    p, ds, cams, _, _ = small_setup(orc, N=8, C=1, res=res)
    f = scene.focal_from_fov(res[0], 60.0)
    cam = scene.look_at(np.array([0.5 + 100.0, 0.5, 0.5]), np.array([1.0, 0.0, 0.0]))
    pay = orc.init_rays_with_payload(p, res, (f, f), (0.5, 0.5), cam)
    assert not pay["alive"].any()
    assert np.array_equal(pay["o"], np.tile(cam[9:12], (16, 1)))
    bf = np.full(p.n_total // 8, 0xff, np.uint8)
    before = pay.copy()
    orc.advance_pos(p, pay, bf)
    assert np.array_equal(pay.view(np.uint8), before.view(np.uint8))


def test_render_ray_reaching_far_inside_empty_space_dies_with_dt_zero(orc):
    """far plane inside the box, nothing occupied: the disparity step collapses to 0 at t >= far and advance_pos clears the flag"""
    res = (3, 3)
    p, ds, cams, _, _ = small_setup(orc, N=8, C=1, res=res, n_max_steps=16)
    f = scene.focal_from_fov(res[0], 60.0)
    bf = np.zeros(p.n_total // 8, np.uint8)
    pay = orc.init_rays_with_payload(p, res, (f, f), (0.5, 0.5), cams[0])
    orc.advance_pos(p, pay, bf)
    assert not pay["alive"].any()
    assert (pay["t"] >= np.float32(p.far_distance)).all() and (pay["t"] < np.float32(p.far_distance) + 1).all()
    assert all(orc.calc_dt(p, t) == 0 for t in pay["t"])
