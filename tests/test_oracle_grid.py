"""Brute-force 3-D loops and invariants that pin the oracle's grid maintenance: splat, decayed max, mean,
threshold to bits, max-pool into coarser cascades, grid-sample generation."""
import numpy as np
import pytest

from oracle import oracle as O


def make_params(orc, N=(8, 8, 8), C=3, **kw):
    return orc.params(aabb_scale=4, grid_size=N, n_cascades=C, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_EXP,
                      sampling_type=O.SAMPLING_DISPARITY, n_max_steps=64, **kw)


def test_decayed_max_update(orc):
    rng = np.random.default_rng(0)
    g = rng.random(4096).astype(np.float32)
    g[::7] = -1.0    # masked cells stay as they are
    cur = (rng.random(4096) * 0.8).astype(np.float32)
    want = np.where(g < 0, g, np.maximum(g * np.float32(0.95), cur))
    got = g.copy()
    orc.ema_grid(cur, 0.95, got)
    assert np.array_equal(got, want)
    assert (got[g >= 0] >= g[g >= 0] * np.float32(0.95)).all()
    # from a zero grid one update reproduces the splat
    z = np.zeros(4096, np.float32)
    orc.ema_grid(cur, 0.95, z)
    assert np.array_equal(z, cur)


def test_splat_is_a_running_maximum(orc):
    p = make_params(orc)
    rng = np.random.default_rng(1)
    n = 5000
    idx = rng.integers(0, p.n_total, n).astype(np.uint32)
    dens = rng.random((n, 4)).astype(np.float32) * 50
    cur = np.zeros(p.n_total, np.float32)
    orc.splat_grid_samples(p, idx, 4, dens, O.ACT_NONE, cur)
    want = np.zeros(p.n_total, np.float32)
    np.maximum.at(want, idx, dens[:, 0] * np.float32(p.min_cone_stepsize))
    assert np.array_equal(cur, want)
    # half-precision input, exponential activation
    densh = (rng.normal(size=(n, 1))).astype(np.float16)
    cur = np.zeros(p.n_total, np.float32)
    orc.splat_grid_samples(p, idx, 1, densh, O.ACT_EXPONENTIAL, cur)
    want = np.zeros(p.n_total, np.float64)
    np.maximum.at(want, idx, np.exp(densh[:, 0].astype(np.float64)) * p.min_cone_stepsize)
    assert np.allclose(cur, want, rtol=3e-6)


@pytest.mark.parametrize("n", [64, 512, 1024, 4096, 32768])
def test_mean_is_close_to_float64_mean_and_order_is_fixed(orc, n):
    rng = np.random.default_rng(n)
    g = (rng.random(n * 2).astype(np.float32) - np.float32(0.2))
    m = orc.grid_mean(g, n)
    want = np.maximum(g[:n].astype(np.float64), 0).mean()
    assert abs(m - want) <= 2e-6 * want
    assert orc.grid_mean(g, n) == m
    # exactly representable case: all terms equal to a power of two
    h = np.full(n, 0.5, np.float32)
    assert orc.grid_mean(h, n) == np.float32(0.5)
    # negative (masked) cells contribute zero
    h[: n // 2] = -1
    assert orc.grid_mean(h, n) == np.float32(0.25)


def test_bitfield_threshold_and_layout(orc):
    rng = np.random.default_rng(2)
    g = rng.random(1024).astype(np.float32) * 0.02
    for mean, mot in ((0.5, 0.01), (0.004, 0.01)):
        bf = orc.grid_to_bitfield(g, mean, mot)
        thr = min(np.float32(mot), np.float32(mean))
        want = np.packbits((g > thr).reshape(-1, 8), axis=1, bitorder="little").ravel()
        assert np.array_equal(bf, want)


def brute_force_max_pool(prev_bits, N):
    """prev_bits: bool [Nx,Ny,Nz] of the finer cascade -> bool [Nx,Ny,Nz] contribution to the next cascade:
    each 2x2x2 block of fine cells ORs into one coarse cell at offset N/4 (centred)."""
    out = np.zeros(N, bool)
    for x in range(N[0]):
        for y in range(N[1]):
            for z in range(N[2]):
                if prev_bits[x, y, z]:
                    out[x // 2 + N[0] // 4, y // 2 + N[1] // 4, z // 2 + N[2] // 4] = True
    return out


def bits_to_3d(orc, bits, N):
    vol = np.zeros(N, bool)
    cells = np.flatnonzero(np.unpackbits(bits, bitorder="little"))
    for c in cells:
        vol[orc.morton3d_invert(int(c)), orc.morton3d_invert(int(c) >> 1), orc.morton3d_invert(int(c) >> 2)] = True
    return vol


@pytest.mark.parametrize("N", [(8, 8, 8), (16, 8, 8), (16, 16, 8)])
def test_update_grid_bitfield_against_brute_force(orc, N):
    C = 3
    p = make_params(orc, N, C)
    rng = np.random.default_rng(sum(N))
    grid = (rng.random(p.n_total) < 0.08).astype(np.float32) * (rng.random(p.n_total).astype(np.float32) + np.float32(0.05))
    bf, mean = orc.update_grid_bitfield(p, grid)
    nc = p.n_cells
    thr = min(np.float32(0.01), mean)
    level_vol = []
    for level in range(C):
        own = np.packbits((grid[level * nc:(level + 1) * nc] > thr).reshape(-1, 8), axis=1, bitorder="little").ravel()
        vol = bits_to_3d(orc, own, N)
        if level > 0:
            vol |= brute_force_max_pool(level_vol[level - 1], N)
        level_vol.append(vol)
        got = bits_to_3d(orc, bf[level * nc // 8:(level + 1) * nc // 8], N)
        assert np.array_equal(got, vol), level
    # a coarse cell is set whenever any of its 8 children in the finer cascade is set
    for level in range(1, C):
        fine = level_vol[level - 1]
        coarse = level_vol[level]
        xs, ys, zs = np.nonzero(fine)
        assert coarse[xs // 2 + N[0] // 4, ys // 2 + N[1] // 4, zs // 2 + N[2] // 4].all()


def test_grid_samples_fall_inside_their_cells(orc):
    p = make_params(orc, (8, 8, 8), 3)
    rng = np.random.default_rng(4)
    grid = rng.random(p.n_total).astype(np.float32)
    r = orc.pcg32(1234)
    n = 4000
    pos, idx = orc.generate_grid_samples(p, n, r, 3, grid, -0.01)
    assert (idx < p.n_total).all()
    C = 3
    for i in range(0, n, 17):
        level, cell = divmod(int(idx[i]), p.n_cells)
        xyz = np.array([orc.morton3d_invert(cell), orc.morton3d_invert(cell >> 1), orc.morton3d_invert(cell >> 2)])
        zoom = 2.0 ** (-(C - level - 1))
        lo = (xyz / 8 - 0.5) * zoom + 0.5
        hi = ((xyz + 1) / 8 - 0.5) * zoom + 0.5
        assert (pos[i] >= lo - 1e-6).all() and (pos[i] <= hi + 1e-6).all()
        # looking the jittered point up again finds the same cell of the same cascade (unless a finer cascade owns it)
        lvl = orc.level_from_pos(p, pos[i], pos[i])
        if lvl == level:
            assert orc.cascaded_grid_idx_at(p, pos[i], pos[i], level) == cell
    # the cell hash of the first probe is the documented one
    i = 5
    want = ((i + 3 * n) * 56924617 + 96925573) % (1 << 32) % p.n_cells
    assert int(idx[i]) % p.n_cells == want
    # with a threshold nothing passes, the tenth probe is kept
    pos2, idx2 = orc.generate_grid_samples(p, n, r, 3, grid, 2.0)
    want10 = ((i + 3 * n) * 56924617 + 9 * 19349663 + 96925573) % (1 << 32) % p.n_cells
    assert int(idx2[i]) % p.n_cells == want10


# ---- camera-visibility mask (occupancy_sampler.cu:12-102) -----------------------------------------
def _look_at(eye, target, up=(0.0, 0.0, 1.0)):
    """column-major 3x4 camera-to-world matrix: columns are the camera's x, y, z axes (z = viewing direction) and its position"""
    eye, target = np.asarray(eye, np.float64), np.asarray(target, np.float64)
    z = target - eye
    z /= np.linalg.norm(z)
    x = np.cross(z, np.asarray(up, np.float64))
    x /= np.linalg.norm(x)
    y = np.cross(z, x)
    return np.concatenate([x, y, z, eye]).astype(np.float32)


def _mask_cell_centres(orc, p, griddist, aabb_scale):
    """float64 centres and radii of all cells as the mask places them; MetricSpace_Exp is scaled and shifted twice, because the
    reference's switch falls through into the MetricSpace_Reciprocal case (occupancy_sampler.cu:52-57)"""
    N, C = np.array(p.grid_size[:3], np.float64), p.n_cascades
    centres, radii = np.empty((p.n_total, 3)), np.empty(p.n_total)
    for i in range(p.n_total):
        level, cell = divmod(i, p.n_cells)
        xyz = np.array([orc.morton3d_invert(cell), orc.morton3d_invert(cell >> 1), orc.morton3d_invert(cell >> 2)], np.float64)
        q = (xyz + 0.5) / N - 0.5
        shrink, parts = 2.0 ** (-(C - level - 1)), float(C - level)
        r = 0.5 * np.sqrt(3.0) * aabb_scale / N[0]
        if griddist == O.GRID_WARPED_EXP:
            w = q * shrink + 0.5
            q = (0.5 - 0.5 * aabb_scale) + w * aabb_scale            # the NGP warp is the affine map of the box onto the unit cube
        elif griddist == O.GRID_WARPED_RECIPROCAL:
            w = q / parts + 0.5
            q = (0.5 - 0.5 * aabb_scale) + w * aabb_scale
        elif griddist == O.GRID_METRIC_EXP:
            q = (q * aabb_scale * shrink + 0.5) * (aabb_scale / parts) + 0.5
        else:
            q = q * (aabb_scale / parts) + 0.5
        centres[i] = q
        radii[i] = r * shrink if griddist in (O.GRID_WARPED_EXP, O.GRID_METRIC_EXP) else r / parts
    return centres, radii


@pytest.mark.parametrize("griddist", [O.GRID_WARPED_EXP, O.GRID_WARPED_RECIPROCAL, O.GRID_METRIC_EXP, O.GRID_METRIC_RECIPROCAL])
def test_camera_visibility_mask_against_plane_distances(orc, griddist):
    """A cell is kept (0) when, for some camera, it lies in front of the camera and its centre is closer than the cell's radius,
    measured along the image axis, to the inside of both pairs of side planes of the viewing pyramid.  Stated here through the signed
    distances to those four planes in float64 (the planes through the camera with normals (+-1, 0, -k) and (0, +-1, -k),
    k = half the image size over the focal length); cells within 1e-4 of the decision are not judged."""
    aabb_scale = 4
    p = orc.params(aabb_scale=aabb_scale, grid_size=(8, 8, 8), n_cascades=2, warping_type=O.WARP_NGP, griddist_type=griddist,
                   sampling_type=O.SAMPLING_ORIGINAL, n_max_steps=64)
    res, focal = (64, 48), (150.0, 190.0)
    rng = np.random.default_rng(griddist + 10)
    cams = np.stack([_look_at(rng.uniform(-3, 4, 3), rng.uniform(-1, 2, 3)) for _ in range(3)])
    got = orc.mark_untrained_density_grid(p, res, focal, cams)
    assert set(np.unique(got)) <= {0.0, -1.0}
    centres, radii = _mask_cell_centres(orc, p, griddist, aabb_scale)
    seen = np.zeros(p.n_total, bool)
    unsure = np.zeros(p.n_total, bool)
    for m in cams.astype(np.float64):
        ax, ay, az, eye = m[0:3], m[3:6], m[6:9], m[9:12]
        local = centres - eye
        X, Y, Z = local @ ax, local @ ay, local @ az
        margins = [Z]
        for coord, k in ((X, res[0] * 0.5 / focal[0]), (Y, res[1] * 0.5 / focal[1])):
            norm = np.sqrt(1 + k * k)
            outside = np.maximum(coord - k * Z, -coord - k * Z) / norm       # signed distance to the nearer side plane, positive outside
            margins.append(radii / norm - outside)
        margin = np.minimum.reduce(margins)
        seen |= margin > 0
        unsure |= np.abs(margin) < 1e-4
    ok = ~unsure
    assert np.array_equal(got[ok] == 0.0, seen[ok])
    assert 0.02 < seen.mean() < 0.98 and ok.mean() > 0.98


def test_camera_visibility_mask_special_cases(orc):
    p = orc.params(aabb_scale=2, grid_size=(8, 8, 8), n_cascades=1, warping_type=O.WARP_NGP, griddist_type=O.GRID_WARPED_EXP,
                   sampling_type=O.SAMPLING_ORIGINAL, n_max_steps=64)
    centre = np.array([0.5, 0.5, 0.5])
    # no camera sees nothing
    assert (orc.mark_untrained_density_grid(p, (32, 32), (20.0, 20.0), np.zeros((0, 12), np.float32)) == -1.0).all()
    # a distant camera with a wide view that looks at the box sees every cell; turned round it sees none
    eye = centre + np.array([30.0, 0.0, 0.0])
    assert (orc.mark_untrained_density_grid(p, (32, 32), (8.0, 8.0), _look_at(eye, centre)[None]) == 0.0).all()
    assert (orc.mark_untrained_density_grid(p, (32, 32), (8.0, 8.0), _look_at(eye, 2 * eye - centre)[None]) == -1.0).all()
    # one camera that sees is enough, wherever it stands in the list
    cams = np.stack([_look_at(eye, 2 * eye - centre), _look_at(eye, centre)])
    assert (orc.mark_untrained_density_grid(p, (32, 32), (8.0, 8.0), cams) == 0.0).all()
