"""Synthetic scenes standing in for datasets and for the network: camera rigs, Gaussian-blob
occupancy evaluated at the cells of the warped cascaded grid, lookup tables of density and
colour.  Everything is seeded and computed with numpy in float64/float32 on the host so that
the same arrays feed the oracle and the HIP library.

Scene coordinates follow the reference: the warp is centred at (0.5, 0.5, 0.5)
(internal/utils/common_device.h:434); cameras are column-major 3x4 {right, down, forward,
origin}, i.e. what spec_opengl_to_opencv (common_device.h:123-141) makes of the OpenGL
matrices script/trajectory/generate_spherical_trajectory.py:22-51 writes.
"""
import math

import numpy as np

CENTRE = np.array([0.5, 0.5, 0.5], dtype=np.float64)


def focal_from_fov(resolution_x, fov_degrees):
    """fov_to_focal_length, internal/utils/common_device.h:105-107"""
    return float(np.float32(0.5) * np.float32(resolution_x) / np.float32(math.tan(0.5 * math.radians(fov_degrees))))


def look_at(position, forward, up=(0.0, 0.0, 1.0)):
    """column-major 3x4 camera {right, down, forward, origin} looking along `forward`"""
    f = np.asarray(forward, np.float64)
    f = f / np.linalg.norm(f)
    u = np.asarray(up, np.float64)
    r = np.cross(f, u)
    if np.linalg.norm(r) < 1e-8:
        r = np.cross(f, np.array([0.0, 1.0, 0.0]))
    r = r / np.linalg.norm(r)
    d = np.cross(f, r)
    return np.concatenate([r, d, f, np.asarray(position, np.float64)]).astype(np.float32)


def single_camera(radius=1.0):
    """config 1: one camera on the radius-`radius` sphere looking at the centre"""
    direction = np.array([0.6, -0.64, 0.48])
    direction /= np.linalg.norm(direction)
    pos = CENTRE + radius * direction
    return look_at(pos, CENTRE - pos)[None, :]


def hemisphere_cameras(n, radius, seed):
    """config 2: n inward-facing cameras on the upper hemisphere (Fibonacci spiral, seeded start angle)"""
    rng = np.random.default_rng(seed)
    phase = rng.random() * 2 * math.pi
    cams = []
    for k in range(n):
        z = (k + 0.5) / n              # cos(polar) in (0, 1): upper hemisphere
        s = math.sqrt(max(0.0, 1 - z * z))
        a = phase + k * math.pi * (3 - math.sqrt(5))
        direction = np.array([s * math.cos(a), s * math.sin(a), z])
        pos = CENTRE + radius * direction
        cams.append(look_at(pos, CENTRE - pos))
    return np.stack(cams)


def ring_cameras(n, radius, pitch_degrees, seed):
    """config 3: n cameras on a ring of the given radius in the z = 0.5 plane, looking outward with seeded pitch jitter"""
    rng = np.random.default_rng(seed)
    pitch = np.radians((rng.random(n) * 2 - 1) * pitch_degrees)
    cams = []
    for k in range(n):
        a = 2 * math.pi * k / n
        radial = np.array([math.cos(a), math.sin(a), 0.0])
        fwd = math.cos(pitch[k]) * radial + math.sin(pitch[k]) * np.array([0.0, 0.0, 1.0])
        cams.append(look_at(CENTRE + radius * radial, fwd))
    return np.stack(cams)


def _morton_invert(idx):
    def inv(x):
        x = x & 0x49249249
        x = (x | (x >> 2)) & 0xc30c30c3
        x = (x | (x >> 4)) & 0x0f00f00f
        x = (x | (x >> 8)) & 0xff0000ff
        x = (x | (x >> 16)) & 0x0000ffff
        return x
    return inv(idx), inv(idx >> 1), inv(idx >> 2)


def cell_centres_metric(grid_size, n_cascades, level, cells):
    """Metric-space centres of the given Morton cells (int64 torch tensor) of one cascade, for the sinusoidal warp and
    a WarpedSpace_Exp grid.  Returns (xyz float64 [n,3], reachable mask, warped radius); warped points whose azimuth
    falls outside [-pi, pi] are never produced by the forward warp and are flagged unreachable."""
    import torch
    ix, iy, iz = _morton_invert(cells)
    scale = 2.0 ** (-(n_cascades - level - 1))
    wx = ((ix.double() + 0.5) / grid_size[0] - 0.5) * scale + 0.5
    wy = ((iy.double() + 0.5) / grid_size[1] - 0.5) * scale + 0.5
    wz = ((iz.double() + 0.5) / grid_size[2] - 0.5) * scale + 0.5
    phi = (wy - 0.5) * math.pi
    cphi = torch.cos(phi)
    theta = (wx - 0.5) * 2 * math.pi / torch.clamp(cphi, min=1e-12)
    reach = theta.abs() <= math.pi
    rho = 2 * wz
    rho = torch.where(rho <= 1, rho, 1.0 / torch.clamp(2 - rho, min=1e-9))
    xyz = torch.stack([rho * cphi * torch.cos(theta) + 0.5, rho * cphi * torch.sin(theta) + 0.5, rho * torch.sin(phi) + 0.5], dim=-1)
    return xyz, reach, wz, ix, iy


def blob_set(n_blobs, max_radius, sigma_range, seed, n_satellites=0, satellite_radius=(1.2, 4.0), satellite_sigma=0.06):
    """Isotropic Gaussian blobs: `n_blobs` with centres uniform in the ball of `max_radius` around the scene centre, plus
    `n_satellites` further out (radius uniform in `satellite_radius`, sigma proportional to the radius)."""
    rng = np.random.default_rng(seed)
    n = n_blobs + n_satellites
    direction = rng.normal(size=(n, 3))
    direction /= np.linalg.norm(direction, axis=1, keepdims=True)
    r = max_radius * rng.random(n) ** (1 / 3)
    sigmas = sigma_range[0] + (sigma_range[1] - sigma_range[0]) * rng.random(n)
    if n_satellites:
        rs = satellite_radius[0] + (satellite_radius[1] - satellite_radius[0]) * rng.random(n_satellites)
        r[n_blobs:] = rs
        sigmas[n_blobs:] = satellite_sigma * rs
        direction[n_blobs:, 2] *= 0.35      # keep them near the cameras' horizon
        direction[n_blobs:] /= np.linalg.norm(direction[n_blobs:], axis=1, keepdims=True)
    centres = CENTRE + direction * r[:, None]
    return centres, sigmas


def density_grid_from_blobs(grid_size, n_cascades, centres, sigmas, occupancy, shell=None, shell_seed=0, device="cpu"):
    """float32 torch grid (cascade-major, Morton order inside a cascade) holding 1 in occupied cells and 0 elsewhere.

    A cell is occupied when the blob density at its centre is among the top `occupancy` fraction of the reachable cells
    of its cascade (`occupancy` a float) or exceeds an absolute level (`occupancy` = ("level", value)), or when it lies
    in the optional shell (warped radius lo, hi, angular coverage in [0,1]) of the
    outermost cascade, patterned by a seeded hash of coarse angular tiles.  `device` only selects where the arithmetic
    runs; the result is meant to be fed, as data, to both the oracle and the HIP library.
    """
    import torch
    n_cells = int(grid_size[0]) * int(grid_size[1]) * int(grid_size[2])
    grid = torch.zeros(n_cells * n_cascades, dtype=torch.float32, device=device)
    c_t = torch.as_tensor(centres, dtype=torch.float64, device=device)
    s_t = torch.as_tensor(sigmas, dtype=torch.float64, device=device)
    chunk = 1 << 22
    for level in range(n_cascades):
        dens = torch.empty(n_cells, dtype=torch.float32, device=device)
        extra = torch.zeros(n_cells, dtype=torch.bool, device=device)
        reach_all = torch.empty(n_cells, dtype=torch.bool, device=device)
        for s0 in range(0, n_cells, chunk):
            cells = torch.arange(s0, min(n_cells, s0 + chunk), dtype=torch.int64, device=device)
            xyz, reach, wz, ix, iy = cell_centres_metric(grid_size, n_cascades, level, cells)
            acc = torch.zeros(cells.numel(), dtype=torch.float64, device=device)
            for k in range(c_t.shape[0]):
                d2 = ((xyz - c_t[k]) ** 2).sum(dim=1)
                acc += torch.exp(-d2 / (2 * s_t[k] * s_t[k]))
            acc[~reach] = 0
            dens[s0:s0 + cells.numel()] = acc.float()
            reach_all[s0:s0 + cells.numel()] = reach
            if shell is not None and level == n_cascades - 1:
                lo, hi, cover = shell
                tile = (ix // max(1, grid_size[0] // 32)) * 7919 + (iy // max(1, grid_size[1] // 16)) * 104729 + int(shell_seed)
                tile = ((tile ^ (tile >> 15)) * 0x2c1b3c6d) & 0xffffffff
                tile = (tile ^ (tile >> 12)) & 0xffff
                extra[s0:s0 + cells.numel()] = (wz >= lo) & (wz <= hi) & reach & (tile < int(cover * 65536))
        occ = extra
        if isinstance(occupancy, tuple):
            occ = occ | ((dens > float(occupancy[1])) & reach_all)
        else:
            k = int(occupancy * int(reach_all.sum()))
            if k > 0:
                thr = torch.topk(dens, k, sorted=True).values[-1]
                occ = occ | ((dens >= thr) & (dens > 0) & reach_all)
        grid[level * n_cells:(level + 1) * n_cells] = occ.float()
    return grid


def field_table(size, seed):
    """(size, 4) float32 rows of (r, g, b, sigma): rgb ~ U(0,1), sigma ~ softplus(N(0,1))"""
    rng = np.random.default_rng(seed)
    t = np.empty((size, 4), np.float32)
    t[:, :3] = rng.random((size, 3), dtype=np.float32)
    z = rng.normal(size=size)
    t[:, 3] = np.log1p(np.exp(z)).astype(np.float32)
    return t


# ---- the five workloads ------------------------------------------------------------------------
def workload(config_id, scale=1.0):
    """Sampler/marcher settings, cameras and scene recipe of one of the five workloads.

    `scale` < 1 shrinks image sizes, camera counts and grids (powers of two) for quick tests; 1.0 is the full size.
    """
    def p2(v):
        return max(4, 1 << int(round(math.log2(max(1.0, v * scale)))))

    base = dict(warping_type="ERP", aabb_scale=64, use_grid=True, init_grid_with_mask=False, grid_distribution_type="WarpedSpace_Exp",
                cone_angle_constant=0.0, far_distance=100.0, sampling_type="Disparity", ema_decay=0.95, min_optical_thickness=0.01,
                snap_to_pixel_centers_in_training=True, snap_to_pixel_centers_in_rendering=True)
    if config_id == 1:
        res = (max(8, int(256 * scale)),) * 2
        return dict(sampler=dict(base, grid_size=p2(64), num_cascades=1, maximum_marching_steps=256, near_distance=0.1),
                    cameras=single_camera(1.0), resolution=res, focal=(focal_from_fov(res[0], 50.0),) * 2,
                    blobs=dict(n_blobs=8, max_radius=0.8, sigma_range=(0.12, 0.3), seed=44), occupancy=0.10, shell=None, seed=44)
    if config_id == 2:
        res = (max(8, int(800 * scale)),) * 2
        return dict(sampler=dict(base, grid_size=p2(128), num_cascades=1, maximum_marching_steps=1024, near_distance=0.05),
                    cameras=hemisphere_cameras(max(2, int(100 * scale)), 4.0, 45), resolution=res, focal=(focal_from_fov(res[0], 40.0),) * 2,
                    blobs=dict(n_blobs=32, max_radius=1.5, sigma_range=(0.08, 0.25), seed=45), occupancy=0.03, shell=None, seed=45)
    if config_id in (3, 4, 5):
        res = (max(16, int(1280 * scale)), max(9, int(720 * scale))) if config_id != 5 else (max(16, int(1920 * scale)), max(9, int(1080 * scale)))
        n = p2(256)
        return dict(sampler=dict(base, grid_size=(2 * n, n, n), num_cascades=5, maximum_marching_steps=2048, near_distance=0.05),
                    cameras=ring_cameras(max(2, int(200 * scale)), 0.5, 15.0, 46), resolution=res, focal=(focal_from_fov(res[0], 60.0),) * 2,
                    blobs=dict(n_blobs=48, max_radius=0.3, sigma_range=(0.04, 0.08), seed=46, n_satellites=16, satellite_sigma=0.09),
                    occupancy=("level", 0.3), shell=(0.9, 1.0, 0.66), seed=46)
    raise ValueError("config_id must be 1..5")


# ---- workload files for the native (torch-free) step driver -------------------------------------
def sampler_config_struct(cfg):
    """the "samlper" dict as the C struct srf_sampler_config (include/srf_hip.h), through the same mapping api.OccupancySampler uses"""
    from . import api
    return api.sampler_config_from_dict(cfg)


def write_workload_file(path, config_id, bitfield, scale=1.0, table_rows=1 << 16):
    """Writes what tests/cpp/step_bench.cpp reads: magic, srf_sampler_config, cameras, image size and focal length, the occupancy
    bitfield (numpy uint8, cascade-major) and a (table_rows, 4) table of (r, g, b, sigma) rows."""
    import ctypes
    import struct
    w = workload(config_id, scale)
    c = sampler_config_struct(w["sampler"])
    raw = bytes(ctypes.string_at(ctypes.addressof(c), ctypes.sizeof(c)))
    cams = np.ascontiguousarray(w["cameras"], np.float32)
    bits = np.ascontiguousarray(bitfield, np.uint8)
    table = field_table(table_rows, 50 + config_id)
    with open(path, "wb") as f:
        f.write(b"SRFWLD01")
        f.write(struct.pack("<I", len(raw)))
        f.write(raw)
        f.write(struct.pack("<Iiiff", cams.shape[0], int(w["resolution"][0]), int(w["resolution"][1]), float(w["focal"][0]), float(w["focal"][1])))
        f.write(cams.tobytes())
        f.write(struct.pack("<I", bits.size))
        f.write(bits.tobytes())
        f.write(struct.pack("<I", table.shape[0]))
        f.write(table.tobytes())
    return path


def _main():
    """python -m sphericalrf_amd.scene --config 4 --out FILE: builds the workload's grid on the GPU, lets the HIP library turn it
    into the bitfield, and writes the workload file."""
    import argparse
    import torch
    from . import api
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, default=4)
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--out", required=True)
    a = ap.parse_args()
    w = workload(a.config, a.scale)
    centres, sigmas = blob_set(**w["blobs"])
    gs = w["sampler"]["grid_size"]
    gs = (gs,) * 3 if isinstance(gs, int) else gs
    grid = density_grid_from_blobs(gs, w["sampler"]["num_cascades"], centres, sigmas, w["occupancy"], w["shell"], w["seed"], device="cuda")
    s = api.OccupancySampler(w["sampler"])
    s.set_density_grid(grid)
    s.update_grid_bitfield()
    torch.cuda.synchronize()
    bits = s.density_grid_bitfield.cpu().numpy()
    write_workload_file(a.out, a.config, bits, a.scale)
    print("%s: config %d, %d bitfield bytes, %.4f of bits set" % (a.out, a.config, bits.size, float(np.unpackbits(bits).mean())))


if __name__ == "__main__":
    _main()
