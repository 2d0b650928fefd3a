"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the oracle must keep reproducing
them (CPU), and the HIP library must reproduce them through the C ABI without the oracle in the loop (GPU)."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from tests import helpers
from tests.golden import make_fixtures as mf

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLD, name + ".npz"), allow_pickle=False)


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


@pytest.mark.parametrize("name", sorted(mf.MARCH_CASES))
def test_oracle_reproduces_march_fixture(orc, name):
    f = load(name)
    got = mf.march_fixture(orc, *mf.MARCH_CASES[name])
    for k in ("bitfield", "rays", "numsteps", "coords", "t_dt", "cell"):
        assert same_bits(got[k], f[k]), k
    assert got["ray_counter"] == int(f["ray_counter"]) and got["numsteps_counter"] == int(f["numsteps_counter"])


def test_oracle_reproduces_composite_and_grid_fixtures(orc):
    f = load("composite_fp16_l2")
    got = mf.composite_fixture(orc)
    for k in ("idx_out", "dloss", "loss", "rgb"):
        assert same_bits(got[k], f[k]), k
    assert got["total"] == int(f["total"])
    f = load("grid_update")
    got = mf.grid_fixture(orc)
    for k in ("grid", "bitfield"):
        assert same_bits(got[k], f[k]), k
    assert np.float32(got["mean"]) == f["mean"]


def test_fixtures_are_not_degenerate():
    f = load("march_w3")
    assert int(f["numsteps_counter"]) > 2000 and len(np.unique(f["cell"])) > 500
    offs = f["numsteps"]
    assert np.array_equal(offs[1:, 1], np.cumsum(offs[:-1, 0], dtype=np.uint32) + offs[0, 1])   # offsets = exclusive scan of counts
    f = load("composite_fp16_l2")
    assert 0 < int(f["total"]) - int(f["counter_start"]) <= int(f["cap"]) and np.abs(f["dloss"]).max() > 0
    assert (f["idx_out"][:, 0] < f["idx_in"][:, 0]).any()      # some rays terminate early or hit the cap


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(mf.MARCH_CASES))
def test_gpu_reproduces_march_fixture(gpu, name):
    torch = gpu
    from sphericalrf_amd import api, scene
    f = load(name)
    w = scene.workload(int(f["config_id"]), float(f["scale"]))
    centres, sigmas = scene.blob_set(**w["blobs"])
    gs = w["sampler"]["grid_size"]
    gs = (gs,) * 3 if isinstance(gs, int) else gs
    grid = scene.density_grid_from_blobs(gs, w["sampler"]["num_cascades"], centres, sigmas, w["occupancy"], w["shell"], w["seed"])
    s = api.OccupancySampler(w["sampler"])
    s.set_density_grid(grid.cuda())
    s.update_grid_bitfield()
    assert same_bits(s.density_grid_bitfield.cpu().numpy(), f["bitfield"])
    n_rays, cap = int(f["n_rays"]), int(f["cap"])
    ds = api.Dataset(torch.from_numpy(w["cameras"]).cuda(), w["resolution"], w["focal"], (0.5, 0.5))
    rays = torch.zeros((n_rays, 6), device="cuda")
    rgba = torch.zeros((n_rays, 4), device="cuda")
    ns = torch.zeros((n_rays, 2), dtype=torch.int32, device="cuda")
    coords = torch.zeros((cap, 7), device="cuda")
    ts, dts = torch.zeros(cap, device="cuda"), torch.zeros(cap, device="cuda")
    cell = torch.zeros(cap, dtype=torch.int32, device="cuda")
    rc = torch.zeros(1, dtype=torch.int32, device="cuda")
    nc = torch.zeros(1, dtype=torch.int32, device="cuda")
    s.sample_coords_from_dataset(n_rays, int(f["shift"]), cap, ds, rays, rgba, rc, ns, coords, nc, api.Pcg32(int(f["seed"])), ts, dts, cell)
    torch.cuda.synchronize()
    n_r, n_s = int(rc.item()), int(nc.item())
    assert n_r == int(f["ray_counter"]) and n_s == int(f["numsteps_counter"])
    assert same_bits(rays.cpu().numpy()[:n_r], f["rays"])
    assert same_bits(ns.cpu().numpy().view(np.uint32)[:n_r], f["numsteps"])
    assert same_bits(cell.cpu().numpy().view(np.uint32)[:n_s], f["cell"])
    assert same_bits(coords.cpu().numpy()[:n_s], f["coords"])
    assert same_bits(np.stack([ts.cpu().numpy(), dts.cpu().numpy()], axis=1)[:n_s], f["t_dt"])


@pytest.mark.gpu
@pytest.mark.parametrize("impl", ["stream", "unfused"])
def test_gpu_reproduces_composite_fixture(gpu, impl, monkeypatch):
    torch = gpu
    from sphericalrf_amd import api
    monkeypatch.setenv("SRF_COMPOSITE_IMPL", impl)
    f = load("composite_fp16_l2")
    n_rays, cap = int(f["n_rays"]), int(f["cap"])
    m = api.RayMarcher(dict(train_with_random_bg_color=False, train_in_linear_color=True, transmittance_threshold=1e-4))
    idx = torch.from_numpy(f["idx_in"].view(np.int32).copy()).cuda()
    dloss = torch.zeros((cap, 4), device="cuda")
    loss, rgb = torch.zeros(n_rays, device="cuda"), torch.zeros((n_rays, 3), device="cuda")
    cnt = torch.full((1,), int(f["counter_start"]), dtype=torch.int32, device="cuda")
    nrc = torch.full((1,), int(f["n_active"]), dtype=torch.int32, device="cuda")
    m.volume_rendering_with_loss_and_gradient(n_rays, cap, torch.from_numpy(f["targets"]).cuda(), nrc, idx, torch.from_numpy(f["dt"]).cuda(),
                                              torch.from_numpy(f["net"]).cuda(), dloss, cnt, loss_output=loss, loss_scale=128.0,
                                              density_grid_mean=torch.ones(1, device="cuda"), use_grid=True, dt_stride=1, rgb_ray_out=rgb,
                                              rgb_activation=api.ACT_NONE, density_activation=api.ACT_NONE, loss_type="L2",
                                              background_color=(0, 0, 0), color_space=api.COLOR_LINEAR, rng=None)
    m.sync_check()
    assert int(cnt.item()) == int(f["total"])
    assert same_bits(idx.cpu().numpy().view(np.uint32), f["idx_out"])
    assert same_bits(dloss.cpu().numpy(), f["dloss"]) and same_bits(loss.cpu().numpy(), f["loss"]) and same_bits(rgb.cpu().numpy(), f["rgb"])


@pytest.mark.gpu
def test_gpu_reproduces_grid_fixture(gpu):
    torch = gpu
    from sphericalrf_amd import api
    f = load("grid_update")
    cfg = dict(warping_type="ERP", aabb_scale=16, grid_size=tuple(int(v) for v in f["grid_size"]), num_cascades=int(f["n_cascades"]),
               grid_distribution_type="WarpedSpace_Exp", init_grid_with_mask=False, maximum_marching_steps=256, sampling_type="Disparity",
               near_distance=0.05, far_distance=10.0)
    s = api.OccupancySampler(cfg)
    s.set_density_grid(torch.from_numpy(f["grid"]).cuda())
    s.update_grid_bitfield()
    torch.cuda.synchronize()
    assert same_bits(s.density_grid_bitfield.cpu().numpy(), f["bitfield"])
    assert s.density_grid_mean.cpu().numpy()[0] == f["mean"]
