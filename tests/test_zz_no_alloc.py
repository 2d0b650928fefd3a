"""The training compositing entry point that allocates nothing
(srf_marcher_volume_rendering_with_loss_and_gradient_noalloc) against the ordinary entry point: same inputs through
both, outputs compared bit for bit (integers and float bit patterns), on two calls in a row, the second with a smaller
input, so that what the first call left in the library's built-in scratch must not matter."""
import numpy as np
import pytest

from tests.test_fused_compositing_on_host import layout

pytestmark = pytest.mark.gpu


def _inputs(torch, seed, n_rays, kind):
    rng = np.random.default_rng(seed)
    counts, base, total = layout(rng, kind, n_rays)
    net = rng.random((total, 4)).astype(np.float16)
    net[:, 3] *= np.float16(3)
    dt = (rng.random(total) * 0.3 + 0.01).astype(np.float32)
    tgt = rng.random((n_rays, 4)).astype(np.float32)
    coords = rng.random((total, 7)).astype(np.float32)
    idx = np.stack([counts, base], axis=1).astype(np.uint32)
    cap = int(counts.sum() * 0.9) + 1          # smaller than what the rays keep: the clamp is exercised too
    dev = lambda x: torch.from_numpy(x).cuda()
    return dict(n_rays=n_rays, total=total, cap=cap, idx=idx, net=dev(net), dt=dev(dt), tgt=dev(tgt), coords=dev(coords))


def _buffers(torch, w):
    n_rays, cap = w["n_rays"], w["cap"]
    return dict(idx=torch.from_numpy(w["idx"].view(np.int32)).cuda(), dloss=torch.zeros((cap, 4), device="cuda"), compacted=torch.zeros((cap, 7), device="cuda"),
                loss=torch.full((n_rays,), -1.0, device="cuda"), rgb=torch.zeros((n_rays, 3), device="cuda"),
                cnt=torch.full((1,), 5, dtype=torch.int32, device="cuda"), nrc=torch.full((1,), n_rays - 3, dtype=torch.int32, device="cuda"),
                mean=torch.full((1,), 0.001, device="cuda"))


def _call(api, marcher, w, b, no_alloc):
    marcher.volume_rendering_with_loss_and_gradient(w["n_rays"], w["cap"], w["tgt"], b["nrc"], b["idx"], w["dt"], w["net"], b["dloss"], b["cnt"], rgb_activation=api.ACT_LOGISTIC,
                                                    density_activation=api.ACT_EXPONENTIAL, loss_output=b["loss"], loss_type="SMAPE", density_grid_mean=b["mean"],
                                                    use_grid=True, background_color=(0.2, 0.4, 0.6), coords=w["coords"], compacted_coords=b["compacted"],
                                                    rgb_ray_out=b["rgb"], no_alloc=no_alloc)
    marcher.sync_check()


def _run(torch, api, marcher, w, no_alloc):
    b = _buffers(torch, w)
    _call(api, marcher, w, b, no_alloc)
    return [b[k].cpu().numpy().view(np.uint32) for k in ("cnt", "idx", "dloss", "compacted", "loss", "rgb")]


def test_no_alloc_entry_point_matches_the_ordinary_one_twice_in_a_row(gpu, monkeypatch):
    torch = gpu
    from sphericalrf_amd import api
    monkeypatch.delenv("SRF_COMPOSITE_IMPL", raising=False)
    cfg = dict(train_with_random_bg_color=True, train_in_linear_color=False)
    ordinary, no_alloc = api.RayMarcher(cfg), api.RayMarcher(cfg)
    first = _inputs(torch, 41, 64 * 900 + 17, "gaps")      # several segments of items, holes between rays
    second = _inputs(torch, 42, 64 * 40 + 5, "split")      # smaller, with groups that are cut into two items
    third = _inputs(torch, 45, 64 * 30 + 7, "parts")       # groups of many windows: cut into items by one entry point, beyond the other's limit of eight
    for w in (first, second, third):
        want = _run(torch, api, ordinary, w, False)
        got = _run(torch, api, no_alloc, w, True)
        assert int(want[0][0]) > 5
        for x, y in zip(want, got):
            assert np.array_equal(x, y)


def test_no_alloc_entry_point_leaves_the_free_device_memory_alone(gpu, monkeypatch):
    """After one call per device (which looks up the scratch symbol and the kernel's occupancy), a call with more rays than any
    before changes the device's free memory by nothing, where the ordinary entry point's growing workspace is seen to."""
    torch = gpu
    from sphericalrf_amd import api
    monkeypatch.delenv("SRF_COMPOSITE_IMPL", raising=False)
    cfg = dict(train_with_random_bg_color=True, train_in_linear_color=False)
    no_alloc, ordinary = api.RayMarcher(cfg), api.RayMarcher(cfg)
    small, large = _inputs(torch, 43, 64 * 30, "short"), _inputs(torch, 44, 64 * 4000 + 3, "short")
    b_small, b_large = _buffers(torch, small), _buffers(torch, large)
    _call(api, no_alloc, small, b_small, True)
    _call(api, ordinary, small, b_small, False)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _call(api, no_alloc, large, b_large, True)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_after == free_before
    _call(api, ordinary, large, b_large, False)       # the control: this one has to grow its workspace (about 19 bytes a ray)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] < free_after


def test_no_alloc_entry_point_rejects_what_it_cannot_serve(gpu, monkeypatch):
    torch = gpu
    from sphericalrf_amd import api, _capi
    monkeypatch.delenv("SRF_COMPOSITE_IMPL", raising=False)
    n_rays = api.NOALLOC_MAX_RAYS + 1
    z = lambda *shape, dtype=torch.float32: torch.zeros(shape, dtype=dtype, device="cuda")
    args = (n_rays, 16, z(n_rays, 4), z(1, dtype=torch.int32), z(n_rays, 2, dtype=torch.int32), z(16), z(16, 4, dtype=torch.float16), z(16, 4), z(1, dtype=torch.int32))
    with pytest.raises(_capi.SrfError, match="SRF_NOALLOC_MAX_RAYS"):
        api.RayMarcher({}).volume_rendering_with_loss_and_gradient(*args, density_grid_mean=z(1), no_alloc=True)
    with pytest.raises(_capi.SrfError, match="distortion"):
        api.RayMarcher(dict(regularization_type="Distortion")).volume_rendering_with_loss_and_gradient(64, *args[1:], density_grid_mean=z(1), no_alloc=True)
