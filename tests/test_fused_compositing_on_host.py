"""The single-launch compositing kernel (sphericalrf_amd/csrc/srf_composite_fused.h), run group by group and phase by phase
on the host, against the oracle: every layout the kernel distinguishes (back-to-back rays, gaps left by dropped rays, rays
longer than a window, caller-shuffled offsets), bit for bit."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O
from tests import helpers
from tests.helpers import ptr
from tests.test_oracle_composite import loss_args


def layout(rng, kind, n_rays):
    if kind == "short":
        counts = rng.integers(0, 40, n_rays)
    elif kind == "long":         # rays longer than one window, and groups spanning several windows
        counts = rng.integers(0, 60, n_rays)
        counts[rng.random(n_rays) < 0.03] = rng.integers(2000, 5000)
        counts[5] = 4097
    elif kind == "split":        # groups longer than one window of the streaming kernel, cut at a ray boundary into two parts
        counts = rng.integers(25, 60, n_rays)
        counts[n_rays // 3:n_rays // 3 + 40] = rng.integers(0, 12, 40)
    elif kind == "parts":        # groups of many windows' worth of samples, none of whose rays exceeds a window: cut into several parts
        counts = rng.integers(60, 400, n_rays)
        counts[70:90] = rng.integers(1000, 1900, 20)
        counts[130:150] = 0
    elif kind == "tiny":
        counts = rng.integers(0, 3, n_rays)
    else:
        counts = rng.integers(1, 40, n_rays)
    base = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int64)
    if kind == "gaps":           # dropped rays leave holes between kept rays
        holes = (rng.random(n_rays) < 0.1) * rng.integers(1, 60, n_rays)
        base = base + np.cumsum(holes)
    if kind == "biggap":
        base[n_rays // 2:] += 500000
    if kind == "shuffled":       # what an atomicAdd-ordered sampler would hand over
        order = rng.permutation(n_rays)
        counts2, base2 = counts.copy(), base.copy()
        counts[order], base[order] = counts2, base2
    total = int((base + counts).max()) if n_rays else 0
    return counts.astype(np.uint32), base.astype(np.uint32), total


@pytest.mark.parametrize("kind", ["short", "long", "split", "parts", "tiny", "gaps", "biggap", "shuffled"])
@pytest.mark.parametrize("hin,hout", [(False, False), (True, False), (True, True)])
def test_fused_equals_oracle(orc, hostsim, kind, hin, hout):
    rng = np.random.default_rng(["short", "long", "tiny", "gaps", "biggap", "shuffled", "split", "parts"].index(kind) + 100)
    n_rays = 64 * 5 + 17
    counts, base, total = layout(rng, kind, n_rays)
    net = helpers.random_network_output(rng, total, np.float16 if hin else np.float32)
    net[:, 3] *= (0.05 if kind in ("long", "parts") else 3)
    coords = rng.random((total, 7)).astype(np.float32)
    coords[:, 3] = coords[:, 3] * 0.3 + 0.01
    tgt = rng.random((n_rays, 4)).astype(np.float32)
    n_used = int(counts.sum())
    cap = int(n_used * 0.9) + 1
    kw = dict(network_output_dtype=O.DTYPE_F16 if hin else O.DTYPE_F32, dloss_dtype=O.DTYPE_F16 if hout else O.DTYPE_F32, dt_stride=7,
              background_color=(O.f32 * 3)(0.1, 0.7, 0.3), mean_density=0.001)
    a = loss_args(n_rays, cap, **kw)
    outs = []
    for fn in ("oracle", "fused", "fused_8_parts", "wave", "wave_stride_128", "wave_stride_4096"):
        idx = np.stack([counts, base], axis=1).astype(np.uint32)
        dloss = np.zeros((cap, 4), np.float16 if hout else np.float32)
        comp = np.zeros((cap, 7), np.float32)
        loss = np.full(n_rays, -1, np.float32)
        rgb = np.zeros((n_rays, 3), np.float32)
        dt = np.ascontiguousarray(coords.ravel()[3:]) if total else np.zeros(1, np.float32)
        n_active = n_rays - 9
        if fn == "oracle":
            tot = orc.volume_rendering_with_loss_and_gradient(a, tgt, n_active, idx, dt, net, dloss, n_compacted_counter=11, coords=coords,
                                                              compacted_coords=comp, loss_output=loss, rgb_ray_out=rgb)
        elif fn.startswith("wave"):
            # the wave-per-item kernel's control flow, with the stride of the sample windows it would choose and with two forced ones
            cnt = np.array([11], np.uint32)
            paths = (C.c_uint32 * 4)()
            stride = int(fn.rsplit("_", 1)[1]) if "stride" in fn else 0
            hostsim.lib.hs_loss_wave(C.byref(a), ptr(tgt), n_active, ptr(idx), ptr(dt), ptr(coords), ptr(comp), ptr(cnt), ptr(net), ptr(dloss),
                                     ptr(loss), ptr(rgb), paths, stride)
            tot = int(cnt[0])
            in_window, chunked, per_ray, several = paths[0], paths[1], paths[2], paths[3]
            table_overflows = stride != 0 and int(base[n_active - 1] - base[0]) // stride + 1 > n_rays // 16 + 64    # (a forced stride can ask for more items than the table holds)
            if kind == "shuffled" or table_overflows:
                assert in_window == 0 and chunked == 0 and per_ray == (n_active + 63) // 64
            else:
                assert per_ray == 0 and (in_window > 0 or kind == "parts")
                if kind in ("long", "parts"):
                    assert chunked > 0
                if stride == 4096 and kind != "parts":
                    assert several > 0      # more than 64 rays start in windows of that size
                if stride == 0 and kind in ("short", "split", "gaps"):
                    assert several == 0 and chunked == 0
        else:
            # the streaming kernel's control flow, with groups cut into as many items as it takes, and into eight at most (the
            # limit of the entry point that allocates nothing: groups that need more take the path of the listed ones)
            cnt = np.array([11], np.uint32)
            ns, nm = C.c_uint32(), C.c_uint32()
            hostsim.lib.hs_fused_set_max_parts(8 if fn == "fused_8_parts" else 64)
            hostsim.lib.hs_loss_fused(C.byref(a), ptr(tgt), n_active, ptr(idx), ptr(dt), ptr(coords), ptr(comp), ptr(cnt), ptr(net), ptr(dloss),
                                      ptr(loss), ptr(rgb), C.byref(ns), C.byref(nm))
            hostsim.lib.hs_fused_set_max_parts(64)
            hostsim.lib.hs_fused_most_parts.restype = C.c_uint32
            most = hostsim.lib.hs_fused_most_parts()
            tot = int(cnt[0])
            if kind in ("shuffled", "biggap"):
                assert ns.value > 0
            else:
                assert ns.value == 0
            assert (nm.value > 0) == (kind == "long" or (kind == "parts" and fn == "fused_8_parts"))
            if kind == "split":
                assert most == 2
            if kind == "parts":
                assert most > 8 if fn == "fused" else 2 < most <= 8
        outs.append((tot, idx, dloss.view(np.uint16 if hout else np.uint32), comp, loss, rgb))
    for other in outs[1:]:
        for name, x, y in zip(("total", "idx", "dloss", "compacted_coords", "loss", "rgb"), outs[0], other):
            assert np.array_equal(x, y), name
    assert outs[0][0] > 11


def test_fused_handles_empty_and_inactive_batches(orc, hostsim):
    rng = np.random.default_rng(0)
    for n_rays, n_active in ((1, 1), (64, 0), (65, 64), (200, 3)):
        counts, base, total = layout(rng, "short", n_rays)
        net = helpers.random_network_output(rng, max(total, 1))
        dt = (rng.random(max(total, 1)) * 0.2 + 0.01).astype(np.float32)
        tgt = rng.random((n_rays, 4)).astype(np.float32)
        a = loss_args(n_rays, max(total, 1))
        res = []
        for fn in ("oracle", "fused", "wave"):
            idx = np.stack([counts, base], axis=1).astype(np.uint32)
            dloss = np.zeros((max(total, 1), 4), np.float32)
            loss = np.full(n_rays, -1, np.float32)
            rgb = np.zeros((n_rays, 3), np.float32)
            if fn == "oracle":
                tot = orc.volume_rendering_with_loss_and_gradient(a, tgt, n_active, idx, dt, net, dloss, loss_output=loss, rgb_ray_out=rgb)
            elif fn == "wave":
                cnt = np.array([0], np.uint32)
                paths = (C.c_uint32 * 4)()
                hostsim.lib.hs_loss_wave(C.byref(a), ptr(tgt), n_active, ptr(idx), ptr(dt), None, None, ptr(cnt), ptr(net), ptr(dloss), ptr(loss), ptr(rgb), paths, 0)
                tot = int(cnt[0])
            else:
                cnt = np.array([0], np.uint32)
                ns, nm = C.c_uint32(), C.c_uint32()
                hostsim.lib.hs_loss_fused(C.byref(a), ptr(tgt), n_active, ptr(idx), ptr(dt), None, None, ptr(cnt), ptr(net), ptr(dloss), ptr(loss), ptr(rgb),
                                          C.byref(ns), C.byref(nm))
                tot = int(cnt[0])
            res.append((tot, idx, dloss, loss, rgb))
        for other in res[1:]:
            for x, y in zip(res[0], other):
                assert np.array_equal(x, y)


@pytest.mark.parametrize("kind", ["split", "parts"])
def test_items_of_a_cut_group_do_not_depend_on_records_already_overwritten(orc, hostsim, kind):
    """The commit writes a ray's compacted count and offset over its record.  An item of a cut group is planned after
    the items before it have committed (always in this host build, now and then on the device), so its plan must come out
    of its own rays' records whatever the earlier rays' now hold: here offsets far above every sample index, because the
    compacted counter starts there."""
    rng = np.random.default_rng(5)
    n_rays = 64 * 3 + 11
    counts, base, total = layout(rng, kind, n_rays)
    net = helpers.random_network_output(rng, total)
    net[:, 3] *= 0.05
    dt = (rng.random(total) * 0.3 + 0.01).astype(np.float32)
    tgt = rng.random((n_rays, 4)).astype(np.float32)
    start = 0xF0000000
    cap = start      # no room behind the counter's starting value: every ray keeps nothing, so no gradient is written up there
    a = loss_args(n_rays, cap)
    res = []
    for fn in ("oracle", "fused"):
        idx = np.stack([counts, base], axis=1).astype(np.uint32)
        dloss = np.zeros((16, 4), np.float32)
        loss = np.full(n_rays, -1, np.float32)
        rgb = np.zeros((n_rays, 3), np.float32)
        if fn == "oracle":
            tot = orc.volume_rendering_with_loss_and_gradient(a, tgt, n_rays, idx, dt, net, dloss, n_compacted_counter=start, loss_output=loss, rgb_ray_out=rgb)
        else:
            cnt = np.array([start], np.uint32)
            ns, nm = C.c_uint32(), C.c_uint32()
            hostsim.lib.hs_loss_fused(C.byref(a), ptr(tgt), n_rays, ptr(idx), ptr(dt), None, None, ptr(cnt), ptr(net), ptr(dloss), ptr(loss), ptr(rgb),
                                      C.byref(ns), C.byref(nm))
            tot = int(cnt[0])
            assert ns.value == 0 and nm.value == 0
        assert not dloss.any()
        res.append((tot, idx, loss, rgb))
    for x, y in zip(res[0], res[1]):
        assert np.array_equal(x, y)
    assert res[0][0] > start and res[0][3].any()
