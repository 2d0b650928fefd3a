"""The snapshot reader against files in the layout Testbed::save_snapshot writes (internal/testbed.cu:135-171)."""
import struct

import numpy as np
import pytest

from sphericalrf_amd import snapshot


def _hand_packed(grid_bytes):
    """msgpack bytes put together by hand, the way nlohmann::json::to_msgpack emits this document: fixmaps, fixstrs, a bin32 for
    the grid, float32 where the value is exactly representable (scene_scale 0.5), float64 otherwise (0.1), fixarray of three"""
    def s(t):
        b = t.encode()
        return bytes([0xa0 | len(b)]) + b
    samlper = bytes([0x83]) + s("warping_type") + s("ERP") + s("grid_size") + bytes([0x08]) + s("num_cascades") + bytes([0x02])
    snap = (bytes([0x83]) + s("density_grid") + b"\xc6" + struct.pack(">I", len(grid_bytes)) + grid_bytes
            + s("scene_scale") + b"\xca" + struct.pack(">f", 0.5)
            + s("scene_offset") + bytes([0x93]) + b"\xca" + struct.pack(">f", 0.25) + b"\xcb" + struct.pack(">d", 0.1) + b"\xca" + struct.pack(">f", -2.0))
    return bytes([0x83]) + s("samlper") + samlper + s("loss") + s("Huber") + s("snapshot") + snap


def test_reads_a_document_packed_the_way_the_reference_packs_it(tmp_path):
    grid = (np.arange(2 * 8 ** 3, dtype=np.float32) * 0.001 - 0.2)
    p = tmp_path / "snap.msgpack"
    p.write_bytes(_hand_packed(grid.astype("<f4").tobytes()))
    snap = snapshot.read_snapshot(str(p))
    assert snap["sampler"] == {"warping_type": "ERP", "grid_size": 8, "num_cascades": 2} and snap["loss"] == "Huber"
    assert np.array_equal(snap["density_grid"], grid) and snap["density_grid"].dtype == np.float32
    assert snap["scene_scale"] == 0.5 and snap["scene_offset"] == (0.25, 0.1, -2.0)


def test_round_trip_and_errors(tmp_path):
    cfg = {"samlper": {"warping_type": "ERP", "grid_size": [16, 8, 8], "num_cascades": 3}, "render": {"train_in_linear_color": False}, "loss": "L2"}
    grid = np.random.default_rng(0).random(3 * 16 * 8 * 8).astype(np.float32)
    p = tmp_path / "a.msgpack"
    snapshot.write_snapshot(str(p), cfg, grid, scene_scale=0.33, scene_offset=(0.5, 0.5, 0.5), network={"params_binary": b"\x00" * 64})
    snap = snapshot.read_snapshot(str(p))
    assert snap["sampler"] == cfg["samlper"] and snap["render"] == cfg["render"]
    assert np.array_equal(snap["density_grid"], grid) and snap["scene_scale"] == 0.33 and snap["scene_offset"] == (0.5, 0.5, 0.5)
    import msgpack
    q = tmp_path / "b.msgpack"
    q.write_bytes(msgpack.packb(cfg))
    with pytest.raises(snapshot.SnapshotError, match="ERROR in loading snapshot."):
        snapshot.read_snapshot(str(q))
    q.write_bytes(msgpack.packb(dict(cfg, snapshot={"density_grid": [1.0, 2.0]})))
    with pytest.raises(snapshot.SnapshotError, match="binary of float32"):
        snapshot.read_snapshot(str(q))


@pytest.mark.gpu
def test_sampler_from_snapshot_rebuilds_the_bitfield(gpu, orc, tmp_path):
    from oracle.support import oracle_params
    cfg = {"samlper": dict(warping_type="ERP", aabb_scale=16, grid_size=[16, 8, 8], num_cascades=3, grid_distribution_type="WarpedSpace_Exp",
                           init_grid_with_mask=False, maximum_marching_steps=128, sampling_type="Disparity")}
    p = oracle_params(orc, cfg["samlper"])
    grid = (np.random.default_rng(1).random(p.n_total) * 0.03).astype(np.float32)
    path = tmp_path / "s.msgpack"
    snapshot.write_snapshot(str(path), cfg, grid, scene_scale=0.5)
    s, snap = snapshot.sampler_from_snapshot(str(path))
    want_bf, want_mean = orc.update_grid_bitfield(p, grid)
    assert np.array_equal(s.density_grid.cpu().numpy(), grid)
    assert np.array_equal(s.density_grid_bitfield.cpu().numpy(), want_bf) and s.density_grid_mean.cpu().numpy()[0] == want_mean
    bad = tmp_path / "bad.msgpack"
    snapshot.write_snapshot(str(bad), cfg, grid[:-8])
    with pytest.raises(snapshot.SnapshotError, match="cells"):
        snapshot.sampler_from_snapshot(str(bad))
