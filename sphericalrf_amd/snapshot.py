"""Reading (and, for tests and tools, writing) the part of a SphericalRF snapshot that the sampler needs.

A snapshot is the model configuration as msgpack (`Testbed::save_snapshot`, internal/testbed.cu:135-150: nlohmann's `json::to_msgpack`)
with a "snapshot" object added: the trainer's serialised network (not read here), `density_grid` (the sampler's float grid as one
msgpack bin: tiny-cuda-nn stores a GPUMemory<float> as a JSON binary), `scene_scale` (number) and `scene_offset` (array of three,
internal/utils/json_binding.h:14-27).  `Testbed::load_snapshot` (:152-171) assigns the grid and rebuilds the bitfield; so does
`sampler_from_snapshot`.  The file is data: it is parsed with msgpack's plain unpacker, which constructs nothing but dicts, lists,
numbers, strings and bytes.
"""
import numpy as np


class SnapshotError(RuntimeError):
    pass


def _unpack(raw):
    import msgpack
    return msgpack.unpackb(raw, raw=False, strict_map_key=False)


def read_snapshot(path):
    """-> dict(sampler=<the "samlper" block>, render=<the "render" block or {}>, loss=<str or None>, density_grid=float32 array,
    scene_scale=float, scene_offset=(x, y, z)).  Raises SnapshotError with the reference's message when the file has no snapshot."""
    with open(path, "rb") as f:
        cfg = _unpack(f.read())
    if not isinstance(cfg, dict) or "snapshot" not in cfg:
        raise SnapshotError("ERROR in loading snapshot.")          # testbed.cu:157-160
    snap = cfg["snapshot"]
    grid = snap.get("density_grid")
    if isinstance(grid, dict) and "bytes" in grid:                 # nlohmann's JSON form of a binary, should a tool have re-encoded the file
        grid = bytes(grid["bytes"])
    if not isinstance(grid, (bytes, bytearray)) or len(grid) % 4:
        raise SnapshotError("snapshot.density_grid: a binary of float32 values expected")
    if "samlper" not in cfg:
        raise SnapshotError('the snapshot holds no "samlper" block')
    if "scene_scale" not in snap or "scene_offset" not in snap:    # testbed.cu:163-164 reads both unconditionally and throws without them
        raise SnapshotError("snapshot.scene_scale and snapshot.scene_offset are required")
    offset = snap["scene_offset"]
    if not isinstance(offset, (list, tuple)) or len(offset) != 3:
        raise SnapshotError("snapshot.scene_offset: an array of three numbers expected")
    return dict(sampler=cfg["samlper"], render=cfg.get("render", {}), loss=cfg.get("loss"),
                density_grid=np.frombuffer(bytes(grid), dtype="<f4").copy(), scene_scale=float(snap["scene_scale"]),
                scene_offset=tuple(float(v) for v in offset))


def write_snapshot(path, model_config, density_grid, scene_scale=1.0, scene_offset=(0.0, 0.0, 0.0), network=None):
    """the layout `Testbed::save_snapshot` writes, without a trained network unless `network` (a dict merged into "snapshot") is given"""
    import msgpack
    cfg = dict(model_config)
    snap = dict(network or {})
    snap["density_grid"] = np.ascontiguousarray(density_grid, dtype="<f4").tobytes()
    snap["scene_scale"] = float(scene_scale)
    snap["scene_offset"] = [float(v) for v in scene_offset]
    cfg["snapshot"] = snap
    with open(path, "wb") as f:
        f.write(msgpack.packb(cfg, use_bin_type=True, use_single_float=False))


def sampler_from_snapshot(path, stream_sync=True):
    """An OccupancySampler configured by the snapshot's "samlper" block, holding its density grid, bitfield rebuilt
    (testbed.cu:165-168).  -> (sampler, snapshot dict)"""
    import torch
    from . import api
    snap = read_snapshot(path)
    s = api.OccupancySampler(snap["sampler"])
    n = int(s.n_total_elements)
    if snap["density_grid"].size != n:
        raise SnapshotError("snapshot.density_grid holds %d values, the configured grid has %d cells" % (snap["density_grid"].size, n))
    s.set_density_grid(torch.from_numpy(snap["density_grid"]).cuda())
    s.update_grid_bitfield()
    if stream_sync:
        torch.cuda.synchronize()
    return s, snap
