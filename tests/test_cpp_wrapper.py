"""include/srf_hip.hpp (the C++ classes named after the reference's OccupancySampler / RayMarcher) compiled by the host
compiler against libsrf_hip.so and run as a program of its own."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "sphericalrf_amd", "lib")
EXE = os.path.join(ROOT, "tests", "cpp", "wrapper_check")


def build():
    if not os.path.exists(os.path.join(LIBDIR, "libsrf_hip.so")):
        pytest.skip("libsrf_hip.so has not been built")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "wrapper_check.cpp"),
                    "-L", LIBDIR, "-lsrf_hip", "-Wl,-rpath," + LIBDIR, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib", "-lamdhip64", "-o", EXE], check=True)


def test_wrapper_compiles_and_reports_a_missing_device_as_an_exception():
    build()
    r = subprocess.run([EXE], stdout=subprocess.PIPE, text=True, timeout=120)
    assert "strings ok" in r.stdout
    assert r.returncode in (0, 3), r.stdout          # 3: no GPU here, the constructor threw std::runtime_error as it should


@pytest.mark.gpu
def test_wrapper_runs_on_the_device(gpu):
    build()
    r = subprocess.run([EXE], stdout=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == 0 and "device ok" in r.stdout, r.stdout


# ---- the C++ snapshot loader (srf::read_snapshot / sampler_from_snapshot; Testbed::load_snapshot, internal/testbed.cu:152-171) ----
SNAPSHOT_CONFIG = {
    "samlper": dict(warping_type="ERP", aabb_scale=16, grid_size=32, num_cascades=3, grid_distribution_type="WarpedSpace_Exp", init_grid_with_mask=False,
                    maximum_marching_steps=256, sampling_type="Disparity", near_distance=0.05, far_distance=10.0, ema_decay=0.9),
    "render": dict(transmittance_threshold=1e-4), "loss": "L2", "network": {"otype": "NGPNetwork", "n_neurons": 64, "layers": [1, 2, [3, 4]]},
}


def _write(tmp_path, drop=None, network=True):
    import numpy as np
    from sphericalrf_amd import snapshot
    rng = np.random.default_rng(5)
    grid = (rng.random(3 * 32 ** 3) ** 4).astype(np.float32)
    grid[rng.random(grid.size) < 0.1] = -1.0
    path = str(tmp_path / "model.msgpack")
    # a stand-in for the trainer's serialised network: nested maps, arrays and a large binary that the loader has to step over
    net = dict(n_params=70000, params_binary=bytes(70000), params_type="__half", optimizer={"step": 3, "moments": [bytes(300), bytes(300)]}) if network else None
    snapshot.write_snapshot(path, SNAPSHOT_CONFIG, grid, scene_scale=0.33, scene_offset=(0.5, -0.25, 2.0), network=net)
    if drop:
        import msgpack
        with open(path, "rb") as f:
            cfg = msgpack.unpackb(f.read(), raw=False)
        for key in drop:
            node = cfg
            for part in key[:-1]:
                node = node[part]
            del node[key[-1]]
        with open(path, "wb") as f:
            f.write(msgpack.packb(cfg, use_bin_type=True))
    return path, grid


def test_cpp_loader_reads_what_the_python_writer_wrote(tmp_path):
    import numpy as np
    build()
    path, grid = _write(tmp_path)
    r = subprocess.run([EXE, path], stdout=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode in (0, 3), r.stdout
    line = [l for l in r.stdout.splitlines() if l.startswith("snapshot ok")][0].split()
    field = lambda name, k=1: line[line.index(name) + 1:line.index(name) + 1 + k]
    assert int(field("cells")[0]) == grid.size
    assert abs(float(field("sum")[0]) - float(grid.astype(np.float64).sum())) < 1e-3
    assert np.float32(field("scale")[0]) == np.float32(0.33) and [float(v) for v in field("offset", 3)] == [0.5, -0.25, 2.0]
    assert field("grid", 3) == ["32", "32", "32"] and field("cascades") == ["3"] and field("steps") == ["256"] and field("mask") == ["0"]
    assert field("warp") == ["4"] and field("griddist") == ["0"] and field("sampling") == ["1"] and np.float32(field("near")[0]) == np.float32(0.05)


@pytest.mark.parametrize("drop,message", [([("snapshot",)], "ERROR in loading snapshot."), ([("snapshot", "scene_scale")], "scene_scale"),
                                          ([("snapshot", "scene_offset")], "scene_offset"), ([("snapshot", "density_grid")], "density_grid"),
                                          ([("samlper",)], "samlper")])
def test_both_loaders_refuse_a_snapshot_with_a_part_missing(tmp_path, drop, message):
    from sphericalrf_amd import snapshot
    build()
    path, _ = _write(tmp_path, drop=drop, network=False)
    r = subprocess.run([EXE, path], stdout=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == 4 and message in r.stdout, r.stdout
    with pytest.raises(snapshot.SnapshotError, match=message):
        snapshot.read_snapshot(path)


def test_cpp_loader_refuses_a_truncated_file(tmp_path):
    build()
    path, _ = _write(tmp_path)
    with open(path, "rb") as f:
        raw = f.read()
    with open(path, "wb") as f:
        f.write(raw[:len(raw) // 2])
    r = subprocess.run([EXE, path], stdout=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == 4 and "ends inside a value" in r.stdout, r.stdout


@pytest.mark.gpu
def test_cpp_loader_builds_the_sampler_on_the_device(gpu, orc, tmp_path):
    """the bitfield that the C++ path rebuilds from the file has as many bits set as the oracle's (occupancy_sampler.cu:1063-1088)"""
    import numpy as np
    from tests import helpers
    build()
    path, grid = _write(tmp_path)
    p = helpers.oracle_params(orc, SNAPSHOT_CONFIG["samlper"])
    bf, _ = orc.update_grid_bitfield(p, grid)
    want = int(np.unpackbits(bf).sum())
    r = subprocess.run([EXE, path], stdout=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == 0 and ("device ok: bits set %d of %d" % (want, grid.size)) in r.stdout, r.stdout
