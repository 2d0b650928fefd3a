#!/usr/bin/env python3
"""Benchmark of the sampling / marching / compositing path on one MI355X.

A "step" is one training step of workload 4: march a batch of 2^20 rays drawn from the 200 ring cameras through the
512x256x256 x 5-cascade occupancy bitfield into a sample buffer capped at 2^24, then composite forward + backward
(fp16 density/colour per sample, fp32 target per ray, L2 loss, fp32 gradients).  Inputs are resident in HBM before the
timed region.  The one JSON line printed on stdout carries the headline metric (marched samples per second over whole
steps), the roofline of the compositing kernels (the HBM-bound part the path is specified against) and a CPU baseline:
the oracle timed on this machine's host cores on a bounded slice of the same workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras]

Under "extras" the same line carries the other workloads, each with a roofline block of its own from its algorithmic bytes: one
frame each of workloads 1, 2, 3 and 5 (fused kernel, and the reference's loop of entry points), workload 5's grid update in both
point orders (the draw of the first 256 steps and the steady-state draw), workload 4 in drop-in mode (Coordinate records written by
the march and compacted by the compositing, as the reference's caller needs them) and workload 4 on a grid with about 15 % of its
bits set, where the batch wants far more than the 2^24 samples there is room for.  --no-extras leaves them out.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
COMPOSITE_BYTES_PER_SAMPLE = 28  # read fp16 rgb-sigma 8 + fp32 dt 4, write fp32 gradients 16
COMPOSITE_BYTES_PER_RAY = 36     # read (count, offset) 8 + target 12, write rgb 12 + loss 4
MARCH_BYTES_PER_SAMPLE = 12      # write t, dt, cell
MARCH_BYTES_PER_RAY = 32         # read ray 24, write (count, offset) 8
# HBM bytes per launch of the compositing kernel at this workload come from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of the native
# harness, scaled by a plain copy of known size; counters cannot be read from inside this process, so the figure is read from the
# committed summary of those runs (None when the file or the line is missing)
COMPOSITE_TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "compositing_config4_hbm_traffic.txt")
EMA_BYTES_PER_CELL = 12
BITFIELD_BYTES_PER_CELL = 4.125
RENDER_BYTES_PER_SAMPLE = 20     # forward-only compositing: read fp32 rgb-sigma 16 + fp32 dt 4
RENDER_BYTES_PER_RAY = 16        # write RGBA
COORD_BYTES = 28                 # one Coordinate record (drop-in mode: written by the march, read and written again by the compositing)


def roofline(kernel, n_bytes, seconds):
    gbs = n_bytes / seconds / 1e9
    return {"kernel": kernel, "bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
            "algorithmic_bytes": n_bytes}


def composite_traffic_bytes():
    try:
        m = re.search(r"^composite_traffic_bytes_per_launch\s*=\s*([0-9.eE+]+)\s*$", open(COMPOSITE_TRAFFIC_PROFILE).read(), re.M)
        return float(m.group(1)) if m else None
    except OSError:
        return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_sampler(torch, api, scene, w, device="cuda"):
    centres, sigmas = scene.blob_set(**w["blobs"])
    gs = w["sampler"]["grid_size"]
    gs = (gs,) * 3 if isinstance(gs, int) else gs
    grid = scene.density_grid_from_blobs(gs, w["sampler"]["num_cascades"], centres, sigmas, w["occupancy"], w["shell"], w["seed"], device=device)
    s = api.OccupancySampler(w["sampler"])
    s.set_density_grid(grid)
    s.update_grid_bitfield()
    torch.cuda.synchronize()
    return s, grid


def timed(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_training_step(torch, api, scene, steps, warmup, n_rays=1 << 20, cap=1 << 24, drop_in=False, shell=None):
    """drop_in: the march also writes the reference's Coordinate records and the compositing copies those of the samples it keeps
    (what Testbed::train hands to the network and its backward pass); shell: replaces the workload's shell (lo, hi, coverage)"""
    w = scene.workload(4)
    if shell is not None:
        w = dict(w, shell=shell)
    t0 = time.perf_counter()
    s, grid = build_sampler(torch, api, scene, w)
    log("scene built in %.1f s" % (time.perf_counter() - t0))
    del grid
    bits = s.density_grid_bitfield
    occupied_bits = sum(float(torch.bitwise_and(bits >> k, 1).float().mean()) for k in range(8)) / 8
    m = api.RayMarcher(dict(train_with_random_bg_color=False, train_in_linear_color=True, transmittance_threshold=1e-4))
    cams = torch.from_numpy(w["cameras"]).cuda()
    ds = api.Dataset(cams, w["resolution"], w["focal"], (0.5, 0.5))
    dev = "cuda"
    rays = torch.zeros((n_rays, 6), device=dev)
    rays_rgba = torch.zeros((n_rays, 4), device=dev)
    ray_idx = torch.zeros((n_rays, 2), dtype=torch.int32, device=dev)
    sample_t = torch.zeros(cap, device=dev)
    sample_dt = torch.zeros(cap, device=dev)
    sample_cell = torch.zeros(cap, dtype=torch.int32, device=dev)
    coords = torch.zeros((cap, 7), device=dev) if drop_in else None
    compacted_coords = torch.zeros((cap, 7), device=dev) if drop_in else None
    n_rays_counter = torch.zeros(1, dtype=torch.int32, device=dev)
    n_coords_counter = torch.zeros(1, dtype=torch.int32, device=dev)
    n_compacted = torch.zeros(1, dtype=torch.int32, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(47)
    net = torch.empty((cap, 4), dtype=torch.float16, device=dev)
    net[:, :3] = torch.rand((cap, 3), generator=g, device=dev).half()
    net[:, 3] = torch.nn.functional.softplus(torch.randn(cap, generator=g, device=dev)).half()
    targets = torch.rand((n_rays, 4), generator=g, device=dev)
    targets[:, 3] = 1.0
    dloss = torch.zeros((cap, 4), device=dev)
    loss = torch.zeros(n_rays, device=dev)
    rgb_out = torch.zeros((n_rays, 3), device=dev)
    rng = api.Pcg32(43)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    times = {"march": [], "composite": []}
    state = {"shift": 0}
    rng_last = [None]           # the generator as the last step's march saw it

    def step(record=False):
        n_rays_counter.zero_()
        n_coords_counter.zero_()
        n_compacted.zero_()
        if record:
            ev[0].record()
        s.sample_coords_from_dataset(n_rays, state["shift"], cap, ds, rays, rays_rgba, n_rays_counter, ray_idx, coords, n_coords_counter, rng,
                                     sample_t, sample_dt, sample_cell)
        if record:
            ev[1].record()
        m.volume_rendering_with_loss_and_gradient(n_rays, cap, targets, n_rays_counter, ray_idx, sample_dt, net, dloss, n_compacted,
                                                  rgb_activation=api.ACT_NONE, density_activation=api.ACT_NONE, loss_output=loss, loss_type="L2",
                                                  loss_scale=128.0, density_grid_mean=s.density_grid_mean, use_grid=True, dt_stride=1, rgb_ray_out=rgb_out,
                                                  coords=coords, compacted_coords=compacted_coords)
        if record:
            ev[2].record()
            torch.cuda.synchronize()
            times["march"].append(ev[0].elapsed_time(ev[1]))
            times["composite"].append(ev[1].elapsed_time(ev[2]))
        state["shift"] += n_rays
        rng_last[0] = api.Pcg32(0)
        rng_last[0].state, rng_last[0].inc = rng.state, rng.inc
        rng.advance()

    step()
    torch.cuda.synchronize()
    n_kept, n_samples, n_comp = int(n_rays_counter.item()), int(n_coords_counter.item()) & 0xffffffff, int(n_compacted.item()) & 0xffffffff
    log("first step: rays kept %d / %d, samples %d (cap %d), compacted %d" % (n_kept, n_rays, n_samples, cap, n_comp))
    sec = timed(torch, step, steps, warmup)
    # per-part times over separate instrumented steps (event records around each entry point, on the stream they run on)
    for _ in range(max(3, min(steps, 10))):
        step(record=True)
    n_kept, n_wanted, n_comp = int(n_rays_counter.item()), int(n_coords_counter.item()) & 0xffffffff, int(n_compacted.item()) & 0xffffffff
    # the samples of the rays that were kept: the counter itself keeps growing past the capacity (occupancy_sampler.cu:638-642)
    # (read after a march on its own: the compositing overwrites the per-ray counts with the compacted ones)
    n_rays_counter.zero_()
    n_coords_counter.zero_()
    state["shift"] -= n_rays
    s.sample_coords_from_dataset(n_rays, state["shift"], cap, ds, rays, rays_rgba, n_rays_counter, ray_idx, coords, n_coords_counter, rng_last[0],
                                 sample_t, sample_dt, sample_cell)
    n_samples = int(ray_idx[:n_kept, 0].long().sum().item())
    march_ms = sum(times["march"]) / len(times["march"])
    comp_ms = sum(times["composite"]) / len(times["composite"])
    comp_bytes = COMPOSITE_BYTES_PER_SAMPLE * n_samples + COMPOSITE_BYTES_PER_RAY * n_kept
    march_bytes = MARCH_BYTES_PER_SAMPLE * n_samples + MARCH_BYTES_PER_RAY * n_rays
    if drop_in:
        comp_bytes += COORD_BYTES * (n_samples + n_comp)       # the kept samples' records read, the compacted ones written
        march_bytes += COORD_BYTES * n_samples
    info = s.info
    return dict(sec_per_step=sec, n_rays=n_rays, n_kept=n_kept, n_samples=n_samples, n_samples_wanted=n_wanted, n_compacted=n_comp, march_ms=march_ms, composite_ms=comp_ms,
                composite_bytes=comp_bytes, march_bytes=march_bytes,
                composite_gbs=comp_bytes / (comp_ms * 1e-3) / 1e9, march_gbs=march_bytes / (march_ms * 1e-3) / 1e9,
                n_max_steps=int(info.n_max_steps), workload=w, sampler=s, occupied_bits=occupied_bits)


def cpu_baseline(result, bf, n_rays_sample=1 << 16):
    """the oracle on a slice of the same workload: the first n_rays_sample rays of a batch, march + compositing fwd/bwd;
    bf: the workload's bitfield in host memory"""
    import numpy as np
    from oracle import oracle as O
    from oracle import support as helpers
    from oracle.support import loss_args
    orc = O.get()
    w = result["workload"]
    p = helpers.oracle_params(orc, w["sampler"])
    ds = orc.make_dataset(w["cameras"], w["resolution"], w["focal"], (0.5, 0.5))
    cap = n_rays_sample * 32
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        out = orc.generate_training_samples(p, n_rays_sample, 0, cap, ds, bf, orc.pcg32(43), want_coords=False, coords_capacity=cap)
        t1 = time.perf_counter()
        n_s, n_r = out["numsteps_counter"], out["ray_counter"]
        rng = np.random.default_rng(0)
        net = helpers.random_network_output(rng, n_s, np.float16)
        tgt = rng.random((n_rays_sample, 4)).astype(np.float32)
        dloss = np.zeros((n_s, 4), np.float32)
        a = loss_args(n_rays_sample, n_s, network_output_dtype=O.DTYPE_F16)
        idx = out["numsteps"].copy()
        dt = np.ascontiguousarray(out["t_dt"][:, 1])
        t2 = time.perf_counter()
        orc.volume_rendering_with_loss_and_gradient(a, tgt, n_r, idx, dt, net, dloss)
        t3 = time.perf_counter()
        tot = (t1 - t0) + (t3 - t2)
        if best is None or tot < best[0]:
            best = (tot, t1 - t0, t3 - t2, n_s, n_r)
    tot, t_march, t_comp, n_s, n_r = best
    return dict(value=n_s / tot, unit="marched samples/s", cores=orc.max_threads(), kind="port",
                sample="first %d rays of one 2^20-ray batch of workload 4 (%d samples): march %.2f s + compositing fwd/bwd %.3f s, best of 2, OpenMP over rays"
                       % (n_rays_sample, n_s, t_march, t_comp),
                march_samples_per_s=n_s / t_march, composite_samples_per_s=n_s / t_comp)


def bench_render(torch, api, scene, config_id, steps, warmup, n_frames=2):
    w = scene.workload(config_id)
    s, _ = build_sampler(torch, api, scene, w)
    m = api.RayMarcher(dict(train_in_linear_color=True, transmittance_threshold=1e-4))
    res = w["resolution"]
    n = res[0] * res[1]
    table = torch.from_numpy(scene.field_table(1 << 16, 50 + config_id)).cuda()
    field = api.Field(table, 1000 + config_id)
    frame = torch.zeros((res[1], res[0], 4), device="cuda")
    ns = torch.zeros(n, dtype=torch.int32, device="cuda")
    cams = w["cameras"]
    k = {"i": 0}

    def step():
        s.render_frame_fused(m, field, res, w["focal"], (0.5, 0.5), cams[k["i"] % len(cams)], frame, ns)
        k["i"] += 1

    sec = timed(torch, step, steps, warmup)
    total = int(ns.long().sum().item())
    # the same frames through the reference's loop of entry points run inside the library (srf_render_frame), the table as the network
    rounds = {"n": 0}

    def loop_step():
        rounds["n"] = s.render_frame(m, field, res, w["focal"], (0.5, 0.5), cams[k["i"] % len(cams)], frame, density_activation=api.ACT_NONE,
                                     rgb_activation=api.ACT_NONE, network_output_dtype=api.DTYPE_F32)
        k["i"] += 1

    k["i"] = 0
    loop_sec = timed(torch, loop_step, steps, warmup)

    def paced_step():       # the same loop with the rounds' numbers kept on the device
        rounds["n"] = s.render_frame(m, field, res, w["focal"], (0.5, 0.5), cams[k["i"] % len(cams)], frame, density_activation=api.ACT_NONE,
                                     rgb_activation=api.ACT_NONE, network_output_dtype=api.DTYPE_F32, paced=True)
        k["i"] += 1

    k["i"] = 0
    paced_sec = timed(torch, paced_step, steps, warmup)
    bits = s.density_grid_bitfield
    occ = float(torch.from_numpy(__import__("numpy").unpackbits(bits.cpu().numpy())).float().mean())
    n_bytes = RENDER_BYTES_PER_SAMPLE * total + RENDER_BYTES_PER_RAY * n
    return dict(workload="render_%d" % config_id, resolution=list(res), ms_per_frame=sec * 1e3, rays_per_s=n / sec, composited_samples_last_frame=total,
                samples_per_s=total / sec, loop_ms_per_frame=loop_sec * 1e3, paced_loop_ms_per_frame=paced_sec * 1e3, loop_rounds_last_frame=rounds["n"], occupied_bits=occ,
                frames_in_workload=len(cams),
                roofline=roofline("whole frame in one kernel: march + forward compositing (bytes: what the reference's loop moves per composited sample and per ray; "
                                  "the fused kernel itself keeps them in registers and is bound by the march's instruction issue)", n_bytes, sec),
                loop_roofline=roofline("the same frame through srf_render_frame's rounds of compact / generate_coords / inference / volume_rendering", n_bytes, loop_sec),
                paced_loop_roofline=roofline("the same rounds with their sizes kept on the device (srf_render_frame_paced)", n_bytes, paced_sec))


def bench_grid_update(torch, api, scene, steps, warmup, cell_order=False, steady_state=False):
    w = scene.workload(5)
    s = api.OccupancySampler(w["sampler"])
    s.set_grid_sample_order(cell_order)
    s.init(1, w["resolution"], w["focal"], (0.5, 0.5), None, None, api.Pcg32(43))
    n_total = int(s.n_total_elements)
    # the reference's draw of its first 256 steps (one uniform point per cell) or of the steps after (a quarter each way)
    n_uni, n_non = (n_total // 4, n_total // 4) if steady_state else (n_total, 0)
    n_points = n_uni + n_non
    pos = torch.zeros((n_points, 3), device="cuda")
    idx = torch.zeros(n_points, dtype=torch.int32, device="cuda")
    g = torch.Generator(device="cuda")
    g.manual_seed(48)
    dens = torch.nn.functional.softplus(torch.randn(n_points, generator=g, device="cuda")).half()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    parts = {"sample_positions": [], "update_grid": [], "update_grid_bitfield": []}

    def step(record=False):
        if record:
            ev[0].record()
        s.sample_positions_from_grid(n_uni, n_non, pos, idx)
        if record:
            ev[1].record()
        s.update_grid(n_points, 1, dens, idx, api.ACT_NONE)
        if record:
            ev[2].record()
        s.update_grid_bitfield()
        if record:
            ev[3].record()
            torch.cuda.synchronize()
            for j, name in enumerate(parts):
                parts[name].append(ev[j].elapsed_time(ev[j + 1]))

    sec = timed(torch, step, steps, warmup)
    for _ in range(3):
        step(record=True)
    avg = {k: sum(v) / len(v) for k, v in parts.items()}
    import numpy as np
    occ = float(np.unpackbits(s.density_grid_bitfield.cpu().numpy()).mean())
    return dict(workload="grid_update_5" + ("_steady_state" if steady_state else "") + ("_cell_order" if cell_order else ""), cells=n_total, points=n_points,
                ms_per_update=sec * 1e3, parts_ms=avg, occupied_bits=occ,
                update_grid_gbs=EMA_BYTES_PER_CELL * n_total / (avg["update_grid"] * 1e-3) / 1e9,
                bitfield_gbs=BITFIELD_BYTES_PER_CELL * n_total / (avg["update_grid_bitfield"] * 1e-3) / 1e9,
                roofline=roofline("update_grid + update_grid_bitfield (12.125 B per cell: density 4 + grid read 4 + grid write 4 + bit 1/8)",
                                  (EMA_BYTES_PER_CELL + 0.125) * n_total, (avg["update_grid"] + avg["update_grid_bitfield"]) * 1e-3))


def bench_grid_sample_draws(torch, api, scene, steps):
    """sample_positions_from_grid on workload 5's trained-looking (sparse) grid: the reference's first-256-steps mode (all
    points uniform), its steady-state mode (a quarter uniform, a quarter looking for cells above the threshold) and all
    points of the second kind"""
    w = scene.workload(5)
    s, grid = build_sampler(torch, api, scene, w)
    del grid
    n = int(s.n_total_elements)
    pos = torch.zeros((n, 3), device="cuda")
    idx = torch.zeros(n, dtype=torch.int32, device="cuda")
    out = {}
    for name, (n_uni, n_non) in (("all_uniform", (n, 0)), ("steady_state", (n // 4, n // 4)), ("all_nonuniform", (0, n))):
        out[name] = timed(torch, lambda: s.sample_positions_from_grid(n_uni, n_non, pos, idx), max(2, steps), 1) * 1e3
    return dict(workload="grid_sample_draws_5", cells=n, ms=out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-extras", action="store_true", help="only the headline workload (the other workloads under \"extras\" take about a minute)")
    ap.add_argument("--all", action="store_true", help="accepted for older command lines: the extras are on by default")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies (read 2^30 B, write 2^30 B each) so that a counter run has a kernel of known traffic to scale by")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this path is built and measured on a single MI355X (--gpus %d refused)" % args.gpus)
        sys.exit(2)
    import torch
    from sphericalrf_amd import api, scene
    assert torch.cuda.is_available(), "bench.py needs a GPU"

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    r = bench_training_step(torch, api, scene, args.steps, args.warmup)
    sec = r["sec_per_step"]
    out = {
        "metric": "marched samples/sec + rays/sec (compositing fwd+bwd), % HBM roofline, 1 GPU",
        "value": r["n_samples"] / sec, "unit": "marched samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 4: training step, 2^20 rays over 200 ring cameras, grid 512x256x256 x 5 cascades, sample cap 2^24, fp16 rgb-sigma in, fp32 gradients out",
                   "rays": r["n_rays"], "rays_kept": r["n_kept"], "samples": r["n_samples"], "compacted_samples": r["n_compacted"], "max_steps_per_ray": r["n_max_steps"],
                   "occupied_bits": r["occupied_bits"],
                   "scene": "48 + 16 Gaussian blobs thresholded at an absolute level, plus a shell at warped radius 0.9-1.0 over two thirds of the outermost cascade's "
                            "angular tiles: about 3 % of all bits of the 5 cascades set, which puts the batch's sample total just under the 2^24 cap (no ray is dropped for lack of room)"},
        "rays_per_s": r["n_rays"] / sec,
        "march": {"ms": r["march_ms"], "samples_per_s": r["n_samples"] / (r["march_ms"] * 1e-3), "rays_per_s": r["n_rays"] / (r["march_ms"] * 1e-3),
                  "steps_per_s": r["n_rays"] * r["n_max_steps"] / (r["march_ms"] * 1e-3), "output_gbs": r["march_gbs"], "frac_hbm": r["march_gbs"] / HBM_PEAK_GBS,
                  "bound": "valu issue (serial disparity chain, warp + cell lookup at probed steps), not hbm"},
        "composite": {"ms": r["composite_ms"], "samples_per_s": r["n_samples"] / (r["composite_ms"] * 1e-3), "rays_per_s": r["n_kept"] / (r["composite_ms"] * 1e-3)},
        "roofline": {"kernel": "compositing forward+backward (volume_rendering_with_loss_and_gradient)", "bound": "hbm",
                     "achieved": r["composite_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": r["composite_gbs"] / HBM_PEAK_GBS, "traffic": composite_traffic_bytes(),
                     "algorithmic_bytes": COMPOSITE_BYTES_PER_SAMPLE * r["n_samples"] + COMPOSITE_BYTES_PER_RAY * r["n_kept"]},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = None      # (keeps its place in the line; measured last, so that the host threads it starts are not around while the GPU is timed)
    bits_host = r["sampler"].density_grid_bitfield.cpu().numpy() if not args.no_cpu_baseline else None
    if not args.no_extras:
        extras = []
        del r["sampler"]
        torch.cuda.empty_cache()
        k = max(2, args.steps // 2)
        for cid in (1, 2, 3, 5):
            extras.append(bench_render(torch, api, scene, cid, k, 1))
            log(json.dumps(extras[-1]))
            torch.cuda.empty_cache()
        for cell_order, steady in ((False, False), (True, False), (False, True), (True, True)):
            extras.append(bench_grid_update(torch, api, scene, k, 1, cell_order=cell_order, steady_state=steady))
            log(json.dumps(extras[-1]))
        extras.append(bench_grid_sample_draws(torch, api, scene, k))
        log(json.dumps(extras[-1]))
        torch.cuda.empty_cache()
        for name, kw in (("training_step_4_drop_in", dict(drop_in=True)),
                         ("training_step_4_dense_grid", dict(shell=(0.05, 1.0, 1.0)))):
            t = bench_training_step(torch, api, scene, k, 1, **kw)
            extras.append(dict(
                workload=name, ms_per_step=t["sec_per_step"] * 1e3, rays=t["n_rays"], rays_kept=t["n_kept"], rays_dropped_or_empty=t["n_rays"] - t["n_kept"],
                samples=t["n_samples"], samples_wanted=t["n_samples_wanted"], sample_cap=1 << 24, compacted_samples=t["n_compacted"], occupied_bits=t["occupied_bits"],
                marched_samples_per_s=t["n_samples"] / t["sec_per_step"], march_ms=t["march_ms"], composite_ms=t["composite_ms"],
                roofline=roofline("compositing forward+backward" + (" with the Coordinate records of the kept samples copied (28 B read + 28 B written each)" if kw.get("drop_in") else ""),
                                  t["composite_bytes"], t["composite_ms"] * 1e-3),
                march_roofline=roofline("training march (output bytes; the kernel is bound by instruction issue)", t["march_bytes"], t["march_ms"] * 1e-3)))
            log(json.dumps(extras[-1]))
            del t
            torch.cuda.empty_cache()
        out["extras"] = extras
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(r, bits_host)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
