#!/usr/bin/env python3
"""Benchmark of the NeuS2 SDF-field hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload step|grid|sdf|lattice|occupancy|mesh] [--no-cpu-baseline]

A step is one full static NeuS2 training step (configuration 4 of BASELINE.json) on a synthetic scene: an analytic sphere of
radius 0.3, Lambertian-textured, seen by 64 cameras at 512x512 on a sphere of radius 2; rays are marched through a
128^3 occupancy bitfield and compacted to 2^18 samples; hash grid + SDF MLP + colour MLP forward, first- and
second-order backward, compositing and Adam, all on the GPU.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

TARGET = 1 << 18
HBM_PEAK_GBS = 8000.0      # MI355X published HBM3E bandwidth
# algorithmic bytes per sample of the kernels a roofline is reported for:
#   grid backward (parameter scatter): 12 (xyz) + 64 (dL_dy, 32 fp16) + 128 x 4 (packed fp16 atomics) = 588
#   grid forward:                      12 (xyz) + 128 x 4 (gathers) + 64 (32 fp16 out)             = 588
#   grid second order:                 12 + 12 (v) + 64 (dL_dy) + 64 (dL_ddLdy) + 128 x 4           = 664
# In a training step the first- and second-order parameter scatters run as ONE merged pass (one write per corner),
# timed under "grid_backward_params": its algorithmic bytes are those of the second-order pass alone, 664 (the
# two passes the reference launches would be 588 + 664).
ALGO_BYTES = {"grid_backward_params": 588, "grid_forward": 588, "grid_second_order": 664}
STEP_ALGO_BYTES = {"grid_backward_params": 664, "grid_forward": 588}
MFMA_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16
# HBM bytes per launch of the step workload's kernels: read from profiles/training_step_2p18_hbm_traffic.json, which
# `bench.py --summarize-traffic` writes from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this file (commands in the JSON
# and in the .txt beside it; counters scaled by what a plain copy of known size reads in the same process)
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "training_step_2p18_hbm_traffic.json")
SCATTER_KERNELS = ("grid_bin_kernel", "grid_reduce_kernel", "grid_combine_kernel")
PROF = {"grid_forward": 0, "grid_backward_params": 1, "grid_second_order": 2, "mlp_forward": 3, "mlp_backward": 4,
        "mlp_second_order": 5, "composite": 6, "sampler": 7, "adam": 8, "field_forward": 9, "field_gather": 10}


def short_kernel_name(name):
    """Base name of a kernel as rocprofv3 prints it (mangled or not); the two weight-gradient instantiations a step
    launches are told apart by their hidden-layer count."""
    import re
    m = re.search(r"([a-z][a-z0-9_]*_kernel)", name)
    base = m.group(1) if m else name.split("(")[0][:48]
    if base == "mlp_wgrad_kernel":
        base += "<colour net>" if "Li3ELi2E" in name or "<3, 2," in name else "<SDF net>"
    return base


def step_traffic():
    """Per-kernel HBM bytes of a step from the committed profile; the scatter's figure is what `roofline.traffic` reports."""
    if not os.path.exists(TRAFFIC_JSON):
        raise SystemExit(f"{TRAFFIC_JSON} is missing: run the two rocprofv3 --pmc commands it records and `bench.py --summarize-traffic`")
    with open(TRAFFIC_JSON) as f:
        t = json.load(f)
    k = t["kernels"]
    missing = [n for n in SCATTER_KERNELS[:2] if n not in k]
    if missing:
        raise SystemExit(f"{TRAFFIC_JSON} holds no entry for {missing}")
    return t, sum(k[n]["fetch_bytes"] + k[n]["write_bytes"] for n in SCATTER_KERNELS if n in k)


def summarize_traffic(fetch_csv, write_csv, copy_mib):
    """rocprofv3 counter CSVs of `bench.py --calibrate-copy MIB` (one run with --pmc FETCH_SIZE, one with WRITE_SIZE) ->
    the JSON this file reads: median launch of the second half of each kernel's launches (steady state), in bytes, scaled so
    that the calibration copy reads its known size."""
    import csv
    import statistics

    def load(path, counter):
        per, copies = {}, []
        for r in csv.DictReader(open(path)):
            if r["Counter_Name"] != counter:
                continue
            v = float(r["Counter_Value"])
            if "copyBuffer" in r["Kernel_Name"]:
                copies.append(v)
            per.setdefault(short_kernel_name(r["Kernel_Name"]), []).append(v)
        if not copies:
            raise SystemExit(f"{path}: no copy kernel found (run bench.py with --calibrate-copy)")
        factor = copy_mib * 1024.0 / max(copies)   # the counters are in KiB
        return {k: statistics.median(v[len(v) // 2:]) * 1024.0 * factor for k, v in per.items()}, factor
    fetch, ff = load(fetch_csv, "FETCH_SIZE")
    write, wf = load(write_csv, "WRITE_SIZE")
    cmd = ("rocprofv3 --pmc {c} --kernel-trace --output-format csv -d gpurun_out/pp/{d} -o f -- python3 bench.py --no-cpu-baseline "
           "--trained-steps 0 --extra-regions 0 --calibrate-copy %d --steps 20 --warmup 5" % copy_mib)
    kernels = {k: {"fetch_bytes": int(fetch.get(k, 0.0)), "write_bytes": int(write.get(k, 0.0))}
               for k in sorted(set(fetch) | set(write)) if "_kernel" in k and not k.startswith("at::")}
    return {"workload": "default benchmark: full training step, 2^18 batch", "command_fetch": cmd.format(c="FETCH_SIZE", d="fetch"),
            "command_write": cmd.format(c="WRITE_SIZE", d="write"),
            "then": "python3 bench.py --calibrate-copy %d --summarize-traffic gpurun_out/pp/fetch/f_counter_collection.csv "
                    "gpurun_out/pp/write/f_counter_collection.csv > profiles/training_step_2p18_hbm_traffic.json" % copy_mib,
            "calibration": {"copy_mib": copy_mib, "fetch_factor": ff, "write_factor": wf,
                            "note": "factor = known bytes of the calibration copy / what the counter read for it"},
            "unit": "bytes per launch (median of the steady-state launches)", "kernels": kernels}


def build_scene(n_cameras=64, resolution=512):
    from neus2_amd import scene
    cams = scene.cameras_on_sphere(n_cameras, resolution)
    rgba = scene.render_sphere_images(cams)
    bits = scene.sphere_bitfield(radius=0.3, band=0.03)
    return cams, rgba, bits


def profile_read(lib, name):
    import ctypes as C
    ms, n = C.c_float(), C.c_uint32()
    lib.n2_profile_read(C.c_int(PROF[name]), C.byref(ms), C.byref(n))
    return float(ms.value), int(n.value)


def cpu_baseline(cams, rgba, bits, sdf_weights, n_rays, n_inference, budget_s=20.0):
    """The oracle's full training step on the host cores at the benchmark's own batch: the same scene, initialisation,
    ray count and 2^18 target as the GPU's timed steps (one step is about 1.5 s on 16 threads, so the bounded sample is a
    few whole steps)."""
    import numpy as np
    from oracle import oracle as orc
    from oracle.field import Field
    from oracle.step import StepState, training_step
    from neus2_amd.training import initial_parameters
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    f = Field(fp16=True)
    offs = [f.off_sdf, f.off_rgb, f.off_grid, f.off_var, f.n_params]
    st = StepState(f, initial_parameters(offs, f.sdf_in_w, seed=1337, sdf_mlp_weights=sdf_weights))
    ocams = []
    for c in cams:
        po = int(c["pixel_offset"])
        ocams.append(orc.Camera((orc.C.c_float * 12)(*c["xform"]), (orc.C.c_float * 2)(*c["focal"]),
                                (orc.C.c_float * 2)(*c["principal"]), (orc.C.c_uint32 * 2)(*c["res"]), po & 0xFFFFFFFF, po >> 32))
    best, done, t_all = None, 0, time.time()
    while done < 2 or (time.time() - t_all < budget_s and done < 8):
        t0 = time.time()
        r = training_step(st, ocams, rgba, bits, n_rays, n_inference, seed=done, target_batch_size=TARGET)
        dt = time.time() - t0
        best = dt if best is None else min(best, dt)
        done += 1
    return {"value": TARGET / best, "unit": "samples/s", "cores": orc.num_threads(), "kind": "port",
            "sample": f"{done} full training steps at the benchmark's 2^18-sample batch ({r['rays']} rays, {r['samples']} marched samples, "
                      f"same scene and initialisation), best step {best * 1e3:.0f} ms"}


def run_step_workload(args):
    import ctypes as C
    import numpy as np
    import torch
    from neus2_amd import capi
    from neus2_amd.tcnn_api import pack_cameras
    from neus2_amd.training import Trainer, default_config
    lib = capi.lib()
    cams, rgba, bits = build_scene()
    sdf_w = np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy"))
    tr = Trainer(default_config(target_batch_size=TARGET, max_rays_per_batch=1 << 16, max_samples=16 * TARGET))
    d_cams, d_rgba, d_bits = pack_cameras(cams), torch.from_numpy(rgba).cuda(), torch.from_numpy(bits).cuda()
    tr.set_scene(d_cams, len(cams), d_rgba, d_bits)
    tr.initialize_params(seed=1337, sdf_mlp_weights=sdf_w)
    # untimed: let the ray-count feedback settle so that the compacted batch fills the 2^18 target
    tr.budget.rays_per_batch = 4096
    for _ in range(6):
        tr.step()
        counters, ok = tr.update_budget()
        if not ok:
            raise SystemExit(f"no samples generated: {counters}")
    n_rays, n_inf = tr.budget.rays_per_batch, tr.budget.n_inference()
    for _ in range(args.warmup):
        tr.step(n_rays=n_rays, n_inference=n_inf)
    torch.cuda.synchronize()
    # one region of the same length is run and discarded first: the first region after the warm-up steps is consistently about
    # one per cent slower than those that follow it (clocks and caches settle), and `value` is to be a steady-state figure
    for _ in range(args.steps):
        tr.step(n_rays=n_rays, n_inference=n_inf)
    torch.cuda.synchronize()
    # timed region: K steps; only the roofline kernel (the parameter scatter) carries events, and only in five of the
    # steps, because every event pair costs stream time (about 13 us) that is charged to the step
    dom = "grid_backward_params"
    period = max(1, args.steps // 5)  # five timed launches per region
    lib.n2_profile_reset()
    lib.n2_profile_select(C.c_uint32(1 << PROF[dom]))
    lib.n2_profile_set_period(C.c_uint32(period))
    lib.n2_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        tr.step(n_rays=n_rays, n_inference=n_inf)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.n2_profile_enable(0)
    counters = tr.read_counters()
    dom_ms, dom_n = profile_read(lib, dom)
    # untimed: the same K steps again with every listed kernel bracketed by events (the per-kernel breakdown)
    lib.n2_profile_reset()
    lib.n2_profile_select(C.c_uint32(0xFFFFFFFF))
    lib.n2_profile_set_period(C.c_uint32(1))
    lib.n2_profile_enable(1)
    for _ in range(args.steps):
        tr.step(n_rays=n_rays, n_inference=n_inf)
    torch.cuda.synchronize()
    lib.n2_profile_enable(0)
    kernels = {}
    for name in PROF:
        ms, n = profile_read(lib, name)
        if n:
            kernels[name] = {"ms_per_step": ms / args.steps, "launches_per_step": n / args.steps, "avg_us": ms / n * 1e3}
    # (one launch per step; dom_n of them were timed)
    kernels[dom] = {"ms_per_step": dom_ms / dom_n, "launches_per_step": 1.0, "avg_us": dom_ms / dom_n * 1e3, "timed_launches": dom_n}
    # per-launch batch of the dominant kernel: the backward kernels always see the 2^18 compacted batch; the forward
    # also runs over the marched samples, so use the average batch per launch
    per_launch = TARGET if dom != "grid_forward" else (TARGET + n_inf) / 2
    achieved = STEP_ALGO_BYTES[dom] * per_launch / (kernels[dom]["avg_us"] * 1e-6) / 1e9
    traffic_profile, scatter_traffic = step_traffic()
    # the other two large memory-bound launches of a step, from the untimed per-kernel pass: the gather over the marched
    # samples (588 B per sample) and Adam (32 B per parameter with the trainer's 16-bit step counters, dense bound)
    n_params = tr.n_params

    def hbm_entry(key, kernel, bytes_per_unit, units, what):
        if key not in kernels:
            return None
        gbs = bytes_per_unit * units / (kernels[key]["avg_us"] * 1e-6) / 1e9
        k = traffic_profile["kernels"].get(kernel)
        return {"kernel": kernel, "bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                "algorithmic_bytes": what, "units_per_launch": units, "avg_launch_us": kernels[key]["avg_us"],
                "traffic": (k["fetch_bytes"] + k["write_bytes"]) if k else None}
    rooflines = {"field_gather": hbm_entry("field_gather", "field_gather_kernel", 588, counters["samples"], "588 B per marched sample (12 xyz + 128 x 4 gathers + 64 features)"),
                 "adam": hbm_entry("adam", "adam_step_kernel", 32, n_params, "32 B per parameter (dense bound, 16-bit step counters)")}
    if args.calibrate_copy:
        # a plain copy of known size in the same process: the scale of the FETCH_SIZE / WRITE_SIZE counters
        src = torch.empty(args.calibrate_copy << 20, dtype=torch.uint8, device="cuda").zero_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
    # MFMA side of the metric: the two weight-gradient launches of a step (colour net: recomputed forward 14336 + data
    # gradients 16384 + weight gradients 16384 flop per batch sample; SDF net: 24576 + its second-order pass 14336), algorithmic
    # flops over their summed durations from the untimed per-kernel pass.  The networks' forward passes run inside the fused
    # field forward, which is timed together with the gather ("field_forward") and is bound by memory.
    mlp_flops = TARGET * (24576 + 14336 + 47104)
    mlp_ms = kernels["mlp_backward"]["ms_per_step"] if "mlp_backward" in kernels else 0.0
    mfma = {"kernels": "mlp_wgrad (colour net) + mlp_wgrad (SDF net with second order): the weight-gradient launches of a step",
            "algorithmic_flops_per_step": mlp_flops,
            "ms_per_step": mlp_ms, "achieved_tflops": mlp_flops / (mlp_ms * 1e-3) / 1e12 if mlp_ms else None, "peak_tflops": MFMA_PEAK_TFLOPS,
            "frac": mlp_flops / (mlp_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS if mlp_ms else None}
    result = {
        "metric": "SDF train samples/sec @2^18 batch (1 GPU)",
        "value": args.steps * TARGET / elapsed,
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "full NeuS2 static training step (BASELINE configs[3]): analytic sphere r=0.3, 64 cameras 512x512 "
                               "on a radius-2 sphere, 128^3 occupancy bitfield, rays compacted to 2^18 samples; hash grid "
                               "L=16 F=2 T=2^19 + SDF MLP 48-64-16 + colour MLP 48-64-64-16, first and second order backward, "
                               "compositing, Adam",
                   "target_batch": TARGET, "rays_per_step": n_rays, "marched_samples_per_step": counters["samples"],
                   "inference_batch": n_inf, "compacted_before_rollover": counters["compacted"], "loss": counters["loss"]},
        "roofline": {"kernel": dom, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": scatter_traffic,
                     "traffic_unit": "bytes per launch of bin + reduce + combine (rocprofv3 FETCH_SIZE + WRITE_SIZE, copy-calibrated; "
                                     "read from profiles/training_step_2p18_hbm_traffic.json)",
                     "algorithmic_bytes_per_sample": STEP_ALGO_BYTES[dom], "samples_per_launch": per_launch,
                     "avg_launch_us": kernels[dom]["avg_us"], "timed_launches": dom_n},
        "mfma": mfma,
        "rooflines": rooflines,
        "kernels": kernels,
        "kernels_note": "grid_backward_params is timed with HIP events inside the timed region (five launches spread over the region); the other entries come from a "
                        "second, untimed pass of the same steps with every listed kernel bracketed by events",
    }
    # untimed extras (the driver's fields above come from the one timed region before them)
    # (i) spread: further regions of K steps each, every one bracketed like the timed region
    regions = [elapsed / args.steps * 1e3]
    for _ in range(args.extra_regions):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            tr.step(n_rays=n_rays, n_inference=n_inf)
        torch.cuda.synchronize()
        regions.append((time.perf_counter() - t0) / args.steps * 1e3)
    srt = sorted(regions)
    result["regions"] = {"ms_per_step": regions, "median": srt[len(srt) // 2], "min": srt[0], "max": srt[-1],
                         "note": f"{len(regions)} consecutive regions of {args.steps} steps; the first one is the timed region of `value`"}
    # (ii) the same loop on a trained field: rays stop at the surface, so a step marches more samples than it keeps
    result["settle_steps"] = args.steps  # the discarded region in front of the timed one (after the `warmup` steps)
    if args.trained_steps > 0:
        del tr
        result["trained_state"] = trained_state_leg(args, lib, d_cams, len(cams), d_rgba, sdf_w)
        # both regimes side by side: `value` is the initial state (every marched sample is kept), the trained field marches
        # about three samples for every one it keeps
        result["config"]["trained_state_ms_per_step"] = result["trained_state"].get("ms_per_step")
        result["config"]["trained_state_samples_per_s"] = result["trained_state"].get("value")
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cams, rgba, bits, sdf_w, n_rays, n_inf)
    return result


def trained_state_leg(args, lib, d_cams, n_cams, d_rgba, sdf_w):
    """The same timed loop on a trained field.  A second trainer runs the loop the way the reference drives it
    (src/testbed.cu:2641-2674): occupancy-grid updates on their cadence from step 0 (the rays march through the trainer's own
    density grid instead of the analytic shell), learning rate 1e-2 (configs/nerf/dtu.json:15), the ray budget's feedback every
    16 steps.  After args.trained_steps steps K steps are timed exactly like the main region (no occupancy update inside)."""
    import ctypes as C
    import numpy as np
    import torch
    from neus2_amd.training import GRID_CELLS, OccupancyGrid, Trainer, default_config
    tr = Trainer(default_config(target_batch_size=TARGET, max_rays_per_batch=1 << 16, max_samples=16 * TARGET, learning_rate=1e-2))
    occ = OccupancyGrid(1, seed=1337, max_chunk=1 << 21)
    tr.set_scene(d_cams, n_cams, d_rgba, occ.bitfield)
    tr.attach_occupancy(occ)
    tr.initialize_params(seed=1337, sdf_mlp_weights=sdf_w)
    for it in range(args.trained_steps):
        tr.training_prep()
        tr.step()
        if it % 16 == 15 or it < 16:
            counters, ok = tr.update_budget()
            if not ok:
                return {"error": f"no samples at step {it}: {counters}"}
    n_rays, n_inf = tr.budget.rays_per_batch, tr.budget.n_inference()
    for _ in range(args.warmup):
        tr.step(n_rays=n_rays, n_inference=n_inf)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        tr.step(n_rays=n_rays, n_inference=n_inf)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    c = tr.read_counters()
    occupied = float(np.unpackbits(occ.bitfield[:GRID_CELLS // 8].cpu().numpy()).mean())
    return {"ms_per_step": elapsed / args.steps * 1e3, "value": args.steps * min(c["compacted"], TARGET) / elapsed, "unit": "samples/s",
            "trained_steps": args.trained_steps, "rays_per_step": n_rays, "marched_samples_per_step": c["samples"], "inference_batch": n_inf,
            "compacted_before_rollover": c["compacted"], "occupied_cells": occupied, "loss": c["loss"],
            "note": "same timed loop after training with the occupancy grid updated on its cadence; `value` counts the samples the "
                    "rays kept (the batch is padded to 2^18 by rollover)"}


def timed_best(fn, budget_s=15.0, min_runs=2, max_runs=8):
    """Best wall time of fn() over a bounded number of runs (host-side baselines)."""
    best, done, t_all = None, 0, time.time()
    while done < min_runs or (time.time() - t_all < budget_s and done < max_runs):
        t0 = time.time()
        fn()
        dt = time.time() - t0
        best = dt if best is None else min(best, dt)
        done += 1
    return best, done


def run_grid_workload(args):
    """Configuration 2 of BASELINE.json: hash-grid encoding only, forward + backward on 2^18 uniform points."""
    import torch
    from neus2_amd import capi
    from neus2_amd.tcnn_api import GRAD_OVERWRITE, GridEncoding
    lib = capi.lib()
    g = GridEncoding()
    gen = torch.Generator(device="cuda").manual_seed(0)
    params = ((torch.rand(g.n_params(), device="cuda", generator=gen) * 2 - 1) * 1e-4).half()
    grads = torch.zeros_like(params)
    g.set_params(params, grads)
    g.reserve_scatter_workspace(TARGET)
    x = torch.rand((3, TARGET), device="cuda", generator=gen)
    dy = torch.randn((32, TARGET), device="cuda", generator=gen).half()

    def step():
        _, ctx = g.forward(x, prepare_input_gradients=True)
        g.backward(ctx, x, dy, want_input_grad=True, mode=GRAD_OVERWRITE)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    lib.n2_profile_reset()
    lib.n2_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.n2_profile_enable(0)
    kernels = {}
    for name in ("grid_forward", "grid_backward_params"):
        ms, n = profile_read(lib, name)
        kernels[name] = {"ms_per_step": ms / args.steps, "avg_us": ms / n * 1e3}
    dom = max(kernels, key=lambda k: kernels[k]["ms_per_step"])
    achieved = ALGO_BYTES[dom] * TARGET / (kernels[dom]["avg_us"] * 1e-6) / 1e9
    result = {"metric": "hash-grid fwd+bwd samples/sec @2^18 batch (1 GPU)", "value": args.steps * TARGET / elapsed, "unit": "samples/s",
              "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
              "config": {"workload": "hash-grid encoding only, forward + backward (BASELINE configs[1])", "batch": TARGET},
              "roofline": {"kernel": dom, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": achieved / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_sample": ALGO_BYTES[dom],
                           "samples_per_launch": TARGET, "avg_launch_us": kernels[dom]["avg_us"]},
              "kernels": kernels}
    if not args.no_cpu_baseline:
        from oracle import oracle as orc
        og = orc.Grid()
        P, xs, dys = params.float().cpu().numpy(), x.cpu().numpy(), dy.float().cpu().numpy()

        def cpu_step():
            og.forward(P, xs, want_dy_dx=True)
            og.backward(P, xs, dys)

        best, done = timed_best(cpu_step)
        result["cpu_baseline"] = {"value": TARGET / best, "unit": "samples/s", "cores": orc.num_threads(), "kind": "port",
                                  "sample": f"the same 2^18 points and gradients: forward with dy_dx + backward (parameters and input), "
                                            f"best of {done} runs, {best * 1e3:.0f} ms"}
    return result


def run_sdf_workload(args):
    """Configuration 3 of BASELINE.json: grid + SDF MLP with the eikonal second-order path on 2^18 uniform points: forward,
    normals, backward of mean|sdf| + 0.1 mean(|grad sdf| - 1)^2 through the encoding and the MLP weights."""
    import numpy as np
    import torch
    from neus2_amd import capi
    from neus2_amd.sdf_net import SdfNet
    lib = capi.lib()
    net = SdfNet(max_batch=TARGET)
    gen = torch.Generator(device="cuda").manual_seed(1)
    P = ((torch.rand(net.grid.n_params(), device="cuda", generator=gen) * 2 - 1) * 1e-4).half()
    W = torch.from_numpy(np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy"))).cuda().half()
    gP, gW = torch.zeros_like(P), torch.zeros_like(W)
    net.set_params(P, gP, W, gW)
    x = torch.rand((3, TARGET), device="cuda", generator=gen)
    loss = None

    def step():
        nonlocal loss
        loss = net.loss_backward(net.forward(x))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    lib.n2_profile_reset()
    lib.n2_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.n2_profile_enable(0)
    kernels, total = {}, 0.0
    for name in PROF:
        ms, n = profile_read(lib, name)
        if n:
            kernels[name] = {"ms_per_step": ms / args.steps, "launches_per_step": n / args.steps, "avg_us": ms / n * 1e3}
            total += ms / args.steps
    sc = kernels["grid_backward_params"]["avg_us"] * 1e-6
    achieved = ALGO_BYTES["grid_second_order"] * TARGET / sc / 1e9
    result = {"metric": "SDF net + eikonal fwd/bwd samples/sec @2^18 batch (1 GPU)", "value": args.steps * TARGET / elapsed, "unit": "samples/s",
              "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
              "config": {"workload": "hash grid + SDF MLP 48-64-16, forward, normals, first and second order backward of "
                                     "mean|sdf| + 0.1 mean(|grad sdf| - 1)^2 (BASELINE configs[2]); 2^18 uniform points",
                         "batch": TARGET, "loss": float(loss), "kernel_ms_per_step": total},
              "roofline": {"kernel": "grid_backward_params (merged first+second order scatter)", "bound": "hbm", "achieved": achieved,
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                           "algorithmic_bytes_per_sample": ALGO_BYTES["grid_second_order"], "samples_per_launch": TARGET,
                           "avg_launch_us": kernels["grid_backward_params"]["avg_us"]},
              "kernels": kernels}
    if not args.no_cpu_baseline:
        from oracle import oracle as orc
        from oracle.sdf_step import sdf_eikonal_step
        Pn, Wn, xn = P.float().cpu().numpy(), W.float().cpu().numpy(), x.cpu().numpy()
        best, done = timed_best(lambda: sdf_eikonal_step(Pn, Wn, xn, 0.1, 128.0))
        result["cpu_baseline"] = {"value": TARGET / best, "unit": "samples/s", "cores": orc.num_threads(), "kind": "port",
                                  "sample": f"the same 2^18 points, one forward + normals + first and second order backward, best of {done} "
                                            f"runs, {best * 1e3:.0f} ms"}
    return result


def run_lattice_workload(args):
    """Configuration 5 of BASELINE.json: SDF inference for mesh extraction (hash grid + SDF MLP forward, fp16) over the 512^3
    lattice p = (i, j, k) / 512, in chunks of 2^22 points; a step is one chunk, chunks are visited in order."""
    import numpy as np
    import torch
    from neus2_amd import capi
    from neus2_amd.tcnn_api import NerfNetwork
    from neus2_amd.training import initial_parameters
    lib = capi.lib()
    CH, RES = 1 << 22, 512
    net = NerfNetwork()
    offs = net.param_offsets()
    p = initial_parameters(offs, 48, seed=1, sdf_mlp_weights=np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy")))
    params = torch.from_numpy(p).cuda().half()
    net.set_params(params, None)
    net.reserve(CH)
    n_chunks = RES ** 3 // CH
    use = min(n_chunks, max(args.steps, 1) + args.warmup)
    # lattice coordinates of the chunks that will be visited, x fastest (generated once, resident in HBM)
    idx = torch.arange(use * CH, device="cuda", dtype=torch.int64)
    xyz = torch.stack(((idx % RES).float() / RES, ((idx // RES) % RES).float() / RES, (idx // (RES * RES)).float() / RES))
    xyz = xyz.view(3, use, CH).permute(1, 0, 2).contiguous()  # [chunk][3][CH]
    del idx

    net.encoding().set_point_order(True)  # x-fastest lattice points, as Testbed::get_density_on_grid produces them

    def chunk(k):
        k %= use
        return net.sdf(xyz[k])

    for k in range(args.warmup):
        out = chunk(k)
    torch.cuda.synchronize()
    lib.n2_profile_reset()
    lib.n2_profile_enable(1)
    t0 = time.perf_counter()
    for k in range(args.steps):
        out = chunk(args.warmup + k)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.n2_profile_enable(0)
    kernels, dom, dom_us, algo = inference_kernels(lib, args.steps)
    achieved = algo * CH / (dom_us * 1e-6) / 1e9
    mlp_us = dom_us if dom == "field_forward" else kernels["mlp_forward"]["avg_us"]
    mlp_tflops = 8192 * CH / (mlp_us * 1e-6) / 1e12
    result = {"metric": "SDF inference points/sec over a 512^3 lattice in 2^22-point chunks (1 GPU)", "value": args.steps * CH / elapsed,
              "unit": "points/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
              "config": {"workload": "hash grid + SDF MLP forward over the 512^3 lattice (BASELINE configs[4]), geometric-init SDF MLP, "
                                     "grid U(-1e-4, 1e-4) seed 1", "chunk": CH, "chunks_in_lattice": n_chunks,
                         "sdf_mean_abs": float(out[0].float().abs().mean())},
              "roofline": {"kernel": dom, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": achieved / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_sample": algo,
                           "samples_per_launch": CH, "avg_launch_us": dom_us},
              "mfma": {"kernel": "SDF net 48-64-16 forward" + (" (inside the fused launch)" if dom == "field_forward" else ""), "flops_per_sample": 8192,
                       "achieved_tflops": mlp_tflops, "peak_tflops": MFMA_PEAK_TFLOPS, "frac": mlp_tflops / MFMA_PEAK_TFLOPS},
              "kernels": kernels}
    # the consumer's form of the same job (Testbed::get_density_on_grid): lattice points formed inside the kernel, only the SDF
    # row kept, as fp32; the whole 512^3 lattice
    from neus2_amd.mesh import density_on_grid
    from neus2_amd.training import Trainer, default_config
    tr = Trainer(default_config(target_batch_size=TARGET, max_rays_per_batch=1 << 12, max_samples=CH))
    tr.initialize_params(seed=1, sdf_mlp_weights=np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy")))
    d = density_on_grid(tr._field, (RES, RES, RES), chunk=CH)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        d = density_on_grid(tr._field, (RES, RES, RES), chunk=CH)
    torch.cuda.synchronize()
    dog = (time.perf_counter() - t0) / 3
    result["density_on_grid"] = {"ms_per_lattice": dog * 1e3, "ms_per_chunk": dog * 1e3 / n_chunks, "points_per_s": RES ** 3 / dog,
                                 "note": "n2_density_on_grid over all 32 chunks: no position array, fp32 SDF row only"}
    del d, tr
    if not args.no_cpu_baseline:
        from oracle import oracle as orc
        from oracle.field import Field
        f = Field(fp16=True)
        sub = 128
        gi = np.arange(sub ** 3, dtype=np.int64)
        sx = np.stack(((gi % sub) / sub, ((gi // sub) % sub) / sub, (gi // (sub * sub)) / sub)).astype(np.float32)
        p16 = params.float().cpu().numpy()
        best, done = timed_best(lambda: f.sdf_values(p16, sx))
        result["cpu_baseline"] = {"value": sub ** 3 / best, "unit": "points/s", "cores": orc.num_threads(), "kind": "port",
                                  "sample": f"the 128^3 lattice p = (i, j, k) / 128 of the same network (1/64 of the points), best of {done} "
                                            f"runs, {best * 1e3:.0f} ms"}
    return result


def inference_kernels(lib, steps):
    """Event timings of an inference workload's launches: the fused launch (grid gather + SDF net in one kernel,
    algorithmic bytes 12 xyz + 128 x 4 gathers + 32 output = 556 per point) or the grid forward (588) followed by the MLP."""
    kernels = {}
    for name in ("field_forward", "grid_forward", "mlp_forward"):
        ms, n = profile_read(lib, name)
        if n:
            kernels[name] = {"ms_per_step": ms / steps, "launches_per_step": n / steps, "avg_us": ms / n * 1e3}
    dom = "field_forward" if "field_forward" in kernels else "grid_forward"
    return kernels, dom, kernels[dom]["avg_us"], 556 if dom == "field_forward" else 588


def run_occupancy_workload(args):
    """The occupancy-grid update that precedes training steps (the reference runs it every step for the first 32 steps,
    then every 2nd ... 16th): a step is one update_density_grid_nerf over all 128^3 cells (uniform samples), i.e. sample
    generation, NerfNetwork::density on 2^21 points, max-splat, decayed maximum, mean, bitfield and its mip levels."""
    import numpy as np
    import torch
    from neus2_amd import capi
    from neus2_amd.training import GRID_CELLS, OccupancyGrid, Trainer, default_config
    lib = capi.lib()
    tr = Trainer(default_config(target_batch_size=TARGET, max_rays_per_batch=1 << 16, max_samples=1 << 21))
    sdf_w = np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy"))
    tr.initialize_params(seed=1337, sdf_mlp_weights=sdf_w)
    occ = OccupancyGrid(1, seed=1337, max_chunk=1 << 21)
    for _ in range(args.warmup):
        occ.update(tr._field, GRID_CELLS, 0)
    torch.cuda.synchronize()
    lib.n2_profile_reset()
    lib.n2_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        occ.update(tr._field, GRID_CELLS, 0)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.n2_profile_enable(0)
    kernels, dom, dom_us, algo = inference_kernels(lib, args.steps)
    achieved = algo * GRID_CELLS / (dom_us * 1e-6) / 1e9
    result = {"metric": "occupancy-grid cells updated per second (128^3 cells per update, 1 GPU)", "value": args.steps * GRID_CELLS / elapsed,
              "unit": "cells/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
              "config": {"workload": "update_density_grid_nerf over all 128^3 cells of one cascade: PCG32 sample generation, field density "
                                     "(hash grid + SDF MLP forward) on 2^21 points, max-splat, decayed maximum, mean, bitfield + 7 mips",
                         "cells": GRID_CELLS, "occupied_fraction": float(np.unpackbits(occ.bitfield[:GRID_CELLS // 8].cpu().numpy()).mean())},
              "roofline": {"kernel": dom, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": achieved / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_sample": algo,
                           "samples_per_launch": GRID_CELLS, "avg_launch_us": dom_us},
              "kernels": kernels}
    if not args.no_cpu_baseline:
        from oracle import oracle as orc
        from oracle.field import Field
        f = Field(fp16=True)
        p16 = tr.params.float().cpu().numpy()
        ref = orc.OccupancyGrid(1, seed=1337)
        n = 1 << 17
        best = None
        for _ in range(3):
            t0 = time.time()
            ref.update(lambda xyz: f.density(p16, xyz)[0], 0.95, n, 0)
            dt = time.time() - t0
            best = dt if best is None else min(best, dt)
        result["cpu_baseline"] = {"value": n / best, "unit": "cells/s", "cores": orc.num_threads(), "kind": "port",
                                  "sample": f"one update with 2^17 uniform samples (1/16 of the cells; the mean/bitfield part still covers all "
                                            f"128^3 cells), best of 3, {best * 1e3:.0f} ms"}
    return result


def run_mesh_workload(args):
    """The consumer of configuration 5 of BASELINE.json: marching cubes over the 512^3 SDF lattice (count per tile, prefix sums over
    the tiles, vertices, faces, normals).  The lattice is evaluated once, untimed (that part is `--workload lattice`); a step is one full extraction."""
    import numpy as np
    import torch
    from neus2_amd.mesh import density_on_grid, marching_cubes
    from neus2_amd.training import Trainer, default_config
    RES = 512
    tr = Trainer(default_config(target_batch_size=TARGET, max_rays_per_batch=1 << 12, max_samples=1 << 22))
    tr.initialize_params(seed=1, sdf_mlp_weights=np.load(os.path.join(ROOT, "tests", "golden", "sdf_mlp_weights_48.npy")))
    d = density_on_grid(tr._field, (RES, RES, RES), chunk=1 << 22)
    for _ in range(args.warmup):
        v, t, n = marching_cubes(d, 0.0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        v, t, n = marching_cubes(d, 0.0)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    n_pts = RES ** 3
    # algorithmic bytes per lattice point: the density is read once (4); the emitting passes touch only the tiles the surface
    # crosses, and vertices / indices / normals are small next to the lattice
    algo = 4
    achieved = algo * n_pts / (elapsed / args.steps) / 1e9
    return {"metric": "marching-cubes lattice points/sec over a 512^3 SDF lattice (1 GPU)", "value": args.steps * n_pts / elapsed, "unit": "points/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "marching cubes (shared vertices, deterministic numbering, vertex normals) over the 512^3 lattice of the "
                                   "geometric-init SDF network, threshold 0; wall clock of the whole extraction including its one host "
                                   "synchronisation and output allocation", "lattice": [RES, RES, RES], "vertices": int(v.shape[0]),
                       "triangles": int(t.shape[0])},
            "roofline": {"kernel": "marching cubes, all kernels of one extraction", "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None, "algorithmic_bytes_per_sample": algo,
                         "samples_per_launch": n_pts, "avg_launch_us": elapsed / args.steps * 1e6}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)   # 85 ms of timed region for the default workload
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["step", "grid", "sdf", "lattice", "occupancy", "mesh"], default="step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--extra-regions", type=int, default=5, help="step workload: untimed repeat regions of K steps (spread of the figure)")
    ap.add_argument("--trained-steps", type=int, default=3000,
                    help="step workload: training steps before the trained-state leg (0 switches the leg off)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="after the timed region, copy MIB mebibytes device-to-device once (counter calibration under a profiler)")
    ap.add_argument("--summarize-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: turn the counter CSVs of two rocprofv3 --pmc runs of this file (FETCH_SIZE, WRITE_SIZE, both with "
                         "--calibrate-copy MIB) into the JSON that `roofline.traffic` is read from, on stdout")
    args = ap.parse_args()
    if args.summarize_traffic:
        if args.calibrate_copy <= 0:
            raise SystemExit("--summarize-traffic needs --calibrate-copy MIB (the size of the calibration copy of the profiled runs)")
        print(json.dumps(summarize_traffic(args.summarize_traffic[0], args.summarize_traffic[1], args.calibrate_copy), indent=1))
        return
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs the hot path on ONE GPU (the reference has no multi-GPU path and the "
                         "benchmark metric is quoted on 1 GPU); run with --gpus 1")
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (there is no CPU fallback of the product path)")
    result = {"step": run_step_workload, "grid": run_grid_workload, "sdf": run_sdf_workload, "lattice": run_lattice_workload,
              "occupancy": run_occupancy_workload, "mesh": run_mesh_workload}[args.workload](args)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
