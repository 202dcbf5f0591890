#!/usr/bin/env python3
"""Headline benchmark: frames per second of the inference rasterizer on one MI355X.

One "step" is one full ``rasterize()`` call (preprocess -> scan -> host read of the instance count ->
duplication -> radix sort -> ranges -> blend) on a seeded synthetic scene whose tensors are already resident
in HBM.  Headline workload: 3 M Gaussians, 1920x1080, HYBRID_BLEND K=16 (the configuration the metric is quoted
on).  Prints ONE JSON line.

Run without ``--config`` / ``--mode`` / ``--train`` / ``--fast`` the line also carries a ``configs`` block: after the
headline's timed region every other benchmark configuration is timed the same way (fewer steps) -- the tiny scene,
1 M / 720p, the 3 M scene under the other three blend modes and through ``fast_rasterize``, the 6 M stress scene with
duplication and sort isolated, and the training step (forward + backward) under each mode -- each with its per-stage
times and the roofline of its dominant kernel.  With one of those flags only that workload is timed.

The per-stage breakdown and the roofline figures are measured in the same process with HIP events on the
stream the kernels are launched on (torch's current stream, which is the stream handed to the C ABI).
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MODE_NAMES = {0: "HYBRID_BLEND", 1: "ALPHA_BLEND_FIRST_K", 2: "ALPHA_BLEND_GLOBAL_ORDERING", 3: "OIT_BLEND"}
HBM_PEAK_GBS = 8000.0
# fp32 vector peak as published: 1024 SIMDs x 32 lanes x 2 flops x 2.4 GHz, i.e. one wave64 v_fma_f32 per two cycles
# and SIMD (measured: 2.2-2.5 cycles)
FP32_PEAK_TFLOPS = 157.3
# flops of the mandatory part of one pixel/instance evaluation as the reference states it (the two planes, m, d,
# |m|^2, |d|^2, cut-off test: R/include/hybrid_blend/kernels/inference.cuh:137-147).  The kernels reach the same
# decision with two quadratics (21 flops), so this prices the problem, not the instructions issued.
FLOPS_PER_EVAL = 46
# CPU baseline: one warm-up run, then this many timed runs; the median is reported
CPU_REPS = 3
COUNTERS_FILE = os.path.join(ROOT, "profiles", "counters.json")
# steps / warm-up steps of the workloads of the ``configs`` block
EXTRA_STEPS, EXTRA_WARMUP = 20, 5


def measured_traffic(key: str):
    """HBM bytes of the dominant kernel's launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, as recorded in
    profiles/counters.json by ``python -m htgs_amd.diagnostics.counters`` -- or None when that file was recorded on
    other kernel sources than the ones in this tree (the figure would describe other code)."""
    try:
        with open(COUNTERS_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    from htgs_amd.build import csrc_digest
    if rec.get("csrc_sha256") != csrc_digest():
        return None
    entry = rec.get("launches", {}).get(key)
    return None if entry is None else entry.get("traffic_bytes")


def workload_key(config, n, mode, K, what) -> str:
    return f"cfg{config}" + (f"-n{n}" if n else "") + f"/mode{mode}/K{K}/{what}"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=None, help="scene: 0 = tiny, 1 = 1M/720p, 2 = 3M/1080p, 3 = 6M stress, 4 = 1M/1080p (training)")
    ap.add_argument("--n", type=int, default=None, help="override the number of Gaussians")
    ap.add_argument("--mode", type=int, default=None)
    ap.add_argument("--K", type=int, default=None)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true", help="time the headline workload alone (no configs block)")
    ap.add_argument("--calibrate", action="store_true",
                    help="only run a plain 1 GiB copy kernel a few times (reference point for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--train", action="store_true", help="time diff_rasterize forward + backward instead of rasterize")
    ap.add_argument("--densification-rows", type=int, default=0, choices=(0, 2, 3),
                    help="with --train: pass a densification_info tensor of this many rows to the backward pass")
    ap.add_argument("--fast", action="store_true", help="time fast_rasterize (image only, reduced accuracy) instead of rasterize")
    return ap.parse_args()


def event_ms(fn, reps):
    import torch
    out = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        out.append(a.elapsed_time(b))
    return out


def timed_steps(step, steps, warmup):
    """Milliseconds per step: ``warmup`` untimed steps, then exactly ``steps`` steps between two device synchronisations."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def oracle_frame(oracle, scene_cpu, mode, K):
    return oracle.Frame(scene_cpu.M.numpy(), scene_cpu.VPM.numpy(), scene_cpu.cam_position.numpy(), mode, K,
                        scene_cpu.active_sh_bases, scene_cpu.width, scene_cpu.height, scene_cpu.near_plane, scene_cpu.far_plane)


def bench_training(scene_cpu, scene, config, n_override, mode, K, steps, warmup, densification_rows=0, cpu_baseline=True, long_list_threshold=0):
    """One step = diff_rasterize forward + backward w.r.t. all six Gaussian tensors from a fixed upstream
    gradient ~N(0,1).  Reported as milliseconds per step with the forward / backward split."""
    import torch
    from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode
    settings = scene.settings(RasterizerMode(mode), K)
    gauss = scene.gaussians()
    grad_image = torch.randn(3, scene.height, scene.width, generator=torch.Generator().manual_seed(4)).to(gauss[0].device)

    info = torch.zeros((densification_rows, scene.positions.shape[0]), device=gauss[0].device) if densification_rows else None

    def step():
        fb = FrameBuffers(*gauss, settings, True, False, train=True, long_list_threshold=long_list_threshold)
        fb.run_forward()
        return fb, fb.run_backward(grad_image, info, info is not None)

    ms_per_step = timed_steps(step, steps, warmup)
    fb = FrameBuffers(*gauss, settings, True, False, train=True, long_list_threshold=long_list_threshold)
    fb.run_forward()
    fwd_blend = statistics.median(event_ms(fb.blend_forward, 10))
    bwd = statistics.median(event_ms(lambda: fb.run_backward(grad_image, info, info is not None), 10))
    fb.run_backward(grad_image, info, info is not None)
    bwd_blend_samples = event_ms(fb.blend_backward, 10)
    bwd_blend = statistics.median(bwd_blend_samples)
    bwd_prim = statistics.median(event_ms(fb.preprocess_backward, 10))
    # roofline of the dominant kernel (the backward blend): it evaluates every (pixel, instance) pair again, priced as
    # in the inference line; its algorithmic bytes are the gathered records, the per-pixel records of the forward pass,
    # the upstream gradient and one 64-byte gradient row per instance
    n_inst, P, Keff = fb.n_instances, fb.width * fb.height, fb.lib.htgs_effective_k(K)
    tile_px = fb.tile * fb.tile
    avg_ms = sum(bwd_blend_samples) / len(bwd_blend_samples)
    records = {0: (20 * Keff + 24) * P, 1: 20 * Keff * P, 2: 12 * P, 3: 24 * P}[mode]
    algo_bytes = 84 * n_inst + records + 12 * P + 64 * n_inst + (4 * n_inst if densification_rows == 3 else 0)
    tflops = FLOPS_PER_EVAL * tile_px * n_inst / (avg_ms / 1e3) / 1e12
    roofline = {"kernel": "blend_backward", "bound": "valu_fp32", "achieved": round(tflops, 3), "peak": FP32_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(tflops / FP32_PEAK_TFLOPS, 4),
                "traffic": measured_traffic(workload_key(config, n_override, mode, K, f"train{densification_rows}")),
                "launch_ms": round(avg_ms, 4), "evals_per_launch": tile_px * n_inst, "algo_GB": round(algo_bytes / 1e9, 4),
                "algo_GBps": round(algo_bytes / 1e9 / (avg_ms / 1e3), 1)}
    baseline = None
    if cpu_baseline:
        import oracle
        fr = oracle_frame(oracle, scene_cpu, mode, K)
        arrays = [t.numpy() for t in scene_cpu.gaussians()]
        gi = grad_image.cpu().numpy()
        runs = []
        for _ in range(1 + CPU_REPS):                       # the first run is the warm-up
            t0 = time.perf_counter()
            fwd = oracle.forward(fr, *arrays)
            t1 = time.perf_counter()
            oracle.backward(fwd, gi, *arrays)
            runs.append((time.perf_counter() - t0, t1 - t0))
        runs = sorted(runs[1:])
        total_s, fwd_s = runs[len(runs) // 2]
        baseline = {"value": round(total_s * 1e3, 1), "unit": "ms/step", "cores": oracle.num_threads(), "kind": "port",
                    "stages_ms": {"forward": round(fwd_s * 1e3, 1), "backward": round((total_s - fwd_s) * 1e3, 1)},
                    "sample": f"whole forward + backward of the same workload, C oracle with OpenMP; median of {CPU_REPS} runs after one warm-up"}
    return {
        "metric": f"training step (diff_rasterize forward + backward) {MODE_NAMES[mode]} K={K}", "value": round(ms_per_step, 4),
        "unit": "ms/step", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{scene.name} {MODE_NAMES[mode]} K={K} forward+backward, {fb.n} Gaussians, "
                               f"{scene.width}x{scene.height}", "n_instances": fb.n_instances,
                   "densification_rows": densification_rows},
        "stages": {"blend_forward_ms": round(fwd_blend, 4), "backward_ms": round(bwd, 4), "blend_backward_ms": round(bwd_blend, 4),
                   "preprocess_backward_ms": round(bwd_prim, 4)},
        "roofline": roofline,
        "cpu_baseline": baseline}


def cpu_frame(oracle, fr, arrays):
    """One inference frame on the CPU oracle, stage by stage; seconds per stage (same stages as the GPU breakdown)."""
    t = [time.perf_counter()]
    pre = oracle.preprocess(fr, *arrays); t.append(time.perf_counter())
    offsets = oracle.inclusive_scan(pre["n_touched"]); t.append(time.perf_counter())
    keys, vals = oracle.create_instances(fr, pre, offsets); t.append(time.perf_counter())
    skeys, svals = oracle.sort_pairs(keys, vals, oracle.end_bit(fr)); t.append(time.perf_counter())
    ranges = oracle.extract_ranges(fr, skeys); t.append(time.perf_counter())
    oracle.blend(fr, pre, ranges, svals, True, False); t.append(time.perf_counter())
    names = ("preprocess", "scan", "create_instances", "sort", "extract_ranges", "blend")
    return {n: t[i + 1] - t[i] for i, n in enumerate(names)}


def bench_inference(scene_cpu, scene, config, n_override, mode, K, steps, warmup, fast=False, cpu_baseline=True):
    """One step = one ``rasterize()`` (``fast_rasterize()``) call; the line of that workload."""
    import torch
    from htgs_amd.torch_bindings import FrameBuffers, RasterizerMode, fast_rasterize, rasterize
    settings = scene.settings(RasterizerMode(mode), K)
    gauss = scene.gaussians()

    def step():
        if fast:
            return fast_rasterize(*gauss, settings, True)
        return rasterize(*gauss, settings, True, False)

    ms_per_step = timed_steps(step, steps, warmup)

    # ---- per-stage breakdown (HIP events on the launch stream), median over reps -------------------
    reps = max(5, min(30, steps))
    fb = FrameBuffers(*gauss, settings, True, False, fast=fast)
    fb.front()
    n_inst = fb.read_instance_count()
    fb.alloc_instances(n_inst)
    fb.back()
    torch.cuda.synchronize()
    n_vis = int((fb.n_touched != 0).sum().item())
    N, P, T = fb.n, fb.width * fb.height, fb.n_tiles
    B, kb = settings.active_sh_bases, fb.key_bytes
    passes = fb.sort_passes
    # every repetition runs the whole frame in order, so that each stage sees the data (and the caches) it sees
    # in a real frame: a radix sort that is re-run on its own sorted output, say, would look twice as fast
    stage_fns = (("preprocess", fb.preprocess), ("scan", fb.scan), ("create_instances", fb.create_instances),
                 ("sort", fb.sort), ("extract_ranges", fb.extract_ranges), ("blend", fb.blend))
    samples = {name: [] for name, _ in stage_fns}
    for rep in range(reps + 3):
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(len(stage_fns) + 1)]
        marks[0].record()
        for k, (_, fn) in enumerate(stage_fns):
            fn()
            marks[k + 1].record()
        marks[-1].synchronize()
        if rep >= 3:
            for k, (name, _) in enumerate(stage_fns):
                samples[name].append(marks[k].elapsed_time(marks[k + 1]))
    stages = {name: statistics.median(v) for name, v in samples.items()}
    blend_avg_ms = sum(samples["blend"]) / len(samples["blend"])
    # GLOBAL_ORDERING with the Gaussians sorted by depth first: the scan stage also sorts N (depth key, index) pairs --
    # every pass moves the 8-byte pairs once each way and reads the keys once more for its histogram -- and gathers
    # rectangles and counts in that order
    depth_passes = fb.lib.htgs_frame_depth_sort_passes(fb._ref)
    algo_bytes = {
        "preprocess": N * (56 + 12 * (B - 1) * (B > 1)) + 4 * N + 88 * n_vis,   # 80 B record + 8 B bounds per visible Gaussian
        "scan": 8 * N + (depth_passes * (2 * 8 + 4) * N + 8 * N + 16 * n_vis if depth_passes else 0),
        "create_instances": 16 * n_vis + (kb + 4) * n_inst,
        # every pass moves the pairs once each way; the keys are read once more for the histograms (the least a sort with
        # one histogram read can do; the kernels here read them once more per pass)
        "sort": passes * 2 * (kb + 4) * n_inst + kb * n_inst,
        "extract_ranges": kb * n_inst + 8 * T,
        "blend": 84 * n_inst + 16 * P,
    }
    stage_report = {
        k: {"ms": round(v, 4), "algo_GB": round(algo_bytes[k] / 1e9, 4),
            "GBps": round(algo_bytes[k] / 1e9 / (v / 1e3), 1), "frac_hbm": round(algo_bytes[k] / 1e9 / (v / 1e3) / HBM_PEAK_GBS, 4)}
        for k, v in stages.items()
    }
    tile_px = fb.tile * fb.tile
    blend_flops = FLOPS_PER_EVAL * tile_px * n_inst
    achieved_tflops = blend_flops / (blend_avg_ms / 1e3) / 1e12
    what = "fast_rasterize" if fast else "rasterize"
    roofline = {
        "kernel": "blend", "bound": "valu_fp32", "achieved": round(achieved_tflops, 3), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved_tflops / FP32_PEAK_TFLOPS, 4),
        "traffic": measured_traffic(workload_key(config, n_override, mode, K, what)),
        "launch_ms": round(blend_avg_ms, 4), "evals_per_launch": tile_px * n_inst,
    }

    if mode == 2:
        # GLOBAL_ORDERING stops a pixel once it is opaque, so the number of evaluations its blend kernel makes depends on
        # the data and 256 per instance would overstate it; the kernel priced here is the next one by time, the per-Gaussian
        # stage, which is bound by its HBM traffic
        pre_gbs = algo_bytes["preprocess"] / 1e9 / (stages["preprocess"] / 1e3)
        roofline = {"kernel": "preprocess", "bound": "hbm", "achieved": round(pre_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(pre_gbs / HBM_PEAK_GBS, 4),
                    "traffic": measured_traffic(workload_key(config, n_override, mode, K, what)),
                    "launch_ms": round(stages["preprocess"], 4)}

    # ---- CPU baseline: the C oracle on this box's host cores, one whole frame of the same workload ----
    baseline = None
    if cpu_baseline:
        import oracle
        fr = oracle_frame(oracle, scene_cpu, mode, K)
        arrays = [t.numpy() for t in scene_cpu.gaussians()]
        runs = [cpu_frame(oracle, fr, arrays) for _ in range(1 + CPU_REPS)][1:]         # the first run is the warm-up
        totals = sorted(sum(r.values()) for r in runs)
        cpu_s = totals[len(totals) // 2]
        baseline = {"value": round(1.0 / cpu_s, 4), "unit": "FPS", "cores": oracle.num_threads(), "kind": "port",
                    "stages_ms": {k: round(statistics.median(r[k] for r in runs) * 1e3, 2) for k in runs[0]},
                    "sample": f"whole frames of the same workload, C oracle with OpenMP; median of {CPU_REPS} runs after one warm-up, {cpu_s:.2f} s per frame"}

    return {
        "metric": f"FPS {MODE_NAMES[mode]} K={K} fast_rasterize (image only, reduced accuracy)" if fast
        else "FPS HYBRID_BLEND K=16 fwd @1080p, 3M Gaussians" if (config, mode, K, n_override) == (2, 0, 16, None)
        else f"FPS {MODE_NAMES[mode]} K={K} fwd",
        "value": round(1e3 / ms_per_step, 2), "unit": "FPS", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{scene.name} {MODE_NAMES[mode]} K={K} forward ({what}), {N} Gaussians, "
                               f"{scene.width}x{scene.height}, SH bases {B}",
                   "n_gaussians": N, "n_visible": n_vis, "n_instances": n_inst, "n_tiles": T, "key_bytes": kb, "sort_passes": passes},
        "stages": stage_report,
        "stage_sum_ms": round(sum(stages.values()), 4),
        "roofline": roofline,
        "cpu_baseline": baseline,
    }


def compact(line: dict) -> dict:
    """An entry of the ``configs`` block: the workload's line without the fields that repeat the headline's."""
    keep = ("metric", "value", "unit", "steps", "warmup", "ms_per_step", "higher_is_better", "config", "stages", "stage_sum_ms", "roofline")
    return {k: line[k] for k in keep if k in line}


def bench_all_configs(dev, headline_scene):
    """Every benchmark configuration beside the headline: name -> compact line.  ``headline_scene`` = the 3 M scene
    already on the device, as (cpu, gpu)."""
    import torch
    from htgs_amd.synthetic import make_scene
    from htgs_amd.torch_bindings.rasterization import ScratchPool
    out = {}

    def release():
        ScratchPool.clear()
        gc.collect()
        torch.cuda.empty_cache()

    scene_cpu, scene = headline_scene
    for mode in (1, 2, 3):
        out[f"cfg2/{MODE_NAMES[mode]}"] = compact(bench_inference(scene_cpu, scene, 2, None, mode, 16, EXTRA_STEPS, EXTRA_WARMUP, cpu_baseline=False))
    for mode in (0, 1, 2, 3):
        out[f"cfg2/{MODE_NAMES[mode]}/fast_rasterize"] = compact(bench_inference(scene_cpu, scene, 2, None, mode, 16, EXTRA_STEPS, EXTRA_WARMUP, fast=True,
                                                                                 cpu_baseline=False))
    del scene
    release()
    for config, K in ((0, 4), (1, 16), (3, 16)):
        scene_cpu = make_scene(config)
        scene = scene_cpu.to(dev)
        out[f"cfg{config}/HYBRID_BLEND"] = compact(bench_inference(scene_cpu, scene, config, None, 0, K, EXTRA_STEPS, EXTRA_WARMUP, cpu_baseline=False))
        del scene
        release()
    scene_cpu = make_scene(4)
    scene = scene_cpu.to(dev)
    for mode in (0, 1, 2, 3):
        out[f"cfg4/{MODE_NAMES[mode]}/train"] = compact(bench_training(scene_cpu, scene, 4, None, mode, 16, EXTRA_STEPS, EXTRA_WARMUP, cpu_baseline=False))
    del scene
    release()
    # a training step on the stress scene's distributions (1 M Gaussians): tiles with very long lists are shared between
    # waves and workgroups; beside it the same step with one wave (workgroup) per tile, as the reference walks them
    scene_cpu = make_scene(3, 1_000_000)
    scene = scene_cpu.to(dev)
    entry = compact(bench_training(scene_cpu, scene, 3, 1_000_000, 0, 16, 10, 3, cpu_baseline=False))
    single = bench_training(scene_cpu, scene, 3, 1_000_000, 0, 16, 5, 2, cpu_baseline=False, long_list_threshold=2 ** 31 - 1)
    entry["one_wave_per_tile"] = {"ms_per_step": single["ms_per_step"], "stages": single["stages"]}
    out["cfg3-n1000000/HYBRID_BLEND/train"] = entry
    del scene
    release()
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build renders one frame on one GPU; --gpus must be 1 "
              "(sharding over tile rows is designed, not implemented)", file=sys.stderr)
        sys.exit(2)
    import torch
    from htgs_amd.synthetic import make_scene

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate:
        from htgs_amd import diagnostics
        n_bytes = 1 << 30                      # larger than the 256 MB memory-side cache: both streams come from HBM
        src = torch.empty(n_bytes // 4, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(5):
            assert diagnostics.lib().htgs_diag_copy_bytes(dst.data_ptr(), src.data_ptr(), n_bytes, torch.cuda.current_stream(dev).cuda_stream) == 0
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "copy_bytes_kernel (htgs_amd/diagnostics/libhtgs_copy.so)", "bytes_read": n_bytes, "bytes_written": n_bytes,
                          "launches": 5}))
        return
    single = args.config is not None or args.mode is not None or args.K is not None or args.n is not None or args.train or args.fast \
        or args.headline_only
    config = 2 if args.config is None else args.config
    mode = 0 if args.mode is None else args.mode
    K = 16 if args.K is None else args.K
    scene_cpu = make_scene(config, args.n)
    scene = scene_cpu.to(dev)

    if args.train:
        line = bench_training(scene_cpu, scene, config, args.n, mode, K, args.steps, args.warmup, args.densification_rows, not args.no_cpu_baseline)
    else:
        line = bench_inference(scene_cpu, scene, config, args.n, mode, K, args.steps, args.warmup, args.fast, not args.no_cpu_baseline)
        if not single:
            line["configs"] = bench_all_configs(dev, (scene_cpu, scene))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
