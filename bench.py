#!/usr/bin/env python3
"""Benchmark of the differentiable tile rasterizer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--mode B]

A step is one forward + backward pass of `trigrad_amd.render` (L2 loss against a
seeded random target) over one synthetic frame that is already resident in HBM.
The default workload is the headline configuration (1,000,000 triangles,
1920x1080, float32, 16x16 tiles).  One JSON line is printed:

  value            forward+backward frames/s (the headline metric)
  roofline         the dominant HBM-bound kernel (one radix-sort sweep pass):
                   algorithmic bytes per launch / average launch duration from
                   events recorded on the launch stream, against 8 TB/s
  cpu_baseline     the CPU oracle (oracle/, a restatement of the reference's
                   algorithm; the reference has no CPU path) on the same frame,
                   OpenMP over tiles on the host cores of this box
  extra            forward-only frames/s, the other compositing mode, sort
                   Gkeys/s in-frame and on 10^7 synthetic keys, per-stage times,
                   binning+sort+ranges fraction of the HBM roofline
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(1, os.path.join(ROOT, "tests"))  # the seeded scene generators live with the tests

HBM_PEAK_GBS = 8000.0

# Bytes per launch of sort_sweep_kernel that pass the L2 on their way to the fabric are measured with rocprofv3 --pmc (read
# and write requests by size, and FETCH_SIZE / WRITE_SIZE scaled by a 256 MiB plain copy) and written into this summary as a
# lines "sort_sweep_kernel_traffic_bytes_per_launch=<bytes> keys=<K> commit=<hash>" and "lists_stage_traffic_bytes_per_frame=...";
# the bench line quotes them only for that K.
TRAFFIC_SUMMARY = os.path.join("profiles", "config2_hbm_traffic_counters.md")


def measured_traffic(what, n_keys):
    """-> (bytes or None, where the figure comes from): the line `<what>=<bytes> keys=<K> commit=<hash>` of the summary"""
    try:
        text = open(os.path.join(ROOT, TRAFFIC_SUMMARY)).read()
    except OSError:
        return None, None
    for line in text.splitlines():
        if line.startswith(what + "="):
            fields = dict(f.split("=", 1) for f in line.split())
            if int(fields.get("keys", -1)) == n_keys:
                return float(fields[what]), f"{TRAFFIC_SUMMARY} @ {fields.get('commit', '?')}"
    return None, f"{TRAFFIC_SUMMARY} holds no measurement for K={n_keys}"


def cpu_oracle_baseline(scene, mode, W, H, cores):
    """The CPU oracle (a restatement of the reference's algorithm; the reference has no CPU render path) on the same frame:
    per-stage wall time, once on one thread and, after a warm-up, as the median of three runs with OpenMP on `cores`
    threads (binning and sort are serial code either way; the blend passes run over tiles in parallel)."""
    import numpy as np
    from oracle import oracle as O
    v, i, c, o = scene["vertices"], scene["indices"], scene["colors"], scene["opacities"]
    T = O.n_tiles(W, H, 16, 16)

    def one_frame():
        t = [time.perf_counter()]
        em = O.bin_emit(v, i, W, H, 16, 16); t.append(time.perf_counter())
        keys, ids = O.sort_pairs_u64(em["keys64"], em["tri"]); t.append(time.perf_counter())
        offsets = O.tile_ranges(keys, T); t.append(time.perf_counter())
        bm = O.bary(v, i); t.append(time.perf_counter())
        fwd = O.forward(v, i, c, o, ids, offsets, bm, W, H, 16, 16, 1 / 256, mode["per_pixel_sort"], mode["max_layers"])
        t.append(time.perf_counter())
        gi = (2.0 * (fwd["image"] - scene["target"]) / fwd["image"].size).astype(np.float32)
        O.backward(gi, np.zeros((H, W), np.float32), v, i, c, o, ids, offsets, bm, fwd, W, H, 16, 16, mode["per_pixel_sort"],
                   mode["max_layers"])
        t.append(time.perf_counter())
        return dict(zip(("binning", "sort", "ranges", "bary", "forward", "backward"), np.diff(t)))

    def totals(stages):
        stages = {k: round(float(s), 4) for k, s in stages.items()}
        fwd = sum(stages[k] for k in ("binning", "sort", "ranges", "bary", "forward"))
        return dict(stage_seconds=stages, forward_seconds=round(fwd, 4), forward_backward_seconds=round(fwd + stages["backward"], 4))

    O.set_threads(1)
    single = totals(one_frame())
    O.set_threads(cores)
    one_frame()  # warm-up
    runs = [one_frame() for _ in range(3)]
    many = totals({k: float(np.median([r[k] for r in runs])) for k in runs[0]})
    return single, many


MODES = {
    "A": dict(per_pixel_sort=True, max_layers=32),    # API defaults
    "B": dict(per_pixel_sort=False, max_layers=-1),   # tile-order compositing, early termination, full reverse traversal
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--mode", choices=sorted(MODES), default="B")
    ap.add_argument("--sort-keys", type=int, default=10_000_000)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain device copies of 256 MiB (a known traffic, for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import trigrad_amd
    from trigrad_amd import _C
    import scenes

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    scene = scenes.config(args.config)
    W, H = scene["width"], scene["height"]
    M = scene["indices"].shape[0]
    T = _C.num_tiles(W, H, 16, 16)
    d = {k: torch.from_numpy(v).to(dev) for k, v in scene.items() if isinstance(v, np.ndarray)}
    verts = d["vertices"].clone().requires_grad_()
    colors = d["colors"].clone().requires_grad_()
    opac = d["opacities"].clone().requires_grad_()

    def step(mode, backward=True):
        verts.grad = colors.grad = opac.grad = None
        image, depthmap = trigrad_amd.render(verts, d["indices"], colors, opac, W, H, 16, 16, 1 / 256, False, **MODES[mode])
        if backward:
            loss = torch.nn.functional.mse_loss(image, d["target"])
            loss.backward()
        return image

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1000.0 / steps

    ms = timed(lambda: step(args.mode), args.steps, args.warmup)

    if args.calibrate_copy:
        src = torch.empty((64 << 20,), dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ---- per-kernel durations from events on the launch stream -------------------
    _C.profile_enable(True)
    _C.profile_report()
    prof_steps = max(3, min(args.steps, 10))
    for _ in range(prof_steps):
        step(args.mode)
    torch.cuda.synchronize()
    prof = _C.profile_report()
    _C.profile_enable(False)
    counts = _C.bin_count(d["vertices"], d["indices"], W, H, 16, 16)
    K = int(counts.sum().item())
    # the 8-bit LSD pipeline that the byte model prices: passes over all key bits.  The frame's sort moves the pairs
    # through memory for the tile bits only (one pass by tile column, one by tile row) and sorts the depth bits per tile
    # in LDS (one more read and write of every pair).
    model_passes = (_C.key_bits(T) + 7) // 8
    sweep_n, sweep_ms = prof["sort_sweep_kernel"]
    sweep_avg_s = sweep_ms / sweep_n / 1000.0
    sweep_bytes = 24.0 * K
    achieved = sweep_bytes / sweep_avg_s / 1e9
    passes_through_memory = sweep_n // prof_steps
    per_step = {k: v[1] / prof_steps for k, v in prof.items()}
    # binning + sort + ranges: every kernel from the triangles to the sorted tile lists and their offsets
    sort_kernels = ["fill_zero_kernel", "sort_histogram_kernel", "sort_bases_kernel", "sort_sweep_kernel", "tile_ranges_kernel",
                    "segment_sort_small_kernel", "segment_sort_large_kernel"]
    bin_sort_kernels = ["bin_count_kernel", "scan_init_kernel", "scan_lookback_kernel", "bin_emit_kernel", "bin_init_kernel",
                        "bin_setup_kernel", "bin_emit_records_kernel", "frame_scan_kernel", "frame_emit_kernel"] + sort_kernels
    bin_sort_ms = sum(per_step.get(k, 0.0) for k in bin_sort_kernels)
    # the byte model of an 8-bit LSD key pipeline: count 64 M, scan 8 M, emit 64 M + 12 K, histogram 8 K, passes 24 K each,
    # ranges 8 K + 4 (T + 1)
    bin_sort_bytes = 136.0 * M + 28.0 * K + 24.0 * model_passes * K + 4.0 * (T + 1)
    # what this build's kernels move: scan (60 M read, 4 M offsets + 48 M records written), emission (records and
    # offsets read, 12 K written), the passes through memory, the per-tile depth sort (24 K), counts and offsets per tile
    moved_bytes = (60.0 + 52.0) * M + (52.0 * M + 12.0 * K) + 24.0 * passes_through_memory * K + 24.0 * K + 12.0 * (T + 1)
    sort_ms = sum(per_step.get(k, 0.0) for k in sort_kernels)
    traffic, traffic_source = measured_traffic("sort_sweep_kernel_traffic_bytes_per_launch", K)
    stage_traffic, stage_traffic_source = measured_traffic("lists_stage_traffic_bytes_per_frame", K)

    out = {
        "metric": "fwd+bwd frames/s (1M tris, 1920x1080)" if args.config == 2 else f"fwd+bwd frames/s (config {args.config})",
        "value": 1000.0 / ms,
        "unit": "frames/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"config{args.config}: {M} triangles, {W}x{H}, 16x16 tiles, K={K} keys, "
                               f"per_pixel_sort={MODES[args.mode]['per_pixel_sort']}, max_layers={MODES[args.mode]['max_layers']}",
                   "mode": args.mode},
        "roofline": {"bound": "hbm", "kernel": "sort_sweep_kernel", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
                     "bytes_per_launch": sweep_bytes, "avg_launch_us": sweep_avg_s * 1e6},
    }

    extra = {
        "kernel_ms_per_step": {k: round(v, 4) for k, v in sorted(per_step.items())},
        "binning_sort_ranges": {"ms": bin_sort_ms, "algorithmic_bytes": bin_sort_bytes,
                                "algorithmic_bytes_model": f"8-bit LSD key pipeline with {model_passes} passes over all key bits",
                                "GBps": bin_sort_bytes / (bin_sort_ms / 1000.0) / 1e9,
                                "frac_of_hbm_peak": bin_sort_bytes / (bin_sort_ms / 1000.0) / 1e9 / HBM_PEAK_GBS,
                                "moved_bytes": moved_bytes,
                                "moved_bytes_model": "what the kernels read and write by their access pattern (not counters)",
                                "frac_of_hbm_peak_moved": moved_bytes / (bin_sort_ms / 1000.0) / 1e9 / HBM_PEAK_GBS,
                                "traffic_bytes_by_counters": stage_traffic, "traffic_source": stage_traffic_source},
        "sort_in_frame": {"keys": K, "passes_through_memory": passes_through_memory, "passes_of_the_byte_model": model_passes,
                          "depth_bits": "sorted per tile in LDS: one more read and write of every pair",
                          "ms": sort_ms, "Gkeys_per_s": K / (sort_ms / 1000.0) / 1e9},
    }
    # the blend kernels against the HBM roofline, to show that it does not bound them: compulsory bytes are
    # 148 B per list entry plus the per-pixel and per-vertex arrays (forward 28 B/pixel; backward 48 B/pixel + 64 B/vertex)
    V, P = d["vertices"].shape[0], W * H
    blend = {}
    for name, nbytes in (("forward", 148.0 * K + 28.0 * P), ("backward", 148.0 * K + 48.0 * P + 64.0 * V)):
        kms = sum(v for k, v in per_step.items() if k.startswith(name))
        if kms > 0:
            blend[name] = {"ms": kms, "compulsory_bytes": nbytes, "GBps": nbytes / (kms / 1000.0) / 1e9,
                           "frac_of_hbm_peak": nbytes / (kms / 1000.0) / 1e9 / HBM_PEAK_GBS, "bound": "vector issue / LDS, not HBM"}
    extra["blend_kernels_vs_hbm"] = blend
    if not args.no_extras:
        extra["forward_only_fps"] = 1000.0 / timed(lambda: step(args.mode, backward=False), args.steps, 1)
        other = "A" if args.mode == "B" else "B"
        extra[f"mode_{other}_fwd_bwd_fps"] = 1000.0 / timed(lambda: step(other), max(3, args.steps // 2), 1)
        extra[f"mode_{other}_forward_only_fps"] = 1000.0 / timed(lambda: step(other, backward=False), max(3, args.steps // 2), 1)
        # what a plain device copy reaches on this box (256 MiB read + 256 MiB written), for scale
        src = torch.empty((64 << 20,), dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        t_copy = timed(lambda: dst.copy_(src), 10, 2)
        extra["device_copy_GBps"] = 2.0 * src.numel() * 4 / (t_copy / 1000.0) / 1e9
        del src, dst
        # standalone sort at the scale the metric names
        n = args.sort_keys
        keys_np, vals_np = scenes.sort_keys(n, T, seed=0)
        keys0 = torch.from_numpy(keys_np.view(np.int64)).to(dev)
        vals0 = torch.from_numpy(vals_np).to(dev)
        kbuf, vbuf = torch.empty_like(keys0), torch.empty_like(vals0)

        def sort_once():
            kbuf.copy_(keys0)
            vbuf.copy_(vals0)
            _C.sort_pairs(kbuf, vbuf, _C.key_bits(T))

        def copy_only():
            kbuf.copy_(keys0)
            vbuf.copy_(vals0)
        t_sort = timed(sort_once, 10, 2) - timed(copy_only, 10, 2)
        extra["sort_standalone"] = {"keys": n, "ms": t_sort, "Gkeys_per_s": n / (t_sort / 1000.0) / 1e9,
                                    "GBps": (8.0 + 24.0 * model_passes) * n / (t_sort / 1000.0) / 1e9}
        # the same pairs through the sort the frame uses (tile bits through memory, depth bits per tile in LDS)
        def tile_sort_once():
            kbuf.copy_(keys0)
            vbuf.copy_(vals0)
            _C.sort_tile_lists(kbuf, vbuf, T)
        t_tile = timed(tile_sort_once, 10, 2) - timed(copy_only, 10, 2)
        extra["tile_list_sort_standalone"] = {"keys": n, "tiles": T, "ms": t_tile, "Gkeys_per_s": n / (t_tile / 1000.0) / 1e9,
                                              "note": "same sorted keys, values and tile ranges as the 45-bit sort + tg_tile_ranges"}
        # the sweep kernel alone at this size, from the library's events: 24 bytes per pair and launch
        _C.profile_enable(True)
        _C.profile_report()
        for _ in range(5):
            sort_once()
        torch.cuda.synchronize()
        big = _C.profile_report()
        _C.profile_enable(False)
        launches, total_ms = big["sort_sweep_kernel"]
        sweep_us = total_ms / launches * 1000.0
        extra["sort_standalone"]["sweep_kernel"] = {"avg_launch_us": sweep_us, "GBps": 24.0 * n / (sweep_us * 1e-6) / 1e9,
                                                    "frac_of_hbm_peak": 24.0 * n / (sweep_us * 1e-6) / 1e9 / HBM_PEAK_GBS}
        # the one scene the reference publishes a time for (notebooks/renderer.ipynb:79, 93-95: 10.9 ms without and
        # 11.5 ms with per-pixel sort, forward only, GPU not stated): 500 x 500 staggered grid, opacity 1, 500 x 500 px
        del kbuf, vbuf, keys0, vals0
        grid = scenes.grid_mesh(500, 500, -0.9, 0.9, -0.9, 0.9)
        g = {k: torch.from_numpy(v).to(dev) for k, v in grid.items() if isinstance(v, np.ndarray)}
        ref_scene = {"triangles": int(grid["indices"].shape[0]), "vertices": int(grid["vertices"].shape[0]),
                     "reference_notebook_ms": {"per_pixel_sort_false": 10.9, "per_pixel_sort_true": 11.5}}
        for pps in (False, True):
            t = timed(lambda: trigrad_amd.render(g["vertices"], g["indices"], g["colors"], g["opacities"], per_pixel_sort=pps), 20, 3)
            ref_scene[f"forward_ms_per_pixel_sort_{str(pps).lower()}"] = t
        extra["reference_timing_scene"] = ref_scene
    out["extra"] = extra

    if not args.no_cpu_baseline:
        from oracle import oracle as O
        cores = min(O.max_threads(), len(os.sched_getaffinity(0)), 16)
        single, many = cpu_oracle_baseline(scene, MODES[args.mode], W, H, cores)
        out["cpu_baseline"] = {"value": 1.0 / many["forward_backward_seconds"], "unit": "frames/s", "cores": cores, "kind": "port",
                               "mode": args.mode,
                               "sample": "the same frame, forward + backward: OpenMP over tiles after one warm-up, median of three "
                                         "runs (binning, sort and ranges are serial code); the single-thread figures are one run",
                               "openmp": many, "single_thread": dict(single, cores=1,
                                                                     value=1.0 / single["forward_backward_seconds"])}
        # the other compositing mode on the same frame, same protocol
        other = "A" if args.mode == "B" else "B"
        single, many = cpu_oracle_baseline(scene, MODES[other], W, H, cores)
        out["cpu_baseline"]["other_mode"] = {"mode": other, "value": 1.0 / many["forward_backward_seconds"], "cores": cores, "openmp": many,
                                             "single_thread": dict(single, cores=1, value=1.0 / single["forward_backward_seconds"])}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
