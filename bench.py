#!/usr/bin/env python3
"""bench.py - throughput of the full 3D-Gaussian-splatting training step (fwd + loss + bwd + Adam) on one MI355X.

    python bench.py [--gpus 1] [--steps 20] [--warmup 5] [--config 3] [--no-cpu-baseline]

Workload (BASELINE.json configs[2], the one the metric is quoted on): 1M SH-degree-3 Gaussians drawn from the
32-cluster mixture, one 1237x822 pinhole camera on a radius-4 orbit, L = 0.8 L1 + 0.2 (1 - SSIM) against the render
of an independently seeded 1M-Gaussian target scene, fused Adam over all parameter tensors.  Inputs are synthetic
and already resident in HBM when the timed region starts.

Prints ONE JSON line: it/s over exactly --steps steps (wall clock; median / min / max of the steps from HIP events
beside it), the dominant kernel's roofline figures measured with HIP events inside the timed region, per-kernel
times / rates from a separate instrumented pass, and the CPU checker timed on the host cores on the same workload (a
reported baseline, not a target) - whose loss of the first iteration is compared with the GPU's (`parity_in_bench`).
The camera tensor changes every step, as in a training loop: the forward pass cannot reuse the previous step's tile
costs (--same-camera hands over one tensor throughout).
"""
import argparse
import ctypes
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG_DIR = os.path.join(ROOT, "lichtfeld-studio_amd")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of the dominant kernel at the default workload come from two rocprofv3 --pmc runs (FETCH_SIZE,
# WRITE_SIZE, each scaled by what the same counter reads for gsx_debug_copy's known 1 GiB + 1 GiB).  Counters cannot
# be read from inside this process: the figure is read from the committed summary of those runs, and only attached
# when the workload is the one it was measured on.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "train_step_1M_1237x822_hbm_traffic.txt")


def measured_traffic_bytes(kernel_prefix):
    """total_MB column of the kernel's row in the traffic summary, in bytes (None without the file / the row)"""
    try:
        with open(TRAFFIC_SUMMARY) as f:
            for line in f:
                if line.startswith(kernel_prefix):
                    return float(line.split()[-1]) * 1e6
    except (OSError, ValueError):
        pass
    return None

# published MI355X peaks
PEAK_HBM_GBS = 8000.0
PEAK_FP32_TFLOPS = 157.3

# algorithmic cost model: bytes per Gaussian / pixel / element, flops per (pixel, Gaussian) pair
FLOPS_PAIR_FWD = 62.0          # evaluate one pair: 2 mat-vec, normalise, cross, dot, alpha/T update
FLOPS_PAIR_FWD_COMPOSITE = 6.0  # colour FMAs of a composited pair
FLOPS_PAIR_BWD_EVAL = 62.0     # recompute
FLOPS_PAIR_BWD_VJP = 180.0     # VJP chain of a valid pair


def load_package():
    name = "lichtfeld_studio_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"),
                                                  submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def algorithmic_bytes(N, K, H, W, n_isects, sort_bits, key_bytes=8):
    """HBM bytes one launch of each streaming stage has to move (reads + writes), per the cost model.
    key_bytes: 8 for (tile << 32 | depth) keys, 2 for the 16-bit tile indices (sort_bits then counts from bit 0)."""
    P = H * W
    # the pairs are emitted in depth order: only the tile (/ camera) bits are sorted
    passes = (sort_bits - (32 if key_bytes == 8 else 0) + 7) // 8
    pair = key_bytes + 4
    return {
        "activate_params": N * (32 + 32),
        "projection_ut_3dgs_fused": N * (44 + 32),
        "activate_project_ut": N * (44 + 32 + 32),
        "activate_project_sh_records": N * (44 + 32 + 32 + 12 * K + 12 + 96),
        "sh_colors_from_world": N * (12 + 12 * K + 8 + 12),
        "intersect_tile_emit": N * (4 + 16 + 4 + 8) + n_isects * pair,
        "intersect_tile_count_ordered": N * (28 + 16 + (8 + 24) * 4 + 8 + 8),
        "radix_sort_pairs": n_isects * (key_bytes + 2 * pair) * passes,
        "intersect_offset": n_isects * key_bytes + (P // 256) * 4,
        "image_from_render": P * (12 + 12 + 12),
        "fusedssim": P * (24 + 12 + 36),
        "photometric_loss_forward": P * (12 + 12 + 36),
        "photometric_loss_backward": P * (12 + 12 + 36 + 12),
        "fusedssim_backward": P * (72 + 12),
        "render_grad_from_loss": P * (12 + 12 + 12 + 12 + 12),
        "pack_raster_records": N * (56 + 96),
        "sh_colors_records_from_world": N * (12 + 12 * K + 8 + 32 + 12 + 96),
        "rasterize_bwd_clear": N * 64,
        "rasterize_bwd_finish": N * (64 + 40 + 56),
        "sh_colors_from_world_bwd": N * (12 + 8 + 12 + 12 + 12 * K),
        "activate_params_bwd": N * (32 + 32 + 32),
        "adam_step_multi": N * (11 + 3 * K) * 28,
        "backward_update_fused": N * ((11 + 3 * K) * 24 + 64 + 64 + 12 + 8),
    }


def run_mcmc_part(ts, dev, reps=5):
    """What configuration 4 runs behind the step (mcmc.cpp:112-190, 349-367): relocation of the 5 % of the Gaussians
    with the lowest opacity onto Gaussians drawn from a multinomial over the others' opacities (Eq. 9 rebalancing,
    n_max = 51), and noise on the means.  The draw is the caller's (torch, outside the timed calls); the two library
    calls are timed with HIP events.  Not part of `value`: the metric is the step."""
    import numpy as np
    import torch
    n_dead = ts.N // 20
    op = torch.sigmoid(ts.params["opacity"].reshape(-1))
    order = torch.argsort(op, stable=True)
    dead = torch.sort(order[:n_dead]).values.contiguous()
    alive = torch.sort(order[n_dead:]).values
    g = torch.Generator(device=dev).manual_seed(44)
    # torch.multinomial takes at most 2^24 categories: draw by inverting the cumulative distribution
    cdf = torch.cumsum(op[alive].double(), 0)
    u = torch.rand(n_dead, generator=g, device=dev, dtype=torch.float64) * cdf[-1]
    sampled = alive[torch.searchsorted(cdf, u).clamp_(max=alive.numel() - 1)].contiguous()
    b = np.zeros((51, 51), np.float32)
    for n in range(51):
        for k in range(n + 1):
            x = np.float32(1.0)
            for i in range(k):
                x = np.float32(x * (np.float32(n - i) / np.float32(i + 1)))
            b[n, k] = x
    binoms = torch.from_numpy(b).to(dev)
    t_rel, t_noise = [], []
    for r in range(reps):
        e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e[0].record()
        ts.relocate(sampled, dead, binoms)
        e[1].record()
        ts.inject_noise(None, seed=r)
        e[2].record()
        torch.cuda.synchronize()
        t_rel.append(e[0].elapsed_time(e[1]))
        t_noise.append(e[1].elapsed_time(e[2]))
    return {"relocated": int(n_dead), "relocate_ms": round(float(np.median(t_rel)), 4),
            "noise_ms": round(float(np.median(t_noise)), 4),
            "what": "gsx_mcmc_relocate (5 % of the Gaussians, caller-drawn index sets) and gsx_add_noise_philox after "
                    "the timed steps; not part of value"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=3, help="BASELINE configuration (3 = the metric's)")
    ap.add_argument("--n", type=int, default=None, help="override the number of Gaussians (parity / debugging)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--separate-update", action="store_true",
                    help="run epilogue / SH backward / activation VJPs / Adam as separate kernels (default: one pass)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="keep every kernel of the step on one stream (default: the SH / record pass and the loss "
                         "reduction run on a second stream beside the sort chain / the backward rasterizer)")
    ap.add_argument("--one-front-pass", action="store_true",
                    help="activations + projection + SH colours + records as one launch")
    ap.add_argument("--same-camera", action="store_true",
                    help="hand the step the same camera tensor every time: the forward pass then orders its tiles by "
                         "the previous step's costs (default: two tensors in turn, same pose, as in a training loop "
                         "that changes camera every step)")
    ap.add_argument("--no-tile-order", action="store_true", help="rasterize the tiles in index order")
    ap.add_argument("--host-count", action="store_true",
                    help="fetch the pair count to the host in every step (default: it stays on the device)")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads for the CPU baseline (0 = all)")
    ap.add_argument("--workload", choices=["gut", "ops_path", "fastgs"], default="gut",
                    help="gut: the training step of the metric (default); ops_path: the same step issued operator by "
                         "operator through the C++ mirror of gsplat/Ops.h, with autograd and ATen glue, as "
                         "LichtFeld's trainer issues it; fastgs: forward + backward of the reference's default "
                         "rasterizer on the same scene (a secondary line, not the metric)")
    ap.add_argument("--no-boundary-path", action="store_true",
                    help="leave the operator-by-operator step (boundary_path) out of the default line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path has no multi-GPU part); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    gsx = load_package()
    gsx._lib.lib()  # fail loudly without the HIP library
    from lichtfeld_studio_amd.trainer import TrainStep
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")

    t0 = time.time()
    sc = gsx.scenes.config(args.config, args.n)
    cam = sc.cameras[0]
    W, H = cam.width, cam.height
    if args.workload == "fastgs":
        return run_fastgs(args, gsx, sc, cam, dev)
    viewmat = torch.from_numpy(cam.viewmat[None].copy()).to(dev)
    Kmat = torch.from_numpy(cam.K[None].copy()).to(dev)
    # target: render of the independently seeded target scene by the same forward, clamped, CHW
    if hasattr(sc, "target_scene"):
        tgt = TrainStep(sc.target_scene, dev)
        tgt.forward(viewmat, Kmat, W, H)
        gt = tgt.render[0].clamp(0, 1).permute(2, 0, 1).contiguous()[None].clone()
        del tgt
        torch.cuda.empty_cache()
    elif hasattr(sc, "target"):
        gt = torch.from_numpy(sc.target[None].copy()).to(dev)
    else:
        sys.exit(f"bench.py: configuration {args.config} has no training target (a forward-only parity case); "
                 "the training step is timed on configurations 1, 3, 4 and 5")
    use_ssim = args.config != 1  # configuration 1 is L1 only
    if args.workload == "ops_path":
        res = run_ops_path(args, gsx, sc, viewmat, Kmat, W, H, gt, dev)
        print(json.dumps({
            "metric": "train it/s issued operator by operator through the gsplat/Ops.h mirror (secondary; the "
                      "BASELINE metric is the default workload)",
            "value": res["it_per_s"], "unit": "it/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": f"BASELINE configs[{args.config - 1}] through OpsPathTrainer "
                                   "(csrc/host/ops_path.cpp)", "n_gaussians": int(sc.means.shape[0]),
                       "image": [W, H]}, "boundary_path": res}))
        return
    ts = TrainStep(sc, dev, use_ssim=use_ssim, fused_update=not args.separate_update,
                   fused_loss=not args.separate_update, overlap=not args.no_overlap,
                   one_front_pass=args.one_front_pass, device_count=not args.host_count)
    ts.order_tiles = not args.no_tile_order
    setup_s = time.time() - t0

    dominant = "rasterize_bwd_accumulate"
    views = [viewmat] if args.same_camera else [viewmat, viewmat.clone()]
    first_loss = None
    for i in range(args.warmup):
        ts.step(views[i % len(views)], Kmat, W, H, gt)
        if i == 0:  # from the initial state: what the CPU baseline's step computes too
            first_loss = [float(x) for x in ts.loss_out.cpu()]
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    ts.start_timing([dominant])  # two event records per step around the dominant kernel
    t1 = time.perf_counter()
    for i in range(args.steps):
        marks[i].record()
        ts.step(views[i % len(views)], Kmat, W, H, gt)
    marks[args.steps].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t1
    in_loop = ts.stop_timing()
    ms_per_step = 1e3 * elapsed / args.steps
    step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    loss = [float(x) for x in ts.loss_out.cpu()]
    lists_error = ts.lists_error()
    assert lists_error == (0, 0), f"tile lists: error bits {lists_error[0]}, steps held back {lists_error[1]}"

    # pair counts of the last forward (for flop rates)
    stats = torch.zeros(8, dtype=torch.int64, device=dev)
    L = gsx._lib
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    L.check(L.lib().gsx_rasterize_pair_stats(
        ctypes.c_int64(ts.n_isects), p(ts.records), ctypes.c_uint32(W), ctypes.c_uint32(H), p(viewmat), p(Kmat),
        p(ts.offsets), p(ts.flatten_ids), p(stats), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    pairs_fwd, pairs_comp, pairs_bwd, wave_iters, wave_skipped, wave_hits, half_rows, half_cols = [
        int(x) for x in stats.cpu()[:8]]
    # ... and of the backward kernel itself: pairs whose alpha it evaluates, pairs that receive a gradient
    bstats = torch.zeros(4, dtype=torch.int64, device=dev)
    L.check(L.lib().gsx_rasterize_bwd_pair_stats(
        ctypes.c_int64(ts.n_isects), p(ts.records), ctypes.c_uint32(W), ctypes.c_uint32(H), p(viewmat), p(Kmat),
        p(ts.offsets), p(ts.flatten_ids), p(ts.alpha), p(ts.last_ids), p(bstats),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    bwd_evaluated, bwd_valid, bwd_wave_iters = [int(x) for x in bstats.cpu()[:3]]

    # instrumented pass: every stage bracketed by events (not part of the timed region)
    ts.start_timing(None)
    n_prof = 6
    for i in range(n_prof):
        ts.step(views[i % len(views)], Kmat, W, H, gt)
    stage_ms = {k: float(np.mean(v)) for k, v in ts.stop_timing().items()}

    mcmc = None
    if args.config == 4:
        mcmc = run_mcmc_part(ts, dev)

    # known-size copy: the yardstick for byte counters and the measured streaming bandwidth of this GPU
    copy_bytes = 1 << 30  # well beyond the 256 MB last-level cache
    cp_src = torch.empty(copy_bytes, dtype=torch.uint8, device=dev)
    cp_dst = torch.empty(copy_bytes, dtype=torch.uint8, device=dev)
    cp_src.zero_()
    copy_ms = []
    for _ in range(4):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        L.check(L.lib().gsx_debug_copy(p(cp_src), p(cp_dst), ctypes.c_size_t(copy_bytes),
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        e1.record()
        torch.cuda.synchronize()
        copy_ms.append(e0.elapsed_time(e1))
    copy_gbs = 2 * copy_bytes / (min(copy_ms[1:]) * 1e-3) / 1e9
    del cp_src, cp_dst

    tile_bits = int(L.lib().gsx_n_bits(ctypes.c_uint32(ts.tw * ts.th)))
    abytes = (algorithmic_bytes(ts.N, ts.K, H, W, ts.n_isects, tile_bits, 2) if ts.compact else
              algorithmic_bytes(ts.N, ts.K, H, W, ts.n_isects, 32 + tile_bits + 1))
    if ts._lists_active:
        # gsx_tile_lists by what it has to move: the projection's outputs in; per Gaussian that touches a tile a key,
        # an id and a rectangle written and four radix passes over key + id (read + write); per (super-tile, Gaussian)
        # entry a key + id written, one radix pass over them and their read by the gather; the lists and offsets out
        _, pairs, visible, entries = ts.lists_counts()
        abytes["tile_lists"] = (ts.N * 20 + visible * (16 + 4 * 24) + entries * (12 + 24 + 12) + pairs * 4 +
                                (ts.tw * ts.th + 1) * 4)
        # the SH / record pass reads every row's radii and skips the rows the projection culled: it is priced by
        # the rows it moves (mean, coefficients, activated parameters in; colour and record out)
        abytes["sh_colors_records_from_world"] = ts.N * 8 + visible * (12 + 12 * ts.K + 32 + 12 + 96)
    kernels = {}
    for k, ms in stage_ms.items():
        e = {"ms": round(ms, 4)}
        if k in abytes and ms > 0:
            gbs = abytes[k] / (ms * 1e-3) / 1e9
            e.update(bound="hbm", alg_bytes=int(abytes[k]), GBps=round(gbs, 1), frac=round(gbs / PEAK_HBM_GBS, 4))
        kernels[k] = e
    # algorithmic flops: 62 + 180 per VALID pair of the backward pass (the pairs that receive a gradient), 62 + 6 per
    # evaluated / composited pair of the forward pass
    flops_fwd = FLOPS_PAIR_FWD * pairs_fwd + FLOPS_PAIR_FWD_COMPOSITE * pairs_comp
    flops_bwd = (FLOPS_PAIR_BWD_EVAL + FLOPS_PAIR_BWD_VJP) * bwd_valid
    flops_bwd_evaluated = FLOPS_PAIR_BWD_EVAL * bwd_evaluated + FLOPS_PAIR_BWD_VJP * bwd_valid
    flops_bwd_reference_walk = FLOPS_PAIR_BWD_EVAL * pairs_bwd + FLOPS_PAIR_BWD_VJP * pairs_comp
    dom_ms = float(np.mean(in_loop[dominant]))
    for k, fl, ms in (("rasterize_to_pixels_from_world_3dgs_fwd", flops_fwd,
                       stage_ms.get("rasterize_to_pixels_from_world_3dgs_fwd", 0.0)), (dominant, flops_bwd, dom_ms)):
        if ms > 0:
            tf = fl / (ms * 1e-3) / 1e12
            kernels.setdefault(k, {}).update(ms=round(ms, 4), bound="fp32_valu", alg_flops=int(fl),
                                             TFLOPs=round(tf, 2), frac=round(tf / PEAK_FP32_TFLOPS, 4))
    tflops = lambda fl: fl / (dom_ms * 1e-3) / 1e12
    dom_tf = tflops(flops_bwd)
    default_workload = args.config == 3 and ts.N == 1_000_000
    roofline = {
        "kernel": "rasterize_bwd_kernel", "bound": "fp32_valu", "achieved": round(dom_tf, 3),
        "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s", "frac": round(dom_tf / PEAK_FP32_TFLOPS, 4),
        "traffic": measured_traffic_bytes("gsx::rasterize_bwd_kernel<3u, false, false, false>") if default_workload else None,
        "avg_launch_ms": round(dom_ms, 4), "launches": len(in_loop[dominant]),
        "frac_nonpacked": round(dom_tf / (PEAK_FP32_TFLOPS / 2), 4),
        "frac_pairs_evaluated": round(tflops(flops_bwd_evaluated) / PEAK_FP32_TFLOPS, 4),
        "frac_reference_walk": round(tflops(flops_bwd_reference_walk) / PEAK_FP32_TFLOPS, 4),
        "pairs_valid": bwd_valid, "pairs_evaluated": bwd_evaluated, "pairs_reference_walk": pairs_bwd,
        "note": "no MFMA and not HBM-bound: per-pair fp32 vector ALU work.  achieved = 242 flops x valid pairs "
                "(pairs that receive a gradient) / the kernel's average launch time inside the timed region; "
                "frac_nonpacked prices it against the 78.6 TFLOP/s this build can issue (packed fp32 is switched "
                "off); frac_pairs_evaluated adds 62 flops for every pair whose alpha the kernel evaluates, "
                "frac_reference_walk counts the pairs the reference's kernel walks.  traffic = HBM bytes per launch "
                "(rocprofv3 FETCH_SIZE + WRITE_SIZE, copy-kernel calibrated) from profiles/",
    }

    # the same step through the C++ layers a LichtFeld build links: operator by operator as its trainer issues them
    # (ops_path), and the C++ step driver over the fused entry points (cpp_train_step)
    boundary = None
    if default_workload and not args.no_boundary_path and not args.separate_update:
        boundary = {"ops_path": run_ops_path(args, gsx, sc, viewmat, Kmat, W, H, gt, dev),
                    "cpp_train_step": run_cpp_step(args, gsx, sc, viewmat, Kmat, W, H, gt, dev)}
        headline = args.steps / elapsed
        boundary["ops_path_vs_headline"] = round(boundary["ops_path"]["it_per_s"] / headline, 3)
        boundary["cpp_train_step_vs_headline"] = round(boundary["cpp_train_step"]["it_per_s"] / headline, 3)

    cpu_baseline, parity = None, None
    if not args.no_cpu_baseline:
        cpu_baseline = run_cpu_baseline(gsx, sc, cam, gt.cpu().numpy()[0], use_ssim, args.cpu_threads)
        if first_loss is not None:
            # both sides ran one iteration from the same initial parameters against the same target image
            diff = max(abs(a - b) for a, b in zip(first_loss, cpu_baseline["loss"]))
            parity = {"what": "loss, L1 and SSIM terms of the first iteration, GPU step vs CPU checker step",
                      "gpu": [round(x, 7) for x in first_loss], "cpu": cpu_baseline["loss"],
                      "max_abs_diff": float(f"{diff:.3e}"), "tolerance": 1e-5, "ok": bool(diff <= 1e-5)}

    out = {
        "metric": "train it/s (fwd+bwd+Adam) at 1M SH3 Gaussians 1237x822; raster fwd/bwd ms",
        "value": round(args.steps / elapsed, 3), "unit": "it/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3),
        "step_ms": {"median": round(step_ms[len(step_ms) // 2], 4), "min": round(step_ms[0], 4),
                    "max": round(step_ms[-1], 4), "note": "per-step HIP-event times inside the timed region"},
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"BASELINE configs[{args.config - 1}]: {ts.N} Gaussians SH degree {ts.sh_degree}, "
                               f"{W}x{H}, fwd + " + ("0.8 L1 + 0.2 (1-SSIM)" if use_ssim else "L1") +
                               " + bwd + fused Adam", "n_gaussians": ts.N, "image": [W, H], "n_isects": ts.n_isects,
                   "tiles": ts.tw * ts.th, "tile_list_counts": dict(zip(("pairs_in_lists", "pairs", "gaussians_on_tiles",
                                                                         "super_tile_entries"), ts.lists_counts())),
                   "pairs_fwd": pairs_fwd, "pairs_composited": pairs_comp,
                   "pairs_bwd": pairs_bwd, "camera_tensor": "same every step" if args.same_camera else "changes every step",
                   "pair_count": "fetched by the host" if args.host_count else "stays on the device",
                   "bwd_wave_iterations": bwd_wave_iters, "wave_iterations": wave_iters,
                   "wave_iterations_skipped_by_bounds": wave_skipped, "wave_iterations_contributing": wave_hits,
                   "contributing_half_blocks_8x4": half_rows, "contributing_half_blocks_4x8": half_cols, "loss": loss, "setup_s": round(setup_s, 1)},
        "raster_fwd_ms": kernels.get("rasterize_to_pixels_from_world_3dgs_fwd", {}).get("ms"),
        "raster_bwd_ms": round(dom_ms, 4),
        "roofline": roofline, "cpu_baseline": cpu_baseline, "parity_in_bench": parity, "boundary_path": boundary,
        "mcmc": mcmc,
        "copy_probe": {"bytes_moved": 2 * copy_bytes, "GBps": round(copy_gbs, 1),
                       "note": "gsx_debug_copy, 1 GiB read + 1 GiB written: measured streaming bandwidth"},
        "kernels": kernels,
    }
    print(json.dumps(out))


def run_ops_path(args, gsx, sc, viewmat, Kmat, W, H, gt, dev, steps=None, warmup=None):
    """The step of the metric issued the way Trainer::train_step issues it (trainer.cpp:599-875): ATen activations and
    concatenation, the autograd Function around rasterize_from_world_with_sh_fwd / _bwd, clamp / permute, l1_loss +
    fused_ssim, loss.backward(), one adam_step_wrapper launch per group - all in C++ (csrc/host/ops_path.cpp)."""
    import numpy as np
    import torch
    from lichtfeld_studio_amd import _lib
    from lichtfeld_studio_amd.trainer import DEFAULT_LRS
    ext = _lib.torch_ext()
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev)
    lrs = [DEFAULT_LRS[k] for k in ("means", "sh0", "shN", "scaling", "rotation", "opacity")]
    tr = ext.OpsPathTrainer(t(sc.means), t(sc.sh0), t(sc.shN), t(sc.scaling_raw), t(sc.rotation_raw),
                            t(sc.opacity_raw.reshape(-1, 1)), int(sc.sh_degree), lrs, 0.2, False)
    gt3 = gt[0].contiguous()
    views = [viewmat, viewmat.clone()]
    first = None
    for i in range(warmup):
        loss = tr.train_step(i + 1, views[i % 2], Kmat, W, H, gt3)
        if i == 0:
            first = float(loss)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for i in range(steps):
        loss = tr.train_step(warmup + i + 1, views[i % 2], Kmat, W, H, gt3)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t1
    # the same with the reference's loss.item() after backward (trainer.cpp:708): the host waits for the device once
    # per step
    t2 = time.perf_counter()
    for i in range(steps):
        loss = tr.train_step(warmup + steps + i + 1, views[i % 2], Kmat, W, H, gt3)
        last = float(loss)
    torch.cuda.synchronize()
    elapsed_item = time.perf_counter() - t2
    return {"it_per_s": round(steps / elapsed, 3), "ms_per_step": round(1e3 * elapsed / steps, 4),
            "it_per_s_with_loss_item": round(steps / elapsed_item, 3), "first_loss": first, "last_loss": last,
            "what": "OpsPathTrainer.train_step: rasterize_from_world_with_sh_fwd/_bwd under autograd, ATen "
                    "activations / cat / clamp / permute / l1_loss, fused_ssim, six adam_step_wrapper launches"}


def run_cpp_step(args, gsx, sc, viewmat, Kmat, W, H, gt, dev, steps=None, warmup=None):
    """gsx::TrainStep (csrc/host/train_step.cpp): the step of the metric over the fused entry points, driven from
    C++ - the launches of the default workload without the interpreter between them."""
    import numpy as np
    import torch
    from lichtfeld_studio_amd import _lib
    from lichtfeld_studio_amd.trainer import DEFAULT_LRS
    ext = _lib.torch_ext()
    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev)
    lrs = [DEFAULT_LRS[k] for k in ("means", "sh0", "shN", "scaling", "rotation", "opacity")]
    cs = ext.TrainStep(t(sc.means), t(np.concatenate([sc.sh0, sc.shN], 1)), t(sc.scaling_raw), t(sc.rotation_raw),
                       t(sc.opacity_raw.reshape(-1)), lrs, sh_degree=int(sc.sh_degree))
    views = [viewmat, viewmat.clone()]
    cs.steps(views, Kmat, W, H, gt, 1)
    first = [float(x) for x in cs.loss_out.cpu()]
    if warmup > 1:
        cs.steps(views, Kmat, W, H, gt, warmup - 1)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    cs.steps(views, Kmat, W, H, gt, steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t1
    assert cs.lists_error() == (0, 0) and cs.steps_held == 0
    return {"it_per_s": round(steps / elapsed, 3), "ms_per_step": round(1e3 * elapsed / steps, 4),
            "first_loss": first, "n_isects": int(cs.n_isects()),
            "what": "gsx::TrainStep::step called from a C++ loop: the 17 launches of the default workload"}


def run_fastgs(args, gsx, sc, cam, dev):
    """forward_wrapper + backward_wrapper of the fastgs backend on the scene of the metric: a secondary line"""
    import numpy as np
    import torch
    from lichtfeld_studio_amd import fastgs
    W, H = cam.width, cam.height
    V = cam.viewmat.astype(np.float32)
    cam_pos = (-V[:3, :3].T @ V[:3, 3]).astype(np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev)
    D = dict(means=t(sc.means), scales_raw=t(sc.scaling_raw), rotations_raw=t(sc.rotation_raw),
             opacities_raw=t(sc.opacity_raw.reshape(-1, 1)), sh0=t(sc.sh0), shN=t(sc.shN))
    bases = (sc.sh_degree + 1) ** 2
    scal = (bases, W, H, float(cam.K[0, 0]), float(cam.K[1, 1]), float(cam.K[0, 2]), float(cam.K[1, 2]), 0.01, 1e10)
    g = torch.Generator(device=dev).manual_seed(1)
    g_img = torch.randn((3, H, W), generator=g, device=dev)
    g_a = torch.randn((1, H, W), generator=g, device=dev)

    def step():
        out = fastgs.forward_wrapper(D["means"], D["scales_raw"], D["rotations_raw"], D["opacities_raw"], D["sh0"],
                                     D["shN"], V, cam_pos, *scal)
        fastgs.backward_wrapper(None, g_img, g_a, out[0], out[1], D["means"], D["scales_raw"], D["rotations_raw"],
                                D["shN"], out[2], out[3], out[4], out[5], V, cam_pos, *scal, *out[6:11])
        return out

    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t1
    print(json.dumps({
        "metric": "fastgs rasterization forward + backward it/s (secondary; not the BASELINE metric)",
        "value": round(args.steps / elapsed, 3), "unit": "it/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(1e3 * elapsed / args.steps, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"fastgs forward_wrapper + backward_wrapper, {sc.means.shape[0]} Gaussians SH degree "
                               f"{sc.sh_degree}, {W}x{H}", "n_instances": out[7]}}))


def run_cpu_baseline(gsx, sc, cam, gt_chw, use_ssim, threads):
    """The CPU checker (a port of the reference kernels; the reference itself has no CPU path) on the host cores:
    one full step - forward, loss, backward, Adam - of the same workload."""
    import numpy as np
    from oracle import oracle as orc
    from oracle.step import OracleTrainStep
    if threads > 0:
        orc.set_num_threads(threads)
    cores = orc.num_threads()
    st = OracleTrainStep(sc, lambda_dssim=0.2 if use_ssim else 0.0)
    gt = np.ascontiguousarray(gt_chw)
    times, first_loss = [], None
    while len(times) < 6 and sum(times) < 12.0:  # a bounded sample: whole steps, about 10 s of CPU work
        t0 = time.perf_counter()
        st.step(cam.viewmat, cam.K, cam.width, cam.height, gt)
        times.append(time.perf_counter() - t0)
        if first_loss is None:
            first_loss = [round(float(x), 7) for x in st.loss]
    dt = sum(times) / len(times)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": round(1.0 / dt, 5), "unit": "it/s", "cores": cores, "kind": "port",
            "sample": f"{len(times)} consecutive full steps of the same workload ({st.params['means'].shape[0]} "
                      f"Gaussians, {cam.width}x{cam.height}), OpenMP over Gaussians / tiles / image planes; value = "
                      "1 / mean step time",
            "seconds": round(sum(times), 2), "cpu": model, "loss": first_loss}


if __name__ == "__main__":
    main()
