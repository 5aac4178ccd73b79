#!/usr/bin/env python3
"""Benchmark of the rasterize forward+backward path on one MI355X.

One "step" = one view: preprocess -> scan -> key expansion -> radix sort -> tile
ranges -> blend forward, then blend backward -> preprocess backward, with every
input already resident in HBM.  Prints ONE JSON line (see the driver contract):
whole-job ms/view, a roofline object for the dominant kernel and the CPU oracle
timed on this box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, vendor peak

# algorithmic HBM bytes per stage: N gaussians, M (tile, gaussian) pairs, P pixels, T tiles
STAGE_BYTES = {
    # K1 with the SH colours split off (they run on a second stream beside the sort): 44 B read
    # (xyz, quaternion, scale, opacity) + 64 B written (depth, radius, uv, conic/opacity, tile count,
    # cov2d, kept-tile record); the colours read 192 B of SH + xyz + radius and write rgb + clamp mask.
    # Together 108 + 221 B against the fused kernel's 297 B / gaussian.
    "preprocess": lambda N, M, P, T, passes: 108 * N,
    "sh_colors": lambda N, M, P, T, passes: 221 * N,
    # binning, priced at what this factorisation has to move (32-bit keys, 32-bit values), not at the
    # reference's single sort of 64-bit keys, which would flatter these stages:
    # depth order of the N gaussians: histogram reads the keys (4), first pass reads keys and writes
    # keys + indices (12), the other passes read and write both (16 each); D passes (3 for 27-bit depth keys)
    "depth_order": lambda N, M, P, T, passes, D=4: (4 + 12 + (D - 1) * 16) * N,
    "scan": lambda N, M, P, T, passes: (12 + 8) * N,
    # order, offset, kept-tile record, depth key per gaussian; tile key + gaussian index per pair
    "make_keys": lambda N, M, P, T, passes: 28 * N + 8 * M,
    # pair sort on the tile bits: histogram reads the keys, `passes` passes read and write key + value
    "sort": lambda N, M, P, T, passes: (4 + 16 * passes) * M,
    "tile_ranges": lambda N, M, P, T, passes: 4 * M + 12 * T,
    "blend_fwd": lambda N, M, P, T, passes: 40 * M + 20 * P,
    "blend_bwd": lambda N, M, P, T, passes: 76 * M + 36 * P,
    # every gaussian's radius and mark are read (5 B); only gaussians whose record received anything (A of them)
    # are worked on: 64 B of record, 250 B of parameters and SH read, 236 B of gradients written.  With A = N this
    # is, up to the marks, the 522 B x N of a kernel that treats every gaussian alike.
    "preprocess_bwd": lambda N, M, P, T, passes, A=None: 5 * N + (64 + 250 + 236) * (N if A is None else A),
}


def committed_traffic_bytes(stage, config_id):
    """HBM bytes per launch of `stage`'s kernel from the committed rocprofv3 --pmc summary (scaled
    FETCH_SIZE + WRITE_SIZE), or None when no summary for this configuration is committed."""
    kernel = {"preprocess": "preprocess_fwd_kernel", "blend_fwd": "blend_fwd_kernel", "blend_bwd": "blend_bwd_kernel",
              "preprocess_bwd": "preprocess_bwd_kernel", "make_keys": "make_keys_kernel"}.get(stage)
    path = os.path.join(ROOT, "profiles", f"config{config_id}_all_kernels.txt")
    if kernel is None or not os.path.exists(path):
        return None
    for line in open(path):
        f = line.split()
        if len(f) == 5 and f[0] == kernel:
            try:
                return int((float(f[3]) + float(f[4])) * 1e6)
            except ValueError:
                return None
    return None


def committed_whole_view_traffic(config_id):
    """(read bytes, written bytes) of HBM traffic per view, every kernel on the view's path times its launches per
    view, from the "whole view" line of the committed rocprofv3 --pmc summary; None when there is none."""
    path = os.path.join(ROOT, "profiles", f"config{config_id}_all_kernels.txt")
    if not os.path.exists(path):
        return None
    for line in open(path):
        f = line.split()
        if line.startswith("whole view:") and "read_MB" in f and "write_MB" in f:
            try:
                return int(float(f[f.index("read_MB") + 1]) * 1e6), int(float(f[f.index("write_MB") + 1]) * 1e6)
            except (ValueError, IndexError):
                return None
    return None


def committed_valu_instructions(stage, config_id):
    """Vector-ALU wave instructions per launch of `stage`'s kernel from the committed rocprofv3 --pmc summary
    (SQ_INSTS_VALU), or None when none is committed for this configuration."""
    kernel = {"blend_fwd": "blend_fwd_kernel", "blend_bwd": "blend_bwd_kernel", "preprocess": "preprocess_fwd_kernel",
              "preprocess_bwd": "preprocess_bwd_kernel", "make_keys": "make_keys_kernel"}.get(stage)
    path = os.path.join(ROOT, "profiles", f"config{config_id}_blend_valu_issue.txt")
    if kernel is None or not os.path.exists(path):
        return None
    for line in open(path):
        f = line.split()
        if len(f) == 10 and f[0] == kernel:
            try:
                return float(f[2])
            except ValueError:
                return None
    return None


def hbm_copy_probe(torch, nbytes=1 << 30, reps=10):
    """GB/s (bytes read + bytes written) of a 1 GiB device-to-device copy, HIP events, best of `reps`."""
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty_like(src)
    src.zero_()
    dst.copy_(src)
    best = float("inf")
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        dst.copy_(src)
        b.record()
        b.synchronize()
        best = min(best, a.elapsed_time(b))
    return round(2 * nbytes / (best * 1e-3) / 1e9, 1)


def orbit_cameras(scene, count, seed=77):
    """`count` poses on an orbit about the world origin: the configuration's camera turned about the vertical axis
    by a seeded angle within +-25 degrees and moved to 0.85 .. 1.15 of its distance, always looking at the origin.
    Configurations whose camera sits at the origin turn in place."""
    import numpy as np
    from d3gs_research_amd.camera import BasicPinholeCamera
    rng = np.random.default_rng(seed)
    base = np.asarray(scene.to_world, np.float64)
    cams = []
    for _ in range(count):
        ang = np.deg2rad(rng.uniform(-25.0, 25.0))
        dist = rng.uniform(0.85, 1.15)
        c, s_ = np.cos(ang), np.sin(ang)
        rot = np.array([[c, 0.0, s_], [0.0, 1.0, 0.0], [-s_, 0.0, c]])
        tw = np.eye(4)
        tw[:3, :3] = rot @ base[:3, :3]
        tw[:3, 3] = rot @ (base[:3, 3] * dist)
        cams.append(BasicPinholeCamera.from_params(scene.fx, scene.fy, scene.cx, scene.cy, scene.width, scene.height, tw))
    return cams


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration id (2 = headline 1M @1080p)")
    ap.add_argument("--filter", type=str, default="OBB_DFVT", help="early_filter_algo: NONE, AABB, ELLIPSE, OBB, OBB_DFVT")
    ap.add_argument("--views", type=int, default=1,
                    help="number of distinct camera poses the steps cycle through (1 = the configuration's own view every "
                         "step, the headline; K > 1 orbits K seeded poses about the scene so that the pair count changes "
                         "from step to step, as in a training loop with a new camera every step)")
    ap.add_argument("--backward-algo", type=str, default="DEFAULT",
                    help="rasterize_backward_algo: DEFAULT (lanes = pixels, wave reduction) or PER_GAUSSIAN (lanes = "
                         "gaussians over the forward's bucket snapshots); the headline is DEFAULT")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--late-gradient-clear", action="store_true",
                    help="let the preprocess backward write the zero gradients itself instead of clearing the arrays "
                         "beside the forward pass (for comparison)")
    ap.add_argument("--op-set", action="append", default=[], metavar="ATTR=0|1",
                    help="set a boolean switch of the operator for an A/B run, e.g. "
                         "overlap_sh_colors=0, poll_pair_count=0, fused_binning=0 (repeatable); the headline runs with the defaults")
    ap.add_argument("--custom-features", type=int, default=0, metavar="F",
                    help="carry F seeded custom feature channels per gaussian through every view, forward and backward "
                         "(a different workload, for profiling the feature kernels: not the headline; no CPU baseline)")
    ap.add_argument("--gaussians", type=int, default=0, help="override the configuration's gaussian count (not the headline)")
    ap.add_argument("--image", type=str, default="", metavar="WxH", help="override the configuration's image size (not the headline)")
    ap.add_argument("--cpu-n", type=int, default=0, help="gaussians in the CPU-baseline sample (0 = full workload)")
    ap.add_argument("--pmc-calibrate", action="store_true",
                    help="only run a plain 256 MiB -> 256 MiB elementwise copy 5 times (reference reading for "
                         "FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the rasterize path is single-device); --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    if args.pmc_calibrate:
        x = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0")
        y = torch.empty_like(x)
        for _ in range(5):
            torch.mul(x, 1.0, out=y)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch.mul(x, 1.0, out=y)", "read_bytes": x.numel() * 4,
                          "write_bytes": y.numel() * 4, "launches": 5}))
        return
    from d3gs_research_amd.config_def import EarlyFilterAlgo, RasterizeBackwardAlgo
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    from d3gs_research_amd.synthetic import gen_scene, scene_config, scene_model

    filt = EarlyFilterAlgo[args.filter]
    resized = bool(args.gaussians or args.image)
    scene = gen_scene(args.config, n=args.gaussians or None,
                      wh=tuple(int(v) for v in args.image.lower().split("x")) if args.image else None)
    cam = scene.camera()
    cams = [cam] + orbit_cameras(scene, args.views - 1)
    op = GaussianSplatOp(scene_config(scene, filt, rasterize_backward_algo=RasterizeBackwardAlgo[args.backward_algo]))
    op.clear_gradients_early = not args.late_gradient_clear
    for item in args.op_set:
        name, _, value = item.partition("=")
        assert hasattr(op, name) and isinstance(getattr(op, name), bool), f"--op-set: the operator has no switch {name!r}"
        setattr(op, name, bool(int(value)))
    model = scene_model(scene, "cuda:0")
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=torch.from_numpy(scene.dT).cuda())

    feat = None
    if args.custom_features > 0:
        gen = torch.Generator(device="cuda:0").manual_seed(5)
        feat = torch.randn((scene.n, args.custom_features), device="cuda:0", generator=gen)
        grads.dcustom_features = torch.randn((1, scene.height, scene.width, args.custom_features), device="cuda:0",
                                             generator=gen)
        args.no_cpu_baseline = True

    pair_counts = []

    def step(i=0):
        c = cams[i % len(cams)]
        out, ctx = op.forward(model, c, training=True, custom_features=feat)
        pair_counts.append(op.last_num_rendered)
        if ctx is None:      # nothing of the scene in this view
            return out, None
        gm, duv, _ = op.backward(model, c, ctx, out, grads, return_uv_grad=True)
        return out, gm

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    del pair_counts[:]
    rebins_before = op.rebin_count
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    views_info = {"poses": len(cams), "pairs_min": int(min(pair_counts)), "pairs_max": int(max(pair_counts)),
                  # views whose pair count outgrew the buffers sized from the previous view and were binned again
                  "rebinned_views": int(op.rebin_count - rebins_before)}
    # a second, short timed loop over eight orbit poses (extra keys; the headline stays the configuration's own
    # view): the pair count changes from view to view, the pair buffers are sized from the previous view's count and
    # a view that outgrows them is binned again
    views8 = None
    if args.views == 1 and feat is None:
        cams8 = [cam] + orbit_cameras(scene, 7)
        counts8 = []

        def step8(i):
            c = cams8[i % 8]
            out, ctx = op.forward(model, c, training=True)
            counts8.append(op.last_num_rendered)
            if ctx is not None:
                op.backward(model, c, ctx, out, grads, return_uv_grad=True)

        for i in range(8):
            step8(i)
        torch.cuda.synchronize()
        del counts8[:]
        rebins8 = op.rebin_count
        steps8 = 16
        t0 = time.perf_counter()
        for i in range(steps8):
            step8(i)
        torch.cuda.synchronize()
        views8 = {"ms_per_view": round((time.perf_counter() - t0) * 1e3 / steps8, 4), "steps": steps8, "poses": 8,
                  "pairs_min": int(min(counts8)), "pairs_max": int(max(counts8)),
                  "rebinned_views": int(op.rebin_count - rebins8)}
    step(0)                  # the stage pass and the figures below are of the configuration's own view
    torch.cuda.synchronize()

    # per-stage durations from a second, untimed-as-a-whole run of the same views: with stage timers on, the
    # operator issues the binning launch by launch (HIP events around every stage) instead of as one library call
    # (a few views first without keeping their timings: issued stage by stage the operator allocates its buffers
    # in a different pattern, and the first view of that pattern can stall on the allocator inside a stage)
    op.stage_events = {}
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    op.stage_events = {}
    for _ in range(min(args.steps, 20)):
        step()
    torch.cuda.synchronize()

    N, P_px, T_tiles = scene.n, scene.width * scene.height, ((scene.width + 15) // 16) * ((scene.height + 15) // 16)
    M = op.last_num_rendered
    radix_passes = lambda bits: min((bits + 7) // 8, (bits + 8) // 9)     # 8-bit digits, 9-bit where that saves a pass
    passes = radix_passes(int(T_tiles).bit_length())      # the pair sort (tile bits only)
    from d3gs_research_amd import _capi
    import ctypes
    depth_passes = radix_passes(_capi.lib().d3gs_depth_key_bits(ctypes.byref(op.make_params(model, cam, True))))
    # gaussians whose gradient record is not all zero after the last view's blend backward
    active = int((op.last_raster_grads.records != 0).any(dim=1).sum())
    stages = {}
    for name, evs in op.stage_events.items():
        ts = sorted(a.elapsed_time(b) for a, b in evs)
        # a host stall between two launches of a stage (allocator, scheduler) shows up as one sample many times
        # the median: such samples are left out of the average and counted
        kept = [t for t in ts if t <= 5.0 * ts[len(ts) // 2]]
        avg = sum(kept) / len(kept)
        extra = {"preprocess_bwd": (active,), "depth_order": (depth_passes,)}.get(name, ())
        nbytes = STAGE_BYTES[name](N, M, P_px, T_tiles, passes, *extra)
        stages[name] = {"ms": round(avg, 4), "ms_p10": round(ts[len(ts) // 10], 4), "ms_p50": round(ts[len(ts) // 2], 4),
                        "ms_p90": round(ts[(len(ts) * 9) // 10], 4), "stalled_samples_left_out": len(ts) - len(kept),
                        "alg_bytes": int(nbytes),
                        "gbs": round(nbytes / (avg * 1e-3) / 1e9, 1)}
    op.stage_events = None
    if "sh_colors" in stages:
        stages["sh_colors"]["overlapped"] = True     # runs on a second stream beside depth_order .. sort
    gpu_sum = sum(s["ms"] for s in stages.values() if not s.get("overlapped"))
    dom = max(stages, key=lambda k: stages[k]["ms"])
    achieved = stages[dom]["gbs"]
    copy_gbs = hbm_copy_probe(torch)
    # "bound": what the counters say limits the dominant kernel.  The two blend kernels retire vector instructions
    # at the rate their mix allows for their whole duration (roofline.valu below) while moving a fraction of a byte
    # per evaluated pair, so they are "valu"; the HBM fraction asked for is reported all the same.
    roofline = {"bound": "valu" if dom in ("blend_fwd", "blend_bwd", "preprocess") else "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 5), "traffic": None if resized else committed_traffic_bytes(dom, args.config),
                "traffic_source": f"profiles/config{args.config}_all_kernels.txt (rocprofv3 --pmc, not this run)",
                "pair_evals_per_s": round(256.0 * M / (stages[dom]["ms"] * 1e-3), 1),
                # what a plain device-to-device copy reaches on this box (read + written bytes per second)
                "measured_copy_gbs": copy_gbs, "frac_of_measured_copy": round(achieved / copy_gbs, 5)}
    # The blend kernels are bound by vector-instruction issue, not by HBM: next to the HBM fraction asked for, the
    # rate at which the dominant kernel retires vector instructions (count from the committed counter summary, time
    # from this run) against 256 CUs x 4 SIMDs x 2.4 GHz / 4 cycles per wave64 instruction.  Plain FP32 operations
    # issue in half that time on this chip, so the ratio can exceed 1; its ceiling for this kernel's mix is about 1.3.
    valu = None if resized else committed_valu_instructions(dom, args.config)
    if valu is not None:
        rate = valu / (stages[dom]["ms"] * 1e-3)
        roofline["valu"] = {"wave_instructions_per_launch": valu, "per_s": round(rate, 1),
                            "vs_4_cycle_issue": round(rate / (256 * 4 * 2.4e9 / 4), 3)}
    # The whole view against the HBM roofline: measured traffic of every kernel on the path (committed counter
    # summary) over this run's time per view.
    hbm_whole_view = None
    whole = None if resized else committed_whole_view_traffic(args.config)
    if whole is not None and filt.name == "OBB_DFVT" and args.backward_algo == "DEFAULT":
        gbs = (whole[0] + whole[1]) / (ms_per_step * 1e-3) / 1e9
        hbm_whole_view = {"read_bytes": whole[0], "written_bytes": whole[1], "traffic_bytes": whole[0] + whole[1],
                          "gbs": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                          "frac_of_measured_copy": round(gbs / copy_gbs, 4),
                          "source": f"profiles/config{args.config}_all_kernels.txt"}
    # tile list lengths of the last view (the blend kernels' work is their sum and their skew)
    _, last_ctx = op.forward(model, cam, training=True)
    lens = (last_ctx.workload_ranges[:, 1] - last_ctx.workload_ranges[:, 0]).to(torch.float64)
    tile_lists = {"mean": round(float(lens.mean()), 1), "median": float(lens.median()), "max": int(lens.max())}

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import d3gs_oracle as O
        O.build()
        cs = scene if args.cpu_n in (0, scene.n) else gen_scene(args.config, n=args.cpu_n)
        Pc = O.params_for_scene(cs, int(filt))
        # repeat whole views until ~10 s of CPU work has been spent (at most 12 views); report the median
        fwd_ms, bwd_ms = [], []
        t_start = time.perf_counter()
        while len(fwd_ms) < 12 and (time.perf_counter() - t_start < 10.0 or len(fwd_ms) < 3):
            c0 = time.perf_counter()
            ref = O.forward(Pc, cs.xyz, cs.quaternion_xyzw, cs.scale, cs.opacity, cs.color_sh)
            c1 = time.perf_counter()
            O.backward(Pc, ref, cs.xyz, cs.quaternion_xyzw, cs.scale, cs.opacity, cs.color_sh, cs.drgb[0], cs.dT[0])
            c2 = time.perf_counter()
            fwd_ms.append((c1 - c0) * 1e3)
            bwd_ms.append((c2 - c1) * 1e3)
        med = lambda v: sorted(v)[len(v) // 2]
        spent = time.perf_counter() - t_start
        # one view on a single thread as well (the scalar figure), if the threaded one says it fits in ~20 s
        threads, single = O.num_threads(), None
        if (med(fwd_ms) + med(bwd_ms)) * threads < 20e3:
            O.set_num_threads(1)
            c0 = time.perf_counter()
            ref1 = O.forward(Pc, cs.xyz, cs.quaternion_xyzw, cs.scale, cs.opacity, cs.color_sh)
            O.backward(Pc, ref1, cs.xyz, cs.quaternion_xyzw, cs.scale, cs.opacity, cs.color_sh, cs.drgb[0], cs.dT[0])
            single = round((time.perf_counter() - c0) * 1e3, 1)
            O.set_num_threads(threads)
        cpu_baseline = {"value": round(med(fwd_ms) + med(bwd_ms), 1), "unit": "ms/view", "cores": threads,
                        "kind": "port", "fwd_ms": round(med(fwd_ms), 1), "bwd_ms": round(med(bwd_ms), 1),
                        "single_thread_ms": single, "cpu": cpu_model_name(), "host_cpus": os.cpu_count(),
                        "sample": f"{len(fwd_ms)} views of config {args.config} with {cs.n} gaussians "
                                  f"({'full workload' if cs.n == scene.n else 'reduced gaussian count'}), "
                                  f"M={ref['num_rendered']}, median, OpenMP over {O.num_threads()} threads, "
                                  f"{spent:.1f} s of CPU work"
                                  + ("" if single is None else "; single_thread_ms: one view on one thread")}

    line = {
        "metric": "fwd+bwd raster ms/view, 1M Gaussians @1080p, 1 MI355X" if (args.config == 2 and not resized)
        else f"fwd+bwd raster ms/view, config {args.config}" + (" with another gaussian count or image size" if resized else ""),
        **({"note": f"with {args.custom_features} custom feature channels: not the headline workload"} if feat is not None else {}),
        "value": round(ms_per_step, 4), "unit": "ms/view", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"config {args.config}: {scene.name}", "gaussians": N, "sh_degree": scene.sh_degree,
                   "image": f"{scene.width}x{scene.height}", "early_filter_algo": filt.name,
                   "rasterize_backward_algo": args.backward_algo, "pairs_M": int(M),
                   "pairs_per_gaussian": round(M / N, 3), "tiles": T_tiles, "tile_list_length": tile_lists,
                   "gaussians_with_gradient": active, "views": views_info,
                   **({"op_set": args.op_set} if args.op_set else {}),
                   **({"custom_features": args.custom_features} if feat is not None else {})},
        "gaussians_per_s": round(N / (ms_per_step * 1e-3), 1),
        "gpu_stage_sum_ms": round(gpu_sum, 4),
        "stages": stages,
        # (the stage pass issues the binning launch by launch, with 32-bit pair keys; the timed views go through the
        # one-call binning, whose pair keys are 16-bit tile ids when the view has at most 2^16 tiles)
        "stages_note": "stage timers on: binning launch by launch, 32-bit pair keys; timed views: one library call, "
                       + ("16" if (op.narrow_tile_keys and T_tiles <= 65536) else "32") + "-bit pair keys",
        "roofline": roofline,
        "hbm_whole_view": hbm_whole_view,
        "views8": views8,
        "cpu_baseline": cpu_baseline,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
