#!/usr/bin/env python3
"""Headline benchmark: 1080p frames/s of the 3DGS forward render at 6M Gaussians
on one MI355X (synthetic city-block scene, SH degree 3, RGB + depth + alpha).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--gaussians P]

A step is one full frame through GaussianRasterizer.forward (the product path:
preprocess -> tile count -> tile scatter -> per-tile sort -> blend) with every
input already resident in HBM.  Prints ONE JSON line with the frame rate, a
per-stage breakdown timed with HIP events on the launch stream, the roofline
figure of the dominant stage and a CPU baseline measured in the same run on
the host cores: the PyTorch-CPU rasterizer of the same semantics on a bounded
sample of the workload, and the C checker over the whole frame, which also
counts the (pixel, Gaussian) pairs the blend's algorithmic flops are defined by.

--config 4 (20M Gaussians, 3840x2160, 30 poses) and --config 5 (Scaffold-GS,
500k anchors decoded on the matrix cores, then rasterized) print lines of the
same structure for those workloads.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X HBM3E
FP32_PEAK_TFLOPS = 157.3  # MI355X fp32 vector peak (packed FMA); this build issues unpacked FP32 only
MFMA_F16_PEAK_TFLOPS = 2500.0

# HBM bytes per launch of the stages of the default workload (6M Gaussians, 1080p), read from hardware counters in
# separate profiler runs of this script, NOT measured by the run that prints them: two `rocprofv3 --pmc` runs
# (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what the same counter reads for the 1 GiB copy of
# --calibration-copy.  The bench line names the file they were read from; tests/test_bench_constants.py holds these
# numbers to that file.  "keys_sort_ranges" is the sum over the kernels of the tile count, scatter and sort stages.
COUNTER_TRAFFIC = {
    "source": "profiles/bench_c3_6M_1080p_hbm_traffic.txt",
    "workload": "configs[2]",
    "bytes": {"blend": 1844.2e6, "preprocess": 1705.8e6, "keys_sort_ranges": 824.4e6},
    # fp32 flops the blend kernel issues per launch (64 lanes x (2 FMA + MUL + ADD) wavefront instructions), from
    # profiles/bench_c3_6M_1080p_valu_counters.txt
    "blend_issued_flops": 10.31e9,
    "blend_issued_flops_source": "profiles/bench_c3_6M_1080p_valu_counters.txt",
    "blend_valu_busy": 0.957,
}

# Same for `--config 5`: HBM bytes per launch of the two decode kernels (count + emit)
COUNTER_TRAFFIC_C5 = {
    "source": "profiles/bench_c5_scaffold_500k_hbm_traffic.txt",
    "workload": "configs[4]",
    "bytes": {"decode": 250.6e6},
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3, choices=[1, 2, 3, 4, 5],
                    help="3 = the headline workload; 4 = 20M Gaussians, 4K, 30 poses; 5 = Scaffold-GS, 500k anchors")
    ap.add_argument("--gaussians", type=int, default=None, help="override the Gaussian / anchor count (not the named workload)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--stage-steps", type=int, default=20)
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--no-model-level", action="store_true",
                    help="skip the model-level variants (their launches of the same kernels on other inputs would "
                         "mix into the per-kernel averages of a profiler run)")
    ap.add_argument("--no-backward", action="store_true", help="skip the backward-pass timing")
    ap.add_argument("--spatial-order", action="store_true",
                    help="store the scene along a Morton curve first (the checkpoint loaders' spatial_order option); "
                         "same Gaussians, coherent memory traffic; not the headline workload")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="default workload only: leave out the compact lines of configs[1], [3] and [4] "
                         "(`other_configs`), e.g. for a profiler run")
    ap.add_argument("--two-in-flight", action="store_true",
                    help="also time the frames with two in flight on alternating streams (reported beside `value`)")
    return ap.parse_args()


def settings_for(scene, device, cam=None, sh_degree=None):
    from landmarksystem_amd import GaussianRasterizationSettings

    cam = (cam or scene.camera).to(device)
    return GaussianRasterizationSettings(
        image_height=cam.height, image_width=cam.width, tanfovx=math.tan(cam.FovX * 0.5),
        tanfovy=math.tan(cam.FovY * 0.5), bg=scene.bg.to(device), scale_modifier=1.0,
        viewmatrix=cam.world_view_transform, projmatrix=cam.full_proj_transform,
        sh_degree=scene.sh_degree if sh_degree is None else sh_degree,
        campos=cam.camera_center, prefiltered=False, debug=False,
    )


# ----------------------------------------------------------------------------------------------------------------
# GPU side: stage timings and algorithmic work of one rasterizer frame

def time_stages(torch, pipeline, inp, out, ws, n_cap, stages, steps):
    for _, m in stages:  # warm
        pipeline.run_stages(inp, out, ws, n_cap, m)
    torch.cuda.synchronize()
    acc = {n: 0.0 for n, _ in stages}
    for _ in range(steps):
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(len(stages) + 1)]
        evs[0].record()
        for k, (_, m) in enumerate(stages):
            pipeline.run_stages(inp, out, ws, n_cap, m)
            evs[k + 1].record()
        torch.cuda.synchronize()
        for k, (n, _) in enumerate(stages):
            acc[n] += evs[k].elapsed_time(evs[k + 1])
    return {n: acc[n] / steps for n in acc}


def stage_breakdown(torch, pipeline, _lib, inp, n_cap, steps):
    """Average milliseconds per stage, HIP events on the launch stream (torch's current stream, the one every
    kernel of the library is enqueued on): the shipped pipeline (tile-bucketed sort) and, beside it, the classic
    duplicate / LSD radix sort / ranges stages it replaces."""
    ws = pipeline.Workspace(inp.device)
    out = pipeline.FrameOutputs(inp)
    # like render() on a steady stream of frames, the sort stage leaves out the launches of the sorter size classes
    # that this frame leaves empty (a hint to the library, read from the header the tile-count stage writes)
    lay = pipeline.run_stages(inp, out, ws, n_cap, _lib.STAGE_PREPROCESS | _lib.STAGE_TILE_COUNT)
    torch.cuda.synchronize()
    words = [int(w) for w in ws.view(lay, "header", inp.P, 0, inp.tiles)[:4].tolist()]
    class_counts = ((words[2] >> 32) & 0xFFFFFFFF, words[3] & 0xFFFFFFFF, (words[3] >> 32) & 0xFFFFFFFF)
    skip = sum(m for m, c in zip(_lib.STAGE_TILESORT_SKIP, class_counts) if c == 0)
    fast = [("preprocess", _lib.STAGE_PREPROCESS), ("tile_count", _lib.STAGE_TILE_COUNT),
            ("tile_scatter", _lib.STAGE_TILE_SCATTER), ("tile_sort", _lib.STAGE_TILESORT | skip),
            ("blend", _lib.STAGE_BLEND)]
    classic = [("scan", _lib.STAGE_SCAN), ("duplicate", _lib.STAGE_DUPLICATE), ("sort", _lib.STAGE_SORT),
               ("ranges", _lib.STAGE_RANGES)]
    ms = time_stages(torch, pipeline, inp, out, ws, n_cap, fast, steps)
    ms.update(time_stages(torch, pipeline, inp, out, ws, n_cap, classic, max(3, steps // 4)))
    lay = _lib.workspace_layout(inp.P, n_cap, inp.width, inp.height)
    hdr = ws.view(lay, "header", inp.P, 0, inp.tiles).cpu()
    ranges = ws.view(lay, "ranges", inp.P, 0, inp.tiles).cpu().numpy().view("uint32")
    stats = {"num_keys": int(hdr[0]), "num_visible": int(hdr[2]) & 0xFFFFFFFF,
             "range_sum": int((ranges[:, 1].astype("int64") - ranges[:, 0]).sum()), "sort_passes": int(lay.sort_passes),
             "sort_class_buckets": list(class_counts)}
    return ms, stats


def algorithmic_work(P, V, N, tiles, npix, colour_bytes, passes):
    """Algorithmic bytes per frame and stage.  `colour_bytes`: bytes of colour input per Gaussian (12 x SH
    coefficients, or 12 for precomputed colours)."""
    b_in = 12 + 12 + 16 + 4 + colour_bytes  # mean, scale, quat, opacity, colour input
    return {
        "preprocess": 12 * P + 8 * P + V * (b_in - 12) + V * 40,
        "scan": 8 * P,
        "duplicate": V * 20 + 12 * N,
        "sort": N * (8 + passes * 24),
        "ranges": 8 * N + 8 * tiles,
        "blend_bytes": 40 * N + 20 * npix,
    }


def raster_report(stage_ms, stats, P, tiles, npix, colour_bytes, pairs, counters):
    """The `stages` object and the roofline of the dominant stage for one rasterizer frame.

    pairs:    {"evaluated", "accepted", "tile_work"} counted by the C checker in this run, or None (then the blend
              is priced with the kernel-independent upper bound 256 x sum of tile range lengths, labelled as such).
    counters: COUNTER_TRAFFIC when it applies to this workload, else None."""
    V, N = stats["num_visible"], stats["num_keys"]
    work = algorithmic_work(P, V, N, tiles, npix, colour_bytes, stats["sort_passes"])
    cbytes = counters["bytes"] if counters else {}

    def hbm(ms, nbytes, counter_bytes=None):
        d = {"ms": round(ms, 4), "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
             "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
        if counter_bytes:
            d.update({"counter_bytes": counter_bytes, "counter_GBps": round(counter_bytes / ms / 1e6, 1),
                      "frac_hbm_counter": round(counter_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)})
        return d

    stages = {"preprocess": hbm(stage_ms["preprocess"], work["preprocess"], cbytes.get("preprocess"))}
    # key generation + sort + ranges.  "bytes" is the algorithmic figure of the stages this path replaces (scan,
    # duplicate, 8-bit LSD radix sort, ranges): an equivalent-work number, not traffic of the shipped kernels, which
    # never run those passes.  counter_bytes / frac_hbm_counter (where present) are what the kernels really moved.
    sort_bytes = work["scan"] + work["duplicate"] + work["sort"] + work["ranges"]
    sort_ms = stage_ms["tile_count"] + stage_ms["tile_scatter"] + stage_ms["tile_sort"]
    for name in ("tile_count", "tile_scatter", "tile_sort"):
        stages[name] = {"ms": round(stage_ms[name], 4)}
    stages["keys_sort_ranges"] = hbm(sort_ms, sort_bytes, cbytes.get("keys_sort_ranges"))
    stages["keys_sort_ranges"]["accounting"] = ("bytes = scan + duplicate + LSD radix sort (%d passes of 24 B/key) + ranges"
                                                " that the tile-bucketed stages replace; floor_bytes = 24 B/key"
                                                % stats["sort_passes"])
    stages["keys_sort_ranges"]["floor_bytes"] = 24 * N
    stages["keys_sort_ranges"]["frac_hbm_floor"] = round(24 * N / sort_ms / 1e6 / HBM_PEAK_GBS, 4) if N else 0.0
    stages["classic_lsd_path"] = {"scan_ms": round(stage_ms["scan"], 4), "duplicate_ms": round(stage_ms["duplicate"], 4),
                                  "sort_ms": round(stage_ms["sort"], 4), "ranges_ms": round(stage_ms["ranges"], 4),
                                  "sort_GBps": round(work["sort"] / stage_ms["sort"] / 1e6, 1),
                                  "sort_frac_hbm": round(work["sort"] / stage_ms["sort"] / 1e6 / HBM_PEAK_GBS, 4)}
    ms = stage_ms["blend"]
    upper = 25 * 256 * stats["range_sum"]
    blend = {"ms": round(ms, 4), "flops_upper": upper, "TFLOPs_upper": round(upper / ms / 1e9, 2),
             "frac_fp32_upper": round(upper / ms / 1e9 / FP32_PEAK_TFLOPS, 4)}
    if pairs:
        flops = 25 * pairs["evaluated"]
        blend.update({
            "pairs_evaluated": pairs["evaluated"], "pairs_accepted": pairs["accepted"], "tile_work": pairs["tile_work"],
            "pairs_source": "C checker (oracle/gs_oracle.c) over the whole frame, in this run",
            "flops_algorithmic": flops, "TFLOPs_algorithmic": round(flops / ms / 1e9, 2),
            "frac_fp32_algorithmic": round(flops / ms / 1e9 / FP32_PEAK_TFLOPS, 4),
            "TFLOPs_tile_work": round(25 * pairs["tile_work"] / ms / 1e9, 2),
            "accepted_pairs_per_s": round(pairs["accepted"] / ms * 1e3)})
    if counters:
        blend.update({"TFLOPs_issued": round(counters["blend_issued_flops"] / ms / 1e9, 2),
                      "frac_fp32_issued": round(counters["blend_issued_flops"] / ms / 1e9 / FP32_PEAK_TFLOPS, 4),
                      "issued_flops_source": counters["blend_issued_flops_source"]})
    stages["blend"] = blend
    pre_sort_ms = stage_ms["preprocess"] + sort_ms
    counter_sum = cbytes.get("preprocess", 0) + cbytes.get("keys_sort_ranges", 0) if counters else None
    stages["preprocess_plus_sort"] = hbm(pre_sort_ms, work["preprocess"] + sort_bytes, counter_sum)
    stages["rates"] = {"gaussians_per_s_preprocess": round(P / stage_ms["preprocess"] * 1e3),
                       "sorted_keys_per_s": round(N / sort_ms * 1e3) if N else 0,
                       "blend_frames_per_s": round(1e3 / stage_ms["blend"], 1)}

    # the dominant KERNEL: preprocess and blend are one kernel each; count / scatter / sort are groups of several
    # kernels, none of which comes near either (their sum is reported as stages.keys_sort_ranges)
    shipped = {"preprocess": stage_ms["preprocess"], "blend": stage_ms["blend"]}
    dominant = max(shipped, key=lambda n: shipped[n])
    # HBM bytes per launch of that kernel, from the committed counter runs (a number quoted from the named file,
    # not an observation of this run)
    traffic = cbytes[dominant] if counters and dominant in cbytes else None
    traffic_source = (counters["source"] + " (rocprofv3 FETCH_SIZE + WRITE_SIZE of an earlier run of this workload)"
                      if traffic else None)
    if dominant == "blend":
        kind = "algorithmic" if pairs else "upper"
        work_rate = {"TFLOPs": blend["TFLOPs_" + kind], "of_peak": blend["frac_fp32_" + kind],
                     "definition": "25 flop x the (pixel, Gaussian) pairs of the reference's per-pixel loop" + (
                         " (counted by the C checker in this run)" if pairs else
                         " (upper bound: 256 x the sum of the tile range lengths)") +
                     " / kernel time: a rate of useful work, NOT a utilisation -- the kernel skips pairs whose alpha is "
                     "provably < 1/255 without evaluating them, so this exceeds 1 on sparse frames"}
        if counters:
            roofline = {"bound": "valu", "kernel": "blend_kernel", "achieved": blend["TFLOPs_issued"],
                        "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": blend["frac_fp32_issued"],
                        "frac_of_unpacked_fp32_peak": round(blend["TFLOPs_issued"] / (FP32_PEAK_TFLOPS / 2), 4),
                        "valu_busy": counters.get("blend_valu_busy"), "traffic": traffic, "traffic_source": traffic_source,
                        "issued_flops_source": counters["blend_issued_flops_source"], "work_rate": work_rate,
                        "note": "achieved = fp32 flops the kernel ISSUED per launch (wavefront FMA / MUL / ADD instructions x "
                                "64 lanes, FMA = 2; hardware counters of an earlier run of this workload, named above) / the "
                                "launch time measured in this run.  peak = MI355X fp32 vector peak with packed FMA (157.3); "
                                "this build issues unpacked fp32 only (packed fp32 is disabled on this pool), whose peak is "
                                "78.6.  valu_busy = share of cycles the vector ALUs were issuing (same counter run): the "
                                "kernel is bound by instruction issue, most of it compares, selects and address arithmetic"}
        else:
            roofline = {"bound": "valu", "kernel": "blend_kernel", "achieved": None, "peak": FP32_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": None, "traffic": None, "work_rate": work_rate,
                        "note": "issued flops need hardware counters, which exist for the default workload only"}
    else:
        roofline = {"bound": "hbm", "kernel": dominant + "_kernel", "achieved": stages[dominant]["GBps"],
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": stages[dominant]["frac_hbm"], "traffic": traffic,
                    "traffic_source": traffic_source}
    return stages, roofline


def backward_report(torch, pipeline, inp, n_cap, N, V, P, sh_coeffs, ms_per_step, stage_steps):
    """Backward pass of the same frame (the training loop's loss.backward() on an image loss): all gradients of a
    forward render, reported beside the forward stages, never part of `value`."""
    dev = inp.device
    ws_b = pipeline.Workspace(dev)
    ws_b.key_capacity = n_cap
    out_b = pipeline.render(inp, ws=ws_b)
    g_image = torch.randn(3, inp.height, inp.width, device=dev)
    t_bwd = {}
    for label, want in (("all_gradients", pipeline.GRAD_NAMES),
                        ("without_sh_gradient", tuple(n for n in pipeline.GRAD_NAMES if n != "shs"))):
        for _ in range(3):
            pipeline.render_backward(inp, out_b, ws_b.buffer, g_image, want=want)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(stage_steps):
            pipeline.render_backward(inp, out_b, ws_b.buffer, g_image, want=want)
        e1.record()
        torch.cuda.synchronize()
        t_bwd[label] = e0.elapsed_time(e1) / stage_steps
    # algorithmic bytes: a 48-B gradient record per key written and read back; per key the sorted
    # value, the 48-B record of its Gaussian, rectangle and first-record index; per visible Gaussian its inputs
    # and record; per Gaussian radius, key count, first-record index and every gradient written
    bwd_bytes = N * (48 + 48 + 4 + 48 + 12) + V * (12 + 12 + 16 + 4 * 3 * sh_coeffs + 48) + \
        P * (12 + 12 + 12 + 4 + 12 + 16 + 4 * 3 * sh_coeffs)
    return {"ms": round(t_bwd["all_gradients"], 4), "ms_without_sh_gradient": round(t_bwd["without_sh_gradient"], 4),
            "bytes": bwd_bytes, "GBps": round(bwd_bytes / t_bwd["all_gradients"] / 1e6, 1),
            "forward_plus_backward_frames_per_s": round(1e3 / (ms_per_step + t_bwd["all_gradients"]), 1)}


# ----------------------------------------------------------------------------------------------------------------
# CPU side (rank 0, N = 1): the checkers timed on the host cores.  Only this leg touches oracle/.

def cpu_pair_stats(scene, cam=None, colors_precomp=None, sh_degree=None, keep_frame=False):
    """The C checker over the whole frame: the (pixel, Gaussian) pair counts that define the blend's algorithmic
    flops, and the checker's own frame time on the host cores.  `keep_frame`: also return everything the checker
    produced (radii, sorted keys and values, ranges, image, depth, alpha) under "frame", for the parity leg."""
    import numpy as np

    from oracle import c_oracle as co
    cam = cam or scene.camera
    fr = co.Frame(cam.width, cam.height, math.tan(cam.FovX * 0.5), math.tan(cam.FovY * 0.5),
                  cam.world_view_transform.cpu().numpy(), cam.full_proj_transform.cpu().numpy(),
                  cam.camera_center.cpu().numpy(), scene.bg.cpu().numpy(), 1.0,
                  scene.sh_degree if sh_degree is None else sh_degree)
    kw = dict(scales=scene.scales.numpy(), rotations=scene.rotations.numpy())
    if colors_precomp is not None:
        kw["colors_precomp"] = np.ascontiguousarray(colors_precomp)
    else:
        kw["shs"] = scene.shs.numpy()
    g = co.Gaussians(scene.means3D.numpy(), scene.opacities.numpy(), **kw)
    threads = co.set_threads(min(os.cpu_count() or 1, 16))
    t0 = time.perf_counter()
    out = co.render(fr, g, keep_intermediates=keep_frame)
    seconds = time.perf_counter() - t0
    return {"evaluated": out["pairs_evaluated"], "accepted": out["pairs_accepted"], "tile_work": out["tile_work"],
            "num_keys": out["num_keys"], "seconds": seconds, "threads": threads, "frame": out if keep_frame else None}


def parity_leg(torch, pipeline, inp, ref):
    """The `parity` object: one frame through the product path (pipeline.render over a workspace of its own) against
    the frame the C checker rendered from the same inputs: radii, key count, every sorted key and value and the
    tile ranges bit for bit; image, depth and alpha as measured errors."""
    import numpy as np

    from oracle import compare
    ws = pipeline.Workspace(inp.device)
    out = pipeline.render(inp, ws=ws)
    torch.cuda.synchronize()
    lay = ws.ensure(inp.P, out.key_capacity, inp.width, inp.height)
    n = out.num_keys
    take = lambda name, kind: ws.view(lay, name, inp.P, n, inp.tiles).cpu().numpy().view(kind)  # noqa: E731
    exact = {"radii": bool(np.array_equal(out.radii.cpu().numpy(), ref["radii"])),
             "num_keys": bool(n == ref["num_keys"])}
    if n == ref["num_keys"]:
        exact["sorted_keys"] = bool(np.array_equal(take("sorted_keys", np.uint64), ref["sorted_keys"]))
        exact["sorted_values"] = bool(np.array_equal(take("sorted_values", np.uint32), ref["sorted_values"]))
        exact["tile_ranges"] = bool(np.array_equal(take("ranges", np.uint32), ref["ranges"]))
    got = dict(image=out.image.cpu().numpy(), depth=out.depth.cpu().numpy(), alpha=out.alpha.cpu().numpy())
    return compare.parity_object(got, ref, exact)


def cpu_baseline(scene, pairs, colors_precomp=None, extra_seconds=0.0, extra_note=""):
    """cpu_baseline object: the PyTorch-CPU rasterizer (bounded sample) with the C checker's whole-frame time beside it."""
    from oracle import torch_oracle

    base = torch_oracle.timed_baseline(scene, colors_precomp=colors_precomp, extra_seconds=extra_seconds,
                                       extra_note=extra_note)
    if pairs:
        base["c_checker"] = {"frames_per_s": round(1.0 / (pairs["seconds"] + extra_seconds), 4), "threads": pairs["threads"],
                             "sample": "oracle/gs_oracle.c, the whole frame (%d keys) in %.2f s" % (pairs["num_keys"],
                                                                                                 pairs["seconds"])}
    return base


def guarded(fn, *a, **kw):
    """The CPU leg is a reported figure, never a reason to lose the GPU numbers."""
    try:
        return fn(*a, **kw), None
    except Exception as exc:  # noqa: BLE001
        return None, repr(exc)


# ----------------------------------------------------------------------------------------------------------------

def frame_loop(torch, rast, kwargs, warmup, steps, settings_list=None):
    """W untimed frames, then exactly K frames bracketed by synchronisation; frames/s and ms per frame."""
    with torch.no_grad():
        for k in range(warmup):
            if settings_list:
                rast.raster_settings = settings_list[k % len(settings_list)]
            rast(**kwargs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(steps):
            if settings_list:
                rast.raster_settings = settings_list[k % len(settings_list)]
            rast(**kwargs)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    return steps / elapsed, elapsed * 1e3 / steps


def synchronised_latency(torch, call, frames):
    """The reference's own protocol: synchronise, forward, synchronise around every frame, the first five frames
    dropped (benchmarks/nerf/origin_gs/gs_evaluator.py:104-114,136), and its spread."""
    per_frame = []
    with torch.no_grad():
        for _ in range(frames + 5):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            call()
            torch.cuda.synchronize()
            per_frame.append((time.perf_counter() - t0) * 1e3)
    per_frame = sorted(per_frame[5:])
    pick = lambda q: round(per_frame[min(len(per_frame) - 1, int(q * len(per_frame)))], 4)  # noqa: E731
    return {"mean_ms": round(sum(per_frame) / len(per_frame), 4), "median_ms": pick(0.5), "p10_ms": pick(0.1),
            "p90_ms": pick(0.9), "frames": len(per_frame), "frames_per_s": round(1e3 * len(per_frame) / sum(per_frame), 2)}


def base_line(metric, fps, ms_per_step, args, warmup, dtype, config):
    return {"metric": metric, "value": round(fps, 2), "unit": "frames/s", "n_gpus": 1, "steps": args.steps,
            "warmup": warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": config}


def bench_vanilla(args, torch, dev):
    """configs[0..2]: one camera, the vanilla rasterizer call of the reference's model.  Returns the bench line."""
    from landmarksystem_amd import GaussianRasterizer, _lib, pipeline, scenes

    t0 = time.time()
    make = scenes.BY_INDEX[args.config]
    scene = make(args.gaussians) if args.gaussians else make()
    gen_s = time.time() - t0
    if args.spatial_order:
        from landmarksystem_amd.models import morton_order
        order = morton_order(scene.means3D)
        scene = scenes.GaussianScene(scene.name + " (Morton order)", scene.means3D[order], scene.scales[order],
                                     scene.rotations[order], scene.opacities[order], scene.shs[order], scene.sh_degree,
                                     scene.cameras, scene.bg)
    d = scene.to(dev)
    rast = GaussianRasterizer(settings_for(scene, dev))
    kwargs = dict(means3D=d.means3D, means2D=None, shs=d.shs, colors_precomp=None, opacities=d.opacities,
                  scales=d.scales, rotations=d.rotations, cov3D_precomp=None)
    fps, ms_per_step = frame_loop(torch, rast, kwargs, args.warmup, args.steps)
    latency = None if args.compact else synchronised_latency(torch, lambda: rast(**kwargs), min(args.steps, 60))

    # the same frames with two in flight (alternating HIP streams, one workspace each): the next frame's
    # HBM-bound preprocess overlaps the current frame's VALU-bound blend.  Reported beside `value`, never as it.
    # Opt-in (--two-in-flight): overlapping kernels would distort the per-kernel durations of a profiler trace.
    fps_two_in_flight = None
    if args.two_in_flight:
        streams = [torch.cuda.Stream(device=dev) for _ in range(2)]
        with torch.no_grad():
            for k in range(4):
                with torch.cuda.stream(streams[k % 2]):
                    rast(**kwargs)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for k in range(args.steps):
                with torch.cuda.stream(streams[k % 2]):
                    rast(**kwargs)
            torch.cuda.synchronize()
        fps_two_in_flight = round(args.steps / (time.perf_counter() - t0), 2)

    # model-level frame rate: the reference's forward sequence (visibility prefilter, gather of the survivors,
    # rasterize), the fused single-pass variant that produces the same frame, and that variant with the scene
    # stored along a Morton curve (a load-time option of the checkpoint loaders)
    from landmarksystem_amd.models import GaussianModel, morton_order
    model_fps = {}
    for name, fuse, ordered in (() if args.no_model_level else (
            ("reference_sequence", False, False), ("fused_prefilter", True, False),
            ("fused_prefilter_spatial_order", True, True))):
        pick = morton_order(d.means3D) if ordered else slice(None)
        model = GaussianModel(d.means3D[pick], d.shs[pick][:, :1].contiguous(), d.shs[pick][:, 1:].contiguous(),
                              torch.log(d.scales[pick]), d.rotations[pick],
                              torch.logit(d.opacities[pick].clamp(1e-6, 1 - 1e-6)), sh_degree=scene.sh_degree,
                              act_cache=True, fuse_prefilter=fuse).eval()
        for _ in range(5):
            model(scene.camera)
        torch.cuda.synchronize()
        n_model, rates = max(20, args.steps // 2), []
        for _ in range(3):  # (the reference's sequence waits for the host every frame: median of three timings)
            t0 = time.perf_counter()
            for _ in range(n_model):
                model(scene.camera)
            torch.cuda.synchronize()
            rates.append(n_model / (time.perf_counter() - t0))
        model_fps[name] = round(sorted(rates)[1], 2)
        del model

    if args.calibration_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)  # 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del src, dst

    inp = pipeline.FrameInputs(rast.raster_settings, d.means3D, opacities=d.opacities, shs=d.shs, scales=d.scales,
                               rotations=d.rotations)
    n_cap = pipeline.default_workspace(dev).key_capacity
    stage_ms, stats = stage_breakdown(torch, pipeline, _lib, inp, n_cap, args.stage_steps)
    P, V, N = scene.P, stats["num_visible"], stats["num_keys"]
    pairs, pairs_error = (None, None) if args.no_cpu_baseline else guarded(cpu_pair_stats, scene, keep_frame=True)
    counters = COUNTER_TRAFFIC if (args.config == 3 and not args.gaussians and not args.spatial_order) else None
    stages, roofline = raster_report(stage_ms, stats, P, inp.tiles, inp.width * inp.height, 12 * scene.shs.shape[1],
                                     pairs, counters)
    parity, parity_error = guarded(parity_leg, torch, pipeline, inp, pairs["frame"]) if pairs else (None, None)
    if pairs:
        pairs["frame"] = None  # (a few hundred MB of host memory)
    if pairs and pairs["num_keys"] != N:
        stages["blend"]["pairs_note"] = "the checker counted %d keys, the GPU %d" % (pairs["num_keys"], N)
    if not args.no_backward:
        stages["backward"] = backward_report(torch, pipeline, inp, n_cap, N, V, P, scene.shs.shape[1], ms_per_step,
                                             args.stage_steps)
    metric = "1080p frames/sec at 6M Gaussians (1 GPU)" if args.config == 3 and not args.gaussians \
        and not args.spatial_order else \
        "%dx%d frames/sec at %d Gaussians (1 GPU)" % (inp.width, inp.height, P)
    result = base_line(metric, fps, ms_per_step, args, args.warmup, "f32", {
        "workload": "configs[%d]: %s, %d Gaussians, SH degree %d, %dx%d, RGB+depth+alpha" %
                    (args.config - 1, scene.name, P, scene.sh_degree, inp.width, inp.height),
        "visible": V, "keys": N, "tiles": inp.tiles, "scene_gen_s": round(gen_s, 1)})
    result.update({"roofline": roofline, "stages": stages, "model_forward_frames_per_s": model_fps,
                   "two_frames_in_flight_frames_per_s": fps_two_in_flight, "synchronised_per_frame": latency,
                   "steady_state_note": "the timed loop re-renders one camera, so the two per-frame hints the driver takes "
                                        "from the previous frame of its workspace (scatter variant, empty sorter classes) "
                                        "are always right; the 30-pose trajectory of configs[3] is the case where they "
                                        "change from frame to frame"})
    if not args.no_cpu_baseline:
        result["parity"] = parity if parity else {"error": parity_error or pairs_error}
        if args.compact:
            return result
        base, err = guarded(cpu_baseline, scene, pairs)
        result["cpu_baseline"] = base if base else {"error": err}
        if pairs_error:
            result["cpu_baseline"]["c_checker_error"] = pairs_error
    return result


def bench_trajectory(args, torch, dev):
    """configs[3]: large slab at 4K over a trajectory of aerial poses.  `value` is the frame rate over the
    trajectory; the stage breakdown, roofline and CPU baseline are those of its first pose."""
    from landmarksystem_amd import GaussianRasterizer, _lib, pipeline, scenes

    t0 = time.time()
    scene = scenes.config4(args.gaussians) if args.gaussians else scenes.config4()
    gen_s = time.time() - t0
    d = scene.to(dev)
    rast = GaussianRasterizer(settings_for(scene, dev))
    base = rast.raster_settings
    poses = [base._replace(viewmatrix=c.world_view_transform, projmatrix=c.full_proj_transform,
                           campos=c.camera_center) for c in d.cameras]
    kwargs = dict(means3D=d.means3D, means2D=None, shs=d.shs, colors_precomp=None, opacities=d.opacities,
                  scales=d.scales, rotations=d.rotations, cov3D_precomp=None)
    keys, visible = [], []
    with torch.no_grad():
        for k in range(len(poses)):  # warm-up pass over the trajectory, also collects the per-pose statistics
            rast.raster_settings = poses[k]
            _, radii, _ = rast(**kwargs)
            keys.append(rast.last_num_keys)
            visible.append(int((radii > 0).sum()))
    fps, ms_per_step = frame_loop(torch, rast, kwargs, 0, args.steps, settings_list=poses)

    rast.raster_settings = poses[0]
    inp = pipeline.FrameInputs(poses[0], d.means3D, opacities=d.opacities, shs=d.shs, scales=d.scales,
                               rotations=d.rotations)
    n_cap = pipeline.default_workspace(dev).key_capacity
    stage_ms, stats = stage_breakdown(torch, pipeline, _lib, inp, n_cap, max(3, args.stage_steps // 2))
    pairs, pairs_error = (None, None) if args.no_cpu_baseline else guarded(cpu_pair_stats, scene)
    stages, roofline = raster_report(stage_ms, stats, scene.P, inp.tiles, inp.width * inp.height,
                                     12 * scene.shs.shape[1], pairs, None)
    # the same scene stored along a Morton curve (the checkpoint loaders' spatial_order option): the survivors'
    # SH blocks are then neighbours in memory instead of isolated reads; same trajectory, reported beside `value`
    ordered = None
    if getattr(args, "spatial_leg", not args.no_model_level):
        from landmarksystem_amd.models import morton_order
        order = morton_order(d.means3D)
        kw2 = {k: (v[order].contiguous() if torch.is_tensor(v) else v) for k, v in kwargs.items()}
        del order
        with torch.no_grad():
            for k in range(len(poses)):
                rast.raster_settings = poses[k]
                rast(**kw2)
        fps2, ms2 = frame_loop(torch, rast, kw2, 0, args.steps, settings_list=poses)
        inp2 = pipeline.FrameInputs(poses[0], kw2["means3D"], opacities=kw2["opacities"], shs=kw2["shs"],
                                    scales=kw2["scales"], rotations=kw2["rotations"])
        ms_stage2, _ = stage_breakdown(torch, pipeline, _lib, inp2, n_cap, max(3, args.stage_steps // 2))
        ordered = {"frames_per_s": round(fps2, 2), "ms_per_frame": round(ms2, 4),
                   "preprocess_ms_pose0": round(ms_stage2["preprocess"], 4),
                   "preprocess_ms_pose0_generated_order": round(stage_ms["preprocess"], 4),
                   "note": "same Gaussians and poses, stored along a 3-D Morton curve; `value` is the generated "
                           "(random) order"}
        del kw2, inp2
    cam = scene.camera
    result = base_line("4K frames/sec at 20M Gaussians over 30 aerial poses (1 GPU)", fps, ms_per_step, args,
                       len(poses), "f32", {
        "workload": "configs[3]: %s, %d Gaussians, SH degree 3, %dx%d, %d poses" %
                    (scene.name, scene.P, cam.width, cam.height, len(poses)),
        "keys_min_mean_max": [min(keys), int(sum(keys) / len(keys)), max(keys)],
        "visible_fraction_min_max": [round(min(visible) / scene.P, 3), round(max(visible) / scene.P, 3)],
        "stages_of": "pose 0 (%d keys, %d visible)" % (stats["num_keys"], stats["num_visible"]),
        "tiles": inp.tiles, "scene_gen_s": round(gen_s, 1)})
    result.update({"roofline": roofline, "stages": stages})
    if ordered:
        result["spatial_order"] = ordered
    if not args.no_cpu_baseline:
        base, err = guarded(cpu_baseline, scene, pairs)
        result["cpu_baseline"] = base if base else {"error": err}
        if pairs_error:
            result["cpu_baseline"]["c_checker_error"] = pairs_error
    return result


def bench_scaffold(args, torch, dev):
    """configs[4]: Scaffold-GS, anchors decoded on the matrix cores, then rasterized."""
    from landmarksystem_amd import _lib, pipeline, scenes
    from landmarksystem_amd.models import OctreeGS, ScaffoldGS

    scene = scenes.config5(args.gaussians) if args.gaussians else scenes.config5()
    A = scene.anchor.shape[0]
    model = ScaffoldGS.from_scene(scene, act_cache=True).to(dev).eval()  # the model as shipped: one-kernel prefilter
    cam = scene.camera.to(dev)
    for _ in range(args.warmup):
        model(cam)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model(cam)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    fps, ms_per_step = args.steps / elapsed, elapsed * 1e3 / args.steps
    latency = None if args.compact else synchronised_latency(torch, lambda: model(cam), min(args.steps, 60))

    # the same frames through the reference's own call sequence (fuse_prefilter=False: prefilter, decoder with the
    # Gaussian count read back, renderer), and an Octree-GS model over the same anchors (random levels 0..4) with the
    # reference's level-of-detail sequence and with the fused prefilter
    variants = {}
    level = torch.randint(0, 5, (A,), generator=torch.Generator().manual_seed(5))
    for name, make in () if args.no_model_level else (
        ("scaffold_reference_sequence", lambda: ScaffoldGS.from_scene(scene, act_cache=True, fuse_prefilter=False)),
        ("octree_reference_sequence", lambda: OctreeGS(
            scene.anchor, scene.anchor_feat, scene.offset, torch.log(scene.scaling), scene.rotation, level,
            voxel_size=0.5, standard_dist=250.0, n_offsets=scene.n_offsets, act_cache=True, fuse_prefilter=False)),
        ("octree_fused_prefilter", lambda: OctreeGS(
            scene.anchor, scene.anchor_feat, scene.offset, torch.log(scene.scaling), scene.rotation, level,
            voxel_size=0.5, standard_dist=250.0, n_offsets=scene.n_offsets, act_cache=True, fuse_prefilter=True)),
    ):
        other = make()
        other.anchor_decoder.load_state_dict(model.anchor_decoder.state_dict())
        other = other.to(dev).eval()
        for _ in range(5):
            other(cam)
        torch.cuda.synchronize()
        rates = []  # these paths wait for the host every frame, and the host is a shared machine: median of three
        for _ in range(3):
            t1 = time.perf_counter()
            for _ in range(args.steps):
                other(cam)
            torch.cuda.synchronize()
            rates.append(args.steps / (time.perf_counter() - t1))
        variants[name] = round(sorted(rates)[1], 2)
        del other

    # stages: anchor prefilter and decode alone (HIP events on the launch stream), then the rasterizer stages on the
    # decoded Gaussians
    def timed(call):
        for _ in range(3):
            call()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.stage_steps):
            res = call()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.stage_steps, res

    with torch.no_grad():
        prefilter_ms, vis = timed(lambda: model.prefilter_voxel(cam))
        dec_args = dict(camera_center=cam.camera_center, anchor=model.get_anchor, anchor_feat=model.get_anchor_feat,
                        offset=model.get_offset, scaling=model.get_scaling, visible_mask=vis)
        dec_ms, dec = timed(lambda: model.anchor_decoder(**dec_args))
        # the same call with weights that fp16 cannot represent (an fp32-trained checkpoint): the decoder then carries
        # them as hi + lo fp16 pairs (more matrix instructions, the low parts in LDS, three wavefronts per workgroup)
        src = model.anchor_decoder
        general = type(src)(src.use_feat_bank, src.add_opacity_dist, src.add_color_dist, src.add_cov_dist, src.view_dim,
                            src.feat_dim, src.n_offsets).to(dev).eval()
        gen = torch.Generator().manual_seed(7)
        for prm, given in zip(general.parameters(), src.parameters()):
            prm.copy_(given * (1.0 + 1e-3 * torch.randn(prm.shape, generator=gen).to(dev)))
        dec32_ms, _ = timed(lambda: general(**dec_args))
        # and with features off the fp16 grid as well (what a trained checkpoint holds): two more matrix instructions
        # per head for their low parts
        feat32 = dec_args["anchor_feat"] * (1.0 + 1e-3 * torch.randn(dec_args["anchor_feat"].shape, generator=gen).to(dev))
        dec32b_ms, _ = timed(lambda: general(**dict(dec_args, anchor_feat=feat32)))
        del general, feat32
    xyz, color, opacity, scaling, rot = dec[:5]
    a_vis, G = int(vis.sum()), int(xyz.shape[0])
    flops = 13952 * a_vis
    dec_bytes = a_vis * (128 + 120 + 24 + 12) + A * 1 + G * 56
    settings = settings_for(scene, dev, sh_degree=1)
    inp = pipeline.FrameInputs(settings, xyz, opacities=opacity, colors_precomp=color, scales=scaling, rotations=rot)
    n_cap = max(pipeline.default_workspace(dev).key_capacity, 1 << 20)
    stage_ms, stats = stage_breakdown(torch, pipeline, _lib, inp, n_cap, args.stage_steps)

    decoded = scenes.GaussianScene("decoded", xyz.cpu(), scaling.cpu(), rot.cpu(), opacity.cpu(),
                                   torch.zeros(G, 1, 3), 1, [scene.camera], scene.bg)
    pairs, pairs_error = (None, None) if args.no_cpu_baseline else guarded(
        cpu_pair_stats, decoded, colors_precomp=color.cpu().numpy(), sh_degree=1)
    stages, roofline = raster_report(stage_ms, stats, G, inp.tiles, inp.width * inp.height, 12, pairs, None)
    stages["anchor_prefilter"] = {"ms": round(prefilter_ms, 4), "bytes": 36 * A,
                                  "GBps": round(36 * A / prefilter_ms / 1e6, 1),
                                  "frac_hbm": round(36 * A / prefilter_ms / 1e6 / HBM_PEAK_GBS, 4)}
    stages["decode"] = {"ms": round(dec_ms, 4), "ms_fp32_weights": round(dec32_ms, 4),
                        "ms_fp32_weights_and_features": round(dec32b_ms, 4), "anchors_per_s": round(a_vis / dec_ms * 1e3), "flops": flops,
                        "TFLOPs": round(flops / dec_ms / 1e9, 3),
                        "frac_mfma_f16": round(flops / dec_ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 6),
                        "bytes": dec_bytes, "GBps": round(dec_bytes / dec_ms / 1e6, 1),
                        "frac_hbm": round(dec_bytes / dec_ms / 1e6 / HBM_PEAK_GBS, 4),
                        "note": "bound by HBM and instruction issue, not by the matrix cores (17 flop/B); bytes = inputs "
                                "of the visible anchors once + the visibility mask + 56 B per emitted Gaussian"}
    quoted = COUNTER_TRAFFIC_C5["bytes"]["decode"] if not args.gaussians else None  # (counted on the named workload)
    if quoted:
        stages["decode"].update({"counter_bytes": quoted, "counter_GBps": round(quoted / dec_ms / 1e6, 1),
                                 "frac_hbm_counter": round(quoted / dec_ms / 1e6 / HBM_PEAK_GBS, 4)})
    if dec_ms > max(stage_ms["preprocess"], stage_ms["blend"]):  # the dominant kernel(s): count + emit of the decode
        roofline = {"bound": "hbm", "kernel": "decode_kernel", "achieved": stages["decode"]["GBps"], "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": stages["decode"]["frac_hbm"], "traffic": quoted,
                    "traffic_source": (COUNTER_TRAFFIC_C5["source"] + " (rocprofv3 FETCH_SIZE + WRITE_SIZE of an earlier "
                                       "run of this workload)") if quoted else None,
                    "mfma_frac": stages["decode"]["frac_mfma_f16"]}
    result = base_line("1080p frames/sec, Scaffold-GS with 500k anchors (1 GPU)", fps, ms_per_step, args, args.warmup,
                       "f32 (decode: f16 matrix inputs as hi+lo pairs, f32 accumulate)", {
        "workload": "configs[4]: %d anchors x %d offsets, 1920x1080" % (A, scene.n_offsets),
        "visible_anchors": a_vis, "decoded_gaussians": G, "keys": stats["num_keys"], "tiles": inp.tiles})
    result.update({"roofline": roofline, "stages": stages, "model_variants_frames_per_s": variants,
                   "synchronised_per_frame": latency})
    if not args.no_cpu_baseline:
        def whole():
            from oracle import anchor_oracle
            t1 = time.perf_counter()
            anchor_oracle.decode(scene.camera.camera_center, scene.anchor, scene.anchor_feat, scene.offset,
                                 scene.scaling, vis.cpu(), scene.mlp, scene.n_offsets)
            dec_s = time.perf_counter() - t1
            return cpu_baseline(decoded, pairs, colors_precomp=color.cpu(), extra_seconds=dec_s,
                                extra_note="anchor decode (oracle/anchor_oracle.py, %d visible anchors) %.2fs + " % (a_vis, dec_s))
        base, err = guarded(whole)
        result["cpu_baseline"] = base if base else {"error": err}
        if pairs_error:
            result["cpu_baseline"]["c_checker_error"] = pairs_error
    return result


def compact_entry(line):
    """What `other_configs` keeps of another workload's bench line: frame rate, the stage times, the dominant
    kernel with its roofline figure, and the parity object where the line has one."""
    stages = line.get("stages", {})
    keep = {"metric": line["metric"], "frames_per_s": line["value"], "ms_per_frame": line["ms_per_step"],
            "steps": line["steps"], "workload": line["config"].get("workload"),
            "stage_ms": {k: v["ms"] for k, v in stages.items() if isinstance(v, dict) and "ms" in v},
            "dominant_kernel": line["roofline"].get("kernel"), "roofline": {
                k: line["roofline"].get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "work_rate", "mfma_frac")
                if line["roofline"].get(k) is not None}}
    for name in ("preprocess", "keys_sort_ranges", "decode"):
        if name in stages and "frac_hbm" in stages[name]:
            keep.setdefault("frac_hbm_algorithmic", {})[name] = stages[name]["frac_hbm"]
    for extra in ("parity", "model_variants_frames_per_s", "spatial_order"):
        if line.get(extra):
            keep[extra] = line[extra]
    for extra in ("keys_min_mean_max", "visible_fraction_min_max", "visible_anchors", "decoded_gaussians", "keys"):
        if extra in line["config"]:
            keep[extra] = line["config"][extra]
    return keep


def other_configs(args, torch, dev):
    """Compact lines of the other single-GPU workloads of the benchmark definition, measured in the same run: configs[1]
    (1M Gaussians, with its parity object), configs[3] (20M Gaussians at 4K over the 30-pose trajectory) and
    configs[4] (Scaffold-GS, 500k anchors)."""
    import copy
    import gc
    out = {}
    for index, fn, steps in ((2, bench_vanilla, 200), (4, bench_trajectory, 60), (5, bench_scaffold, 200)):
        sub = copy.copy(args)
        sub.config, sub.gaussians, sub.spatial_order, sub.two_in_flight, sub.calibration_copy = index, None, False, False, False
        sub.steps, sub.warmup, sub.stage_steps, sub.compact = steps, 10, 10, True
        sub.no_model_level, sub.no_backward, sub.spatial_leg = index != 5, True, index == 4
        sub.no_cpu_baseline = index != 2  # the C checker renders the 1M-Gaussian frame in well under a second
        line, err = guarded(fn, sub, torch, dev)
        out["configs[%d]" % (index - 1)] = compact_entry(line) if line else {"error": err}
        del line
        gc.collect()
        torch.cuda.empty_cache()
    return out


def main():
    args = parse_args()
    args.compact = False
    if args.gpus != 1:
        print("bench.py: this build renders on one GPU; --gpus %d is not supported (run with --gpus 1)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch

    from landmarksystem_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _lib.load()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.config == 4:
        result = bench_trajectory(args, torch, dev)
    elif args.config == 5:
        result = bench_scaffold(args, torch, dev)
    else:
        result = bench_vanilla(args, torch, dev)
        if args.config == 3 and not args.gaussians and not args.spatial_order and not args.no_other_configs:
            import gc
            gc.collect()
            torch.cuda.empty_cache()
            result["other_configs"] = other_configs(args, torch, dev)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
