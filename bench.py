#!/usr/bin/env python3
"""Benchmark of the blending point rasterizer on one MI355X.

One step = one forward + backward pass of the hot path over one frame of synthetic input (BASELINE config 3: 2 M points
on 200 planes/spheres, 1920x1080, 4 layers, K=16, gradients to descriptors, confidence and xyz). Inputs, outputs and
the workspace are resident in HBM before the timed region starts. Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|3|5] [--point-order vet_preprocess|generated]
                  [--no-cpu-baseline] [--no-second-order | --no-other-order]
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_config3.md")


def algorithmic_bytes(N, P, F, Fk, Cn):
    """Compulsory bytes per view and kernel, each datum counted once per producer and once per consumer (4-byte scalars):
    B_fwd = 32N + 36P + 24F + 28Fk, B_bwd = 32P + 116Fk + 40N for C = 4.

    N points, P pixels over all layers, F fragments, Fk fragments kept after the top-K cut.
    """
    fwd = {
        # the model's terms, booked on the kernels that do the corresponding work here
        # one pass over the points projects them, counts the bins and writes the fragment records (the model reads the
        # positions twice, as the reference's two passes do; both reads are booked here)
        "COUNT": 32 * N + 8 * F,
        "FILL": 0,                                    # files the few records that overflow a bin's own room
        # per-pixel counts, counts -> offsets, records read and written sorted; then the blend: lists, descriptor +
        # confidence, offsets, out, weight
        "BUILD": 4 * P + 8 * P + 16 * F + 8 * Fk + (4 * Cn + 4) * Fk + 4 * P + 4 * Cn * P + 4 * P,
    }
    # The per-pixel kernel reads upstream grads and forward outputs (8CP), lists (8Fk), descriptor+confidence (4(C+1)Fk)
    # and writes one half of the gradient read-modify-write (4(C+1+4)Fk); the per-point kernel reads positions (16Fk in the
    # model), that half back, and writes the gradient rows (4(C+1+4+1)N, the term the reference spends on zero-filling).
    rmw_half = 4 * (Cn + 1 + 4) * Fk
    bwd = {
        "BACKWARD_BLEND": 8 * Cn * P + 8 * Fk + (4 * Cn + 4) * Fk + rmw_half,
        "BACKWARD_GATHER": 16 * Fk + rmw_half + 4 * (Cn + 1 + 4 + 1) * N,
    }
    return fwd, bwd


def measured_traffic():
    """HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, read from the committed summary
    (rows `| SCOPE | fetch KiB | write KiB |`, already scaled by the copy-kernel calibration). Empty if absent."""
    res = {}
    if not os.path.exists(TRAFFIC_FILE):
        return res
    in_table = False
    for line in open(TRAFFIC_FILE):
        if line.startswith("## "):
            in_table = line.startswith("## Per scope")
        if not in_table:
            continue
        m = re.match(r"^\|\s*([A-Z_]+)\s*\|\s*([0-9.]+)\s*\|\s*([0-9.]+)\s*\|", line)
        if m:
            res[m.group(1)] = (float(m.group(2)) + float(m.group(3))) * 1024.0
    return res


def run_scene(scene, backward, steps, warmup, profile=True, render_mode=1):
    import torch

    from vet_amd import abi
    from vet_amd.rasterizer import DeviceScene, Rasterizer, make_params

    params = make_params(scene, need_point_gradient=1 if backward else 0, render_mode=render_mode)
    N, Cn, L = scene.num_points, scene.num_channels, scene.num_layers
    rast = Rasterizer()
    dev = DeviceScene(scene)
    lay = rast.layout(scene, render_mode)
    workspace = torch.empty(lay.total_bytes, dtype=torch.uint8, device="cuda")
    out = [torch.empty((len(scene.views), Cn, h, w), dtype=torch.float32, device="cuda") for (w, h) in scene.layer_sizes()]
    fwd = rast.forward(dev, params, save_for_backward=backward, workspace=workspace, out=out)
    torch.cuda.synchronize()
    off = fwd.offsets(0)
    P = fwd.total_pixels()
    counts = np.diff(off)
    K = params.debug_max_list_length
    F = int(off[-1])
    Fk = int(fwd.kept(0).sum())  # fragments that took part in the blend (top-K cut, in mode 3 also saturation)
    bases = fwd.layer_bases()
    F_layers = [int(off[bases[l + 1]] - off[bases[l]]) for l in range(L)]

    bargs = None
    if backward:
        grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
        first = rast.backward(fwd, grad_out)  # allocates the gradient tensors once; reused below
        bargs = first["_args"]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lib, ctx = rast.lib, rast.ctx

    def forward_only():
        abi.check(lib.vetrast_forward(ctx, C.byref(fwd.args), stream), "forward")

    def step():
        forward_only()
        if backward:
            abi.check(lib.vetrast_backward(ctx, C.byref(bargs), stream), "backward")

    def timed(fn, nwarm, nsteps):
        for _ in range(nwarm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(nsteps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / nsteps

    res = {"ms_step": timed(step, warmup, steps)}
    res["ms_fwd"] = timed(forward_only, 2, steps) if backward else res["ms_step"]
    res.update(N=N, P=P, F=F, Fk=Fk, F_layers=F_layers, K=K, Cn=Cn, L=L, params=params)
    if profile:
        # per-kernel times: HIP events recorded by the library on the launch stream around every scope
        rast.set_profiling(True)
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        rast.reset_scope_times()
        prof_steps = max(5, min(steps, 20))
        for _ in range(prof_steps):
            step()
        torch.cuda.synchronize()
        scopes = rast.scope_times()
        rast.set_profiling(False)
        res["per_launch_ms"] = {k: (ms / n if n else 0.0) for k, (ms, n) in scopes.items()}
        res["per_step_ms"] = {k: ms / prof_steps for k, (ms, n) in scopes.items()}
    del workspace, out, fwd
    torch.cuda.empty_cache()
    return res


def time_fused_steps(scene, render_mode, steps):
    """The steps VET runs either side of the rasterizer, fused into the library: the frame with the confidence sigmoid
    and |texture| folded in (raw tensors in, raw gradients out), and the one-kernel Adam step over texture, confidence
    and background (vetrast_adam_step). Reported beside the headline number, not part of it."""
    import torch

    from vet_amd import abi
    from vet_amd.rasterizer import DeviceScene, Rasterizer, make_params

    rast = Rasterizer()
    dev = DeviceScene(scene)
    params = make_params(scene, need_point_gradient=1, render_mode=render_mode, confidence_activation=1,
                         confidence_scale=10.0, texture_abs=1)
    fwd = rast.forward(dev, params, save_for_backward=True)
    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    bargs = rast.backward(fwd, grad_out)["_args"]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n

    def frame():
        abi.check(rast.lib.vetrast_forward(rast.ctx, C.byref(fwd.args), stream), "forward")
        abi.check(rast.lib.vetrast_backward(rast.ctx, C.byref(bargs), stream), "backward")

    ms_frame = timed(frame, steps)
    n = (scene.num_channels + 1) * scene.num_points + scene.num_channels
    p, g, m, v = (torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(4))
    g.normal_()
    state = {"step": 0}

    def adam():
        state["step"] += 1
        rast.adam_step(p, g, m, v, state["step"], 1e-3)

    ms_adam = timed(adam, steps)
    adam_bytes = 28.0 * n  # param, grad, two moments read; param and moments written
    return {"frame_with_fused_sigmoid_abs_ms": round(ms_frame, 5), "adam_step_ms": round(ms_adam, 5),
            "adam_elements": n, "adam_GBps": round(adam_bytes / 1e6 / ms_adam, 1),
            "adam_frac_of_hbm_peak": round(adam_bytes / 1e6 / ms_adam / HBM_PEAK_GBS, 4)}


def time_lift_error(scene, steps, cpu_threads):
    """Error lifting (vetrast_lift_error; the reference's FillSceneGridWithLoss), the step that runs once per view in the
    epoch before VET adds points: the scene's grid at 0.25 m under the scene's own camera and a synthetic 3-channel
    error image. Reported beside the headline number, not part of it; the CPU oracle is timed on the same call."""
    import torch

    from vet_amd import synthetic
    from vet_amd.rasterizer import Rasterizer

    rast = Rasterizer()
    cell_size = 0.25
    mn, ln = synthetic.cell_grid(scene.position[:, :3], cell_size)
    view = scene.views[0]
    img = synthetic.error_image(5, 3, view.h, view.w)
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    d_mn, d_ln, d_img, d_pose, d_intr = (to_dev(a) for a in (mn, ln, img, scene.poses_se3, scene.intrinsics))
    val = torch.zeros(len(mn), dtype=torch.float32, device="cuda")
    cnt = torch.zeros(len(mn), dtype=torch.int32, device="cuda")
    ws = rast.lift_error(d_mn, d_ln, val, cnt, view, d_pose, d_intr, d_img)
    torch.cuda.synchronize()
    pixels = int(cnt.sum().item())
    queued = int(ws[128:132].view(torch.int32).item())
    for _ in range(3):
        rast.lift_error(d_mn, d_ln, val, cnt, view, d_pose, d_intr, d_img, workspace=ws)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        rast.lift_error(d_mn, d_ln, val, cnt, view, d_pose, d_intr, d_img, workspace=ws)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    out = {"cells": int(len(mn)), "cell_size_m": cell_size, "cells_on_shared_path": queued, "pixels_added": pixels,
           "ms_per_call": round(ms, 5), "pixels_added_per_s": round(pixels / ms * 1e3, 0)}
    if cpu_threads:
        from oracle import oracle_py

        v = np.zeros(len(mn), np.float32)
        c = np.zeros(len(mn), np.int32)
        t0 = time.perf_counter()
        oracle_py.lift_error(mn, ln, v, c, view, scene.poses_se3, scene.intrinsics, img, num_threads=cpu_threads)
        out["cpu_oracle_ms"] = round((time.perf_counter() - t0) * 1e3, 1)
        out["cpu_oracle_threads"] = cpu_threads
        out["counts_equal_cpu_oracle"] = bool(np.array_equal(c, cnt.cpu().numpy() // (steps + 4)))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=3, choices=[2, 3, 5])
    ap.add_argument("--points", type=int, default=None, help="override the point count (debug runs)")
    ap.add_argument("--point-order", default="vet_preprocess", choices=["vet_preprocess", "generated"])
    ap.add_argument("--render-mode", type=int, default=1, choices=[1, 2, 3],
                    help="1 = FULL_BLEND (the headline workload), 3 = BILINEAR_BLEND (four fragments per point and layer)")
    ap.add_argument("--no-second-order", action="store_true",
                    help="skip everything beside the headline: the other point order, the fused steps, the error lifting")
    ap.add_argument("--no-other-order", action="store_true", help="skip timing the other point order only")
    ap.add_argument("--calibration-kernel", action="store_true",
                    help="also run the Adam kernel a few times: a streaming kernel that reads 16 and writes 12 bytes per "
                         "element, against which byte counters of a profiler run are scaled")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--lift-only", action="store_true",
                    help="time only the error lifting on the configuration's scene and print its object")
    ap.add_argument("--cpu-threads", type=int, default=0, help="0 = min(16, available cores)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the rasterizer on ONE GPU (views of a batch are rendered back to back); "
              "--gpus N with N > 1 is not available", file=sys.stderr)
        sys.exit(2)

    import torch

    from vet_amd import synthetic

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path in the product)", file=sys.stderr)
        sys.exit(2)

    kw = {"point_order": args.point_order}
    if args.points is not None:
        kw["num_points"] = args.points
    make = {2: synthetic.config2, 3: synthetic.config3, 5: synthetic.config5}[args.config]
    backward = args.config != 2
    scene = make(**kw)
    if args.lift_only:
        threads = 0 if args.no_cpu_baseline else (args.cpu_threads or min(16, len(os.sched_getaffinity(0))))
        print(json.dumps({"lift_error": time_lift_error(scene, args.steps, threads)}))
        return
    r = run_scene(scene, backward, args.steps, args.warmup, render_mode=args.render_mode)
    N, P, F, Fk, Cn, L, K = r["N"], r["P"], r["F"], r["Fk"], r["Cn"], r["L"], r["K"]
    ms_step, ms_fwd = r["ms_step"], r["ms_fwd"]

    fwd_b, bwd_b = algorithmic_bytes(N, P, F, Fk, Cn)
    alg = dict(fwd_b)
    if backward:
        alg.update(bwd_b)
    traffic = measured_traffic() if (args.config == 3 and args.points is None and args.point_order == "vet_preprocess"
                                     and args.render_mode == 1) else {}
    kernels = {}
    for k, nbytes in alg.items():
        t = r["per_step_ms"].get(k, 0.0)
        kernels[k] = {"ms": round(t, 5), "alg_MB": round(nbytes / 1e6, 3),
                      "GBps": round(nbytes / 1e6 / t, 1) if t > 0 else None,
                      "frac": round(nbytes / 1e6 / t / HBM_PEAK_GBS, 4) if t > 0 else None}
        if k in traffic:
            kernels[k]["hbm_traffic_MB"] = round(traffic[k] / 1e6, 1)
    for k in ("PREPARE", "PACK", "SCAN", "BACKWARD_PREPARE", "BACKWARD_POST"):
        if r["per_step_ms"].get(k, 0.0) > 0:
            kernels[k] = {"ms": round(r["per_step_ms"][k], 5), "alg_MB": 0.0, "GBps": None, "frac": None}
    dominant = max(alg.keys(), key=lambda k: r["per_step_ms"].get(k, 0.0))
    dom_ms = r["per_launch_ms"][dominant]
    achieved = alg[dominant] / 1e6 / dom_ms if dom_ms > 0 else 0.0
    total_alg = sum(alg.values())

    result = {
        "metric": "fwd+bwd ms/frame (1080p, 2M pts, 4 layers)" if backward else "fwd ms/frame (1080p, 2M pts, 4 layers)",
        "value": round(ms_step, 5),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"BASELINE config {args.config} ({scene.name}): N={N} points, {scene.views[0].w}x{scene.views[0].h}, "
                        f"L={L} layers, K={K}, C={Cn}, B=1 view, " + ("forward+backward" if backward else "forward")
                        + f", point order {args.point_order}"
                        + {1: ", render_mode 1 (FULL_BLEND)", 2: ", render_mode 2 (FUZZY_BLEND, depth_accept_blend 0.01)",
                           3: ", render_mode 3 (BILINEAR_BLEND)"}[args.render_mode],
            "point_order": args.point_order, "render_mode": args.render_mode,
            "fragments_per_layer": r["F_layers"], "fragments": F, "fragments_kept": Fk, "pixels": P,
        },
        "forward_ms": round(ms_fwd, 5),
        "backward_ms": round(ms_step - ms_fwd, 5) if backward else None,
        "step_algorithmic_MB": round(total_alg / 1e6, 3),
        "step_GBps": round(total_alg / 1e6 / ms_step, 1),
        "step_frac_of_hbm_peak": round(total_alg / 1e6 / ms_step / HBM_PEAK_GBS, 4),
        "roofline": {
            "kernel": dominant,
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": int(traffic[dominant]) if dominant in traffic else None,
            "avg_launch_ms": round(dom_ms, 5),
            "algorithmic_bytes_per_launch": alg[dominant],
        },
        "kernels": kernels,
    }

    if not (args.no_second_order or args.no_other_order):
        # VET hands the rasterizer Morton-ordered clouds with shuffled 256-point blocks; the generator's raw order
        # (random inside each primitive) is timed as well so that the effect of that order is visible.
        other = "generated" if args.point_order == "vet_preprocess" else "vet_preprocess"
        r2 = run_scene(make(**dict(kw, point_order=other)), backward, max(10, args.steps // 2), 5, profile=False,
                       render_mode=args.render_mode)
        result["other_point_order"] = {"point_order": other, "ms_per_step": round(r2["ms_step"], 5),
                                       "forward_ms": round(r2["ms_fwd"], 5)}

    if backward and not args.no_second_order:
        result["fused_steps"] = time_fused_steps(scene, args.render_mode, max(10, args.steps // 2))
    if args.calibration_kernel:
        import torch

        from vet_amd.rasterizer import Rasterizer

        n = (scene.num_channels + 1) * scene.num_points + scene.num_channels
        p_, g_, m_, v_ = (torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(4))
        rast_c = Rasterizer()
        for k in range(3):
            rast_c.adam_step(p_, g_, m_, v_, k + 1, 1e-3)
        torch.cuda.synchronize()
        result["calibration_kernel"] = {"kernel": "adam_step_kernel", "elements": n, "read_bytes": 16 * n,
                                        "write_bytes": 12 * n}

    if not args.no_second_order:
        lift_threads = 0 if args.no_cpu_baseline else (args.cpu_threads or min(16, len(os.sched_getaffinity(0))))
        result["lift_error"] = time_lift_error(scene, max(10, args.steps // 2), lift_threads)

    if not args.no_cpu_baseline:
        from oracle import oracle_py

        cores = args.cpu_threads or min(16, len(os.sched_getaffinity(0)))
        oracle_py.load()
        cpu_grad_out = scene.grad_out() if backward else None

        def cpu_step(threads):
            t0 = time.perf_counter()
            f = oracle_py.forward(scene, r["params"], num_threads=threads)
            t1 = time.perf_counter()
            if backward:
                oracle_py.backward(f, cpu_grad_out, num_threads=threads)
            t2 = time.perf_counter()
            return (t2 - t0) * 1e3, (t1 - t0) * 1e3

        single_ms, _ = cpu_step(1)
        runs = [cpu_step(cores) for _ in range(3)]
        multi_ms = float(np.median([x[0] for x in runs]))
        result["cpu_baseline"] = {
            "value": round(multi_ms, 2),
            "unit": "ms",
            "cores": cores,
            "kind": "port",
            "sample": f"the same frame (config {args.config}, all {N} points): CPU oracle, median of 3 runs on {cores} "
                      f"threads; one run on 1 thread = {single_ms:.1f} ms",
            "single_thread_ms": round(single_ms, 2),
            "forward_ms": round(float(np.median([x[1] for x in runs])), 2),
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
