#!/usr/bin/env python3
"""Benchmark of the blending point rasterizer on one MI355X.

One step = one forward + backward pass of the hot path over one frame of synthetic input (config 3: 2 M points on 200
planes/spheres, 1920x1080, 4 layers, K=16, gradients to descriptors, confidence and xyz). Inputs, outputs and the
workspace are resident in HBM before the timed region starts. Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|3|5] [--no-cpu-baseline]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E


def algorithmic_bytes(N, P, F, Fk, Cn):
    """Compulsory bytes per view and pass, each datum counted once per producer and once per consumer (4-byte scalars).

    N points, P pixels over all layers, F fragments, Fk fragments kept after the top-K cut.
    """
    fwd = {
        "COUNT": 16 * N + 4 * P,                      # positions read, counts written
        "SCAN": 8 * P,                                # counts read, offsets written
        "FILL": 16 * N + 8 * F,                       # positions read again, fragment records written
        "SORT": 16 * F,                               # records read and written
        "BLEND": 8 * Fk + (4 * Cn + 4) * Fk + 4 * P + 4 * Cn * P + 4 * P,  # lists, descriptor+confidence, offsets, out, weight
    }
    # B_bwd = 32P + 116Fk + 40N for C = 4, split over the two backward kernels: the per-pixel kernel reads upstream
    # grads and forward outputs (8CP), lists (8Fk), descriptor+confidence (4(C+1)Fk), positions (16Fk) and writes one
    # half of the gradient read-modify-write (4(C+1+4)Fk); the per-point kernel reads that half back and writes the
    # gradient rows (4(C+1+4+1)N, the term the reference spends on zero-filling them).
    rmw_half = 4 * (Cn + 1 + 4) * Fk
    bwd = {
        "BACKWARD_BLEND": 8 * Cn * P + 8 * Fk + (4 * Cn + 4) * Fk + 16 * Fk + rmw_half,
        "BACKWARD_GATHER": rmw_half + 4 * (Cn + 1 + 4 + 1) * N,
    }
    return fwd, bwd


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=3, choices=[2, 3, 5])
    ap.add_argument("--points", type=int, default=None, help="override the point count (parity/debug runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-threads", type=int, default=0, help="0 = min(16, available cores)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the rasterizer on ONE GPU (views of a batch are rendered back to back); "
              "--gpus N with N > 1 is not available", file=sys.stderr)
        sys.exit(2)

    import torch

    from vet_amd import abi, synthetic
    from vet_amd.rasterizer import DeviceScene, Rasterizer, make_params

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path in the product)", file=sys.stderr)
        sys.exit(2)

    kw = {} if args.points is None else {"num_points": args.points}
    if args.config == 2:
        scene, backward = synthetic.config2(**kw), False
    elif args.config == 3:
        scene, backward = synthetic.config3(**kw), True
    else:
        scene, backward = synthetic.config5(**kw), True
    params = make_params(scene, need_point_gradient=1 if backward else 0)
    N, Cn, L = scene.num_points, scene.num_channels, scene.num_layers

    rast = Rasterizer()
    dev = DeviceScene(scene)
    lay = rast.layout(scene)
    workspace = torch.empty(lay.total_bytes, dtype=torch.uint8, device="cuda")
    out = [torch.empty((1, Cn, h, w), dtype=torch.float32, device="cuda") for (w, h) in scene.layer_sizes()]
    fwd = rast.forward(dev, params, save_for_backward=backward, workspace=workspace, out=out)
    torch.cuda.synchronize()
    off = fwd.offsets(0)
    P = fwd.total_pixels()
    counts = np.diff(off)
    K = params.debug_max_list_length
    F = int(off[-1])
    Fk = int(np.minimum(counts, K).sum()) if K > 0 else F
    F_layers = [int(off[int(lay.layer_pixel_base[l + 1])] - off[int(lay.layer_pixel_base[l])]) for l in range(L)]

    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()] if backward else None
    bargs = None
    if backward:
        first = rast.backward(fwd, grad_out)  # allocates the gradient tensors once; reused below
        bargs = first["_args"]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lib, ctx = rast.lib, rast.ctx

    def step():
        abi.check(lib.vetrast_forward(ctx, C.byref(fwd.args), stream), "forward")
        if backward:
            abi.check(lib.vetrast_backward(ctx, C.byref(bargs), stream), "backward")

    def forward_only():
        abi.check(lib.vetrast_forward(ctx, C.byref(fwd.args), stream), "forward")

    def timed(fn, warmup, steps):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    ms_step = timed(step, args.warmup, args.steps)
    ms_fwd = timed(forward_only, 2, args.steps) if backward else ms_step

    # ---- per-kernel times, HIP events on the launch stream ------------------------------------------------------
    rast.set_profiling(True)
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    rast.reset_scope_times()
    prof_steps = max(5, min(args.steps, 20))
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    scopes = rast.scope_times()
    rast.set_profiling(False)
    per_launch_ms = {k: (ms / n if n else 0.0) for k, (ms, n) in scopes.items()}
    per_step_ms = {k: ms / prof_steps for k, (ms, n) in scopes.items()}

    fwd_b, bwd_b = algorithmic_bytes(N, P, F, Fk, Cn)
    alg = dict(fwd_b)
    if backward:
        alg.update(bwd_b)
    kernels = {}
    for k, nbytes in alg.items():
        t = per_step_ms.get(k, 0.0)
        kernels[k] = {"ms": round(t, 5), "alg_MB": round(nbytes / 1e6, 3),
                      "GBps": round(nbytes / 1e6 / t, 1) if t > 0 else None}
    kernels["PREPARE"] = {"ms": round(per_step_ms.get("PREPARE", 0.0), 5), "alg_MB": 0.0, "GBps": None}
    dominant = max(alg.keys(), key=lambda k: per_step_ms.get(k, 0.0))
    dom_ms = per_step_ms[dominant]
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
                        f"L={L} layers, K={K}, C={Cn}, B=1 view, " + ("forward+backward" if backward else "forward"),
            "fragments_per_layer": F_layers, "fragments": F, "fragments_kept": Fk, "pixels": P,
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
            "traffic": None,
            "avg_launch_ms": round(per_launch_ms[dominant], 5),
            "algorithmic_bytes_per_launch": alg[dominant],
        },
        "kernels": kernels,
    }

    if not args.no_cpu_baseline:
        from oracle import oracle_py

        cores = args.cpu_threads or min(16, len(os.sched_getaffinity(0)))
        oracle_py.load()
        cpu_grad_out = scene.grad_out() if backward else None

        def cpu_step(threads):
            t0 = time.perf_counter()
            f = oracle_py.forward(scene, params, num_threads=threads)
            t1 = time.perf_counter()
            if backward:
                oracle_py.backward(f, cpu_grad_out, num_threads=threads)
            t2 = time.perf_counter()
            return (t2 - t0) * 1e3, (t1 - t0) * 1e3

        single_ms, single_fwd = cpu_step(1)
        runs = [cpu_step(cores) for _ in range(3)]
        multi_ms = float(np.median([r[0] for r in runs]))
        result["cpu_baseline"] = {
            "value": round(multi_ms, 2),
            "unit": "ms",
            "cores": cores,
            "kind": "port",
            "sample": f"the same frame (config {args.config}, all {N} points): CPU oracle, median of 3 runs on {cores} "
                      f"threads; one run on 1 thread = {single_ms:.1f} ms",
            "single_thread_ms": round(single_ms, 2),
            "forward_ms": round(float(np.median([r[1] for r in runs])), 2),
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
