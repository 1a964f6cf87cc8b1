#!/usr/bin/env python3
"""Benchmark of the blending point rasterizer on one MI355X.

One step = one forward + backward pass of the hot path over one frame of synthetic input (BASELINE config 3: 2 M points
on 200 planes/spheres, 1920x1080, 4 layers, K=16, gradients to descriptors, confidence and xyz). Inputs, outputs and
the workspace are resident in HBM before the timed region starts. After --warmup untimed steps, --samples groups of
--steps steps are timed with HIP events on the launch stream; `value` is the median over the groups (p10/p90 beside
it). Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--samples S] [--config 2|3|4|5] [--render-mode 1|2|3]
                  [--point-order vet_preprocess|generated|grown] [--no-cpu-baseline] [--no-second-order]
"""
import argparse
import ctypes as C
import glob
import hashlib
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
TRAFFIC_FILES = {1: os.path.join(ROOT, "profiles", "hbm_traffic_config3.md"),
                 3: os.path.join(ROOT, "profiles", "hbm_traffic_config3_bilinear.md")}


def algorithmic_bytes(N, P, F, Fk, Cn, render_mode=1):
    """Compulsory bytes per kernel, each datum counted once per producer and once per consumer (4-byte scalars), summed
    over the views: N = points x views, P = pixels of all layers x views, F fragments, Fk fragments that were blended.

    FULL_BLEND / FUZZY_BLEND: B_fwd = 32N + 36P + 24F + 28Fk, B_bwd = 32P + 116Fk + 40N for C = 4.
    BILINEAR_BLEND adds the 16-byte side record (point id, u, v, corner) the reference writes per fragment in its
    collection pass (src/lib/rendering/RenderForward.cu:1011-1137) and reads per blended fragment in the blend and in
    the backward kernel (RenderBackward.cu:2911-2931): B_fwd = 32N + 36P + 40F + 44Fk, B_bwd = 32P + 132Fk + 40N.
    """
    side = 16 if render_mode == 3 else 0
    fwd = {
        # one pass over the points projects them, counts the bins and writes the fragment records (the model reads the
        # positions twice, as the reference's two passes do; both reads are booked here)
        "COUNT": 32 * N + (8 + side) * F,
        "FILL": 0,                                    # files the few records that overflow a bin's own room
        # per-pixel counts, counts -> offsets, records read and written sorted; then the blend: lists, side record,
        # descriptor + confidence, offsets, out, weight
        "BUILD": 4 * P + 8 * P + 16 * F + (8 + side) * Fk + (4 * Cn + 4) * Fk + 4 * P + 4 * Cn * P + 4 * P,
    }
    # The per-pixel kernel reads upstream grads and forward outputs (8CP), lists (8Fk), descriptor+confidence (4(C+1)Fk)
    # and writes one half of the gradient read-modify-write (4(C+1+4)Fk); the per-point kernel reads positions (16Fk in the
    # model), that half back, and writes the gradient rows (4(C+1+4+1)N, the term the reference spends on zero-filling).
    rmw_half = 4 * (Cn + 1 + 4) * Fk
    bwd = {
        "BACKWARD_BLEND": 8 * Cn * P + (8 + side) * Fk + (4 * Cn + 4) * Fk + rmw_half,
        "BACKWARD_GATHER": 16 * Fk + rmw_half + 4 * (Cn + 1 + 4 + 1) * N,
    }
    return fwd, bwd


def kernel_sources_digest():
    """sha256 over the kernel sources the library is built from; a counter profile records the digest of the sources it
    measured, and its figures are only attached to a bench line of the same sources."""
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(ROOT, "vet_amd", "csrc", "*"))):
        if path.endswith((".h", ".hip")):
            h.update(os.path.basename(path).encode())
            h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(render_mode):
    """HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, read from the committed summary
    (rows `| SCOPE | fetch KiB | write KiB |`, already scaled by the copy-kernel calibration).
    Returns (bytes per scope, provenance); the first is empty when there is no summary or when the summary was taken
    from other kernel sources than the ones in the tree."""
    path = TRAFFIC_FILES.get(render_mode)
    if not path or not os.path.exists(path):
        return {}, {"profile": None, "state": "no counter profile for this workload"}
    text = open(path).read()
    m = re.search(r"kernel sources digest:\s*`?([0-9a-f]{16})`?", text)
    k = re.search(r"kernels:\s*(.+)", text)
    src = {"profile": os.path.relpath(path, ROOT), "profile_sources_digest": m.group(1) if m else None,
           "tree_sources_digest": kernel_sources_digest(),
           "kernels": [s.strip(" `") for s in k.group(1).split(";")] if k else None}
    if not m or m.group(1) != src["tree_sources_digest"]:
        src["state"] = "stale: the profile was taken from other kernel sources; traffic withheld"
        return {}, src
    src["state"] = "current"
    res = {}
    in_table = False
    for line in text.splitlines():
        if line.startswith("## "):
            in_table = line.startswith("## Per scope")
        if not in_table:
            continue
        mm = re.match(r"^\|\s*([A-Z_]+)\s*\|\s*([0-9.]+)\s*\|\s*([0-9.]+)\s*\|", line)
        if mm:
            res[mm.group(1)] = (float(mm.group(2)) + float(mm.group(3))) * 1024.0
    return res, src


def timed_samples(fn, warmup, steps, samples):
    """`warmup` untimed calls, then `samples` groups of `steps` calls, each group bracketed by HIP events recorded on the
    stream the kernels are launched on. Returns ms per call: dict(median, p10, p90, samples, wall)."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(samples)]
    t0 = time.perf_counter()
    for a, b in pairs:
        a.record()
        for _ in range(steps):
            fn()
        b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / (steps * samples)
    ms = sorted(a.elapsed_time(b) / steps for a, b in pairs)
    return {"median": float(np.median(ms)), "p10": float(np.percentile(ms, 10)), "p90": float(np.percentile(ms, 90)),
            "samples": [round(x, 5) for x in ms], "wall": wall}


def run_scene(scene, backward, steps, warmup, samples, profile=True, render_mode=1, graph=False, processing_order=False,
              **param_overrides):
    """processing_order: hand the library a Morton order built on the device (vetrast_forward_args.point_order), as
    the shim does for every cloud; its build time is reported, not part of the step."""
    import torch

    from vet_amd import abi
    from vet_amd.rasterizer import DeviceScene, Rasterizer, make_params

    params = make_params(scene, need_point_gradient=1 if backward else 0, render_mode=render_mode, **param_overrides)
    N, Cn, L, B = scene.num_points, scene.num_channels, scene.num_layers, len(scene.views)
    rast = Rasterizer()
    dev = DeviceScene(scene)
    lay = rast.layout(scene, render_mode)
    workspace = torch.empty(lay.total_bytes, dtype=torch.uint8, device="cuda")
    out = [torch.empty((B, Cn, h, w), dtype=torch.float32, device="cuda") for (w, h) in scene.layer_sizes()]
    order, order_ms = None, None
    if processing_order:
        from vet_amd import torch_ops

        d_pos = torch.from_numpy(scene.position).cuda()
        order_ms = timed_samples(lambda: torch_ops.processing_order_on_device(d_pos), 2, 5, 3)["median"]
        order = torch_ops.processing_order_on_device(d_pos)
    fwd = rast.forward(dev, params, save_for_backward=backward, workspace=workspace, out=out, point_order=order)
    torch.cuda.synchronize()
    P = fwd.total_pixels()
    K = params.debug_max_list_length
    bases = fwd.layer_bases()
    F, Fk, F_layers = 0, 0, [0] * L
    for b in range(B):
        off = fwd.offsets(b)
        F += int(off[-1])
        Fk += int(fwd.kept(b).sum())  # fragments that took part in the blend (top-K cut, in mode 3 also saturation)
        for l in range(L):
            F_layers[l] += int(off[bases[l + 1]] - off[bases[l]])

    bargs = None
    if backward:
        grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
        first = rast.backward(fwd, grad_out)  # allocates the gradient tensors once; reused below
        bargs = first["_args"]
    lib, ctx = rast.lib, rast.ctx

    def forward_only(stream=None):
        s = stream or C.c_void_p(torch.cuda.current_stream().cuda_stream)
        abi.check(lib.vetrast_forward(ctx, C.byref(fwd.args), s), "forward")

    def step(stream=None):
        s = stream or C.c_void_p(torch.cuda.current_stream().cuda_stream)
        abi.check(lib.vetrast_forward(ctx, C.byref(fwd.args), s), "forward")
        if backward:
            abi.check(lib.vetrast_backward(ctx, C.byref(bargs), s), "backward")

    t_step = timed_samples(step, warmup, steps, samples)
    t_fwd = timed_samples(forward_only, 2, steps, samples) if backward else t_step
    res = {"step": t_step, "fwd": t_fwd, "ms_step": t_step["median"], "ms_fwd": t_fwd["median"],
           "workspace_bytes": int(lay.total_bytes), "order_build_ms": order_ms}
    res.update(N=N, P=P, F=F, Fk=Fk, F_layers=F_layers, K=K, Cn=Cn, L=L, B=B, params=params)
    if graph:
        # The same step with descriptor records the caller keeps current (vetrast_pack_descriptors): what a viewer or
        # an evaluation loop pays per frame while the texture stands still. Reported beside the headline, never as it:
        # the headline call is self-contained.
        packed = rast.pack_descriptors(dev, params)
        kept_args = abi.ForwardArgs()
        C.memmove(C.byref(kept_args), C.byref(fwd.args), C.sizeof(abi.ForwardArgs))
        kept_args.packed_descriptors = packed.data_ptr()
        kept_bargs = None
        if backward:
            kept_bargs = abi.BackwardArgs()
            C.memmove(C.byref(kept_bargs), C.byref(bargs), C.sizeof(abi.BackwardArgs))
            kept_bargs.fwd.packed_descriptors = packed.data_ptr()

        def kept_forward():
            abi.check(lib.vetrast_forward(ctx, C.byref(kept_args), C.c_void_p(torch.cuda.current_stream().cuda_stream)),
                      "forward")

        def kept_step():
            kept_forward()
            if backward:
                abi.check(lib.vetrast_backward(ctx, C.byref(kept_bargs),
                                               C.c_void_p(torch.cuda.current_stream().cuda_stream)), "backward")

        res["kept_descriptors"] = {
            "ms_per_step": round(timed_samples(kept_step, 3, steps, samples)["median"], 5),
            "plain_step_timed_right_after_ms": round(timed_samples(step, 3, steps, samples)["median"], 5),
            "forward_ms": round(timed_samples(kept_forward, 3, steps, samples)["median"], 5),
            "pack_ms": round(timed_samples(lambda: rast.pack_descriptors(dev, params, out=packed), 3, steps, samples)["median"], 5),
            "what": "the same step with vetrast_forward_args.packed_descriptors set (records written once by "
                    "vetrast_pack_descriptors, pack_ms, outside the step): not the headline",
        }
        del packed
    if graph:
        # the same step replayed from a HIP graph: no launch calls from the host between the kernels
        side = torch.cuda.Stream()
        g = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                step(C.c_void_p(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        res["graph"] = timed_samples(g.replay, 3, steps, samples)
        del g
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
        res["launches_per_step"] = {k: n / prof_steps for k, (ms, n) in scopes.items()}
    del workspace, out, fwd
    torch.cuda.empty_cache()
    return res


def time_fused_steps(scene, render_mode, steps, samples):
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

    def frame():
        abi.check(rast.lib.vetrast_forward(rast.ctx, C.byref(fwd.args), stream), "forward")
        abi.check(rast.lib.vetrast_backward(rast.ctx, C.byref(bargs), stream), "backward")

    ms_frame = timed_samples(frame, 3, steps, samples)["median"]
    n = (scene.num_channels + 1) * scene.num_points + scene.num_channels
    p, g, m, v = (torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(4))
    g.normal_()
    state = {"step": 0}

    def adam():
        state["step"] += 1
        rast.adam_step(p, g, m, v, state["step"], 1e-3)

    ms_adam = timed_samples(adam, 3, steps, samples)["median"]
    adam_bytes = 28.0 * n  # param, grad, two moments read; param and moments written
    return {"frame_with_fused_sigmoid_abs_ms": round(ms_frame, 5), "adam_step_ms": round(ms_adam, 5),
            "adam_elements": n, "adam_GBps": round(adam_bytes / 1e6 / ms_adam, 1),
            "adam_frac_of_hbm_peak": round(adam_bytes / 1e6 / ms_adam / HBM_PEAK_GBS, 4)}


def time_shim_path(scene, render_mode, steps, samples, **overrides):
    """The same frame through the libtorch shim as a trainer calls it: BlendPointCloud with train = true, then
    autograd's backward with the upstream gradients; workspace and output allocation, the autograd graph and the
    gradient tensors torch allocates are all inside the timed region. `overrides`: RenderParams members by name."""
    import torch

    from vet_amd import torch_ops

    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    texture, background = cu(scene.texture, True), cu(scene.background, True)
    points, confidence = cu(scene.position, True), cu(scene.confidence.reshape(1, -1), True)
    tangents = torch.zeros((scene.poses_se3.shape[0], 6), dtype=torch.float64, device="cuda")
    intrinsics, poses = cu(scene.intrinsics), cu(scene.poses_se3)
    index = None if scene.index is None else cu(scene.index)
    views = [(v.w, v.h, v.image_index, v.camera_index, v.camera_model_type, *v.crop_transform, *v.crop_rotation)
             for v in scene.views]
    grads = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    leaves = (texture, background, points, confidence)

    def step():
        for t in leaves:
            t.grad = None
        kw = dict(train=True, use_environment_map=0, need_point_gradient=1, drop_out_points_by_radius=0,
                  debug_max_list_length=scene.max_list_length, render_mode=render_mode)
        kw.update(overrides)
        outs = torch_ops.blend_point_cloud(texture, background, points, tangents, intrinsics, confidence, poses, index,
                                           views, scene.num_layers, **kw)
        torch.autograd.backward(outs[:scene.num_layers], grads)

    for _ in range(40):  # (the cache reads the fragment counts of a call back every 16th call and sizes bins from them)
        step()
    t = timed_samples(step, 3, steps, samples)
    _, ws_bytes = torch_ops.train_workspace_info()
    return {"ms_per_step": round(t["median"], 5), "p10": round(t["p10"], 5), "p90": round(t["p90"], 5),
            "workspace_bytes_kept_between_steps": int(ws_bytes),
            "what": "torch_ops.blend_point_cloud(train=True) + torch.autograd.backward, allocations included"}


def time_lift_error(scene, steps, cpu_threads):
    """Error lifting (vetrast_lift_error; the reference's FillSceneGridWithLoss), the step that runs once per view in the
    epoch before VET adds points: the scene's grid at 0.25 m under the scene's own camera and a synthetic 3-channel
    error image. Reported beside the headline number, not part of it; the CPU oracle is timed on the same call."""
    import torch

    from vet_amd import abi, synthetic
    from vet_amd.rasterizer import Rasterizer

    rast = Rasterizer()
    # 0.25 m cells; a scene whose box would need more than four million of them (config 4's outdoor scene: the grid is
    # built on the host) gets cells twice as large until it does not
    cell_size = 0.25
    xyz = scene.position[:, :3]
    extent = (xyz.max(axis=0) - xyz.min(axis=0)).astype(np.float64) + 0.02
    while float(np.prod(np.ceil(extent / cell_size))) > 4e6:
        cell_size *= 2.0
    mn, ln = synthetic.cell_grid(xyz, cell_size)
    view = scene.views[0]
    img = synthetic.error_image(5, 3, view.h, view.w)
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    d_mn, d_ln, d_img, d_pose, d_intr = (to_dev(a) for a in (mn, ln, img, scene.poses_se3, scene.intrinsics))
    val = torch.zeros(len(mn), dtype=torch.float32, device="cuda")
    cnt = torch.zeros(len(mn), dtype=torch.int32, device="cuda")
    ws = rast.lift_error(d_mn, d_ln, val, cnt, view, d_pose, d_intr, d_img)
    torch.cuda.synchronize()
    pixels = int(cnt.sum().item())
    queued = int(ws[abi.LIFT_QUEUE_LENGTH_OFFSET:abi.LIFT_QUEUE_LENGTH_OFFSET + 4].view(torch.int32).item())
    calls = [1]

    def call():
        calls[0] += 1
        rast.lift_error(d_mn, d_ln, val, cnt, view, d_pose, d_intr, d_img, workspace=ws)

    ms = timed_samples(call, 3, steps, 3)["median"]
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
        out["counts_equal_cpu_oracle"] = bool(np.array_equal(c, cnt.cpu().numpy() // calls[0]))
    return out


def time_training_crops(steps, samples, render_mode):
    """A batch as VET trains on it (configs/config.ini: batch_size 4, train_crop_size 512, no list cut, radius drop-out):
    four 512x512 crops out of config 3's frame, radii spread log-normally. Timed without and with
    vetrast_params.expected_fragments set to the per-layer fragment counts of the call before (what the shim does)."""
    import torch

    from vet_amd import abi, synthetic
    from vet_amd.rasterizer import DeviceScene, Rasterizer, make_params

    scene = synthetic.config3(radius_spread=0.5, K=-1)
    scene.views = [synthetic.ViewSpec(512, 512, image_index=0, crop_transform=(1.0, 1.0, -float(ox), -float(oy), 0.0))
                   for (ox, oy) in ((200, 100), (900, 300), (1300, 500), (600, 560))]
    rast = Rasterizer()
    dev = DeviceScene(scene)
    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {"what": "4 crops of 512x512 of config 3's frame in one call, K = -1, drop_out_points_by_radius, "
                   "forward+backward, ms per batch", "render_mode": render_mode}
    hint = [0.0] * 5
    for name in ("ms_per_batch", "ms_per_batch_with_expected_fragments"):
        params = make_params(scene, need_point_gradient=1, render_mode=render_mode, drop_out_points_by_radius=1,
                             expected_fragments=hint)
        fwd = rast.forward(dev, params)
        bargs = rast.backward(fwd, grad_out)["_args"]

        def step():
            abi.check(rast.lib.vetrast_forward(rast.ctx, C.byref(fwd.args), stream), "forward")
            abi.check(rast.lib.vetrast_backward(rast.ctx, C.byref(bargs), stream), "backward")

        out[name] = round(timed_samples(step, 3, steps, samples)["median"], 5)
        off, bases = fwd.offsets(0), fwd.layer_bases()
        counts = [int(off[bases[l + 1]] - off[bases[l]]) for l in range(scene.num_layers)]
        out["fragments_per_layer_of_view_0"] = counts
        hint = [float(c) for c in counts] + [0.0] * (5 - len(counts))
        del fwd, bargs
    del dev
    torch.cuda.empty_cache()
    # the same batch as a trainer issues it: through the libtorch shim, which sizes the bins from its own history
    out["ms_per_batch_through_the_shim"] = time_shim_path(scene, render_mode, steps, samples, drop_out_points_by_radius=1,
                                                          debug_max_list_length=-1)["ms_per_step"]
    return out


def host_threads(requested):
    """Threads for the CPU legs: every core this process may run on, within the worker limit the box sets for a job
    (OMP_NUM_THREADS where the environment has it). Returns (threads, cores visible, limit or None)."""
    visible = len(os.sched_getaffinity(0))
    limit = os.environ.get("OMP_NUM_THREADS")
    limit = int(limit) if limit and limit.isdigit() else None
    if requested:
        return requested, visible, limit
    return (min(visible, limit) if limit else visible), visible, limit


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--samples", type=int, default=5, help="timed groups of --steps steps (median, p10, p90 over them)")
    ap.add_argument("--config", type=int, default=3, choices=[2, 3, 4, 5])
    ap.add_argument("--points", type=int, default=None, help="override the point count (debug runs)")
    ap.add_argument("--point-order", default="vet_preprocess", choices=["vet_preprocess", "generated", "grown"])
    ap.add_argument("--render-mode", type=int, default=1, choices=[1, 2, 3],
                    help="1 = FULL_BLEND (the headline workload), 3 = BILINEAR_BLEND (four fragments per point and layer)")
    ap.add_argument("--no-second-order", action="store_true",
                    help="skip everything beside the headline: the other point orders, the graph replay, the fused "
                         "steps, the shim path, the error lifting")
    ap.add_argument("--no-other-order", action="store_true", help="skip timing the other point orders only")
    ap.add_argument("--calibration-kernel", action="store_true",
                    help="also run the Adam kernel a few times: a streaming kernel that reads 16 and writes 12 bytes per "
                         "element, against which byte counters of a profiler run are scaled")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--lift-only", action="store_true",
                    help="time only the error lifting on the configuration's scene and print its object")
    ap.add_argument("--cpu-threads", type=int, default=0,
                    help="0 = every core this process may use, within the box's worker limit (OMP_NUM_THREADS)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the rasterizer on ONE GPU (the views of a batch share it); "
              "--gpus N with N > 1 is not available", file=sys.stderr)
        sys.exit(2)

    import torch

    from vet_amd import synthetic

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path in the product)", file=sys.stderr)
        sys.exit(2)

    make = {2: synthetic.config2, 3: synthetic.config3, 4: synthetic.config4, 5: synthetic.config5}[args.config]
    kw = {"point_order": args.point_order}
    if args.points is not None:
        kw["surface_points_n" if args.config == 4 else "num_points"] = args.points
    backward = args.config != 2
    scene = make(**kw)
    cpu_threads, cores_visible, cores_limit = host_threads(args.cpu_threads)
    if args.lift_only:
        print(json.dumps({"lift_error": time_lift_error(scene, args.steps, 0 if args.no_cpu_baseline else cpu_threads)}))
        return
    extras = not args.no_second_order
    r = run_scene(scene, backward, args.steps, args.warmup, args.samples, render_mode=args.render_mode, graph=extras)
    N, P, F, Fk, Cn, L, K, B = r["N"], r["P"], r["F"], r["Fk"], r["Cn"], r["L"], r["K"], r["B"]
    ms_step, ms_fwd = r["ms_step"], r["ms_fwd"]

    fwd_b, bwd_b = algorithmic_bytes(N * B, P * B, F, Fk, Cn, args.render_mode)
    alg = dict(fwd_b)
    if backward:
        alg.update(bwd_b)
    headline_workload = (args.config == 3 and args.points is None and args.point_order == "vet_preprocess")
    traffic, traffic_source = measured_traffic(args.render_mode) if headline_workload else \
        ({}, {"profile": None, "state": "no counter profile for this workload"})
    kernels = {}
    for k, nbytes in alg.items():
        t = r["per_step_ms"].get(k, 0.0)
        kernels[k] = {"ms": round(t, 5), "alg_MB": round(nbytes / 1e6, 3),
                      "GBps": round(nbytes / 1e6 / t, 1) if t > 0 else None,
                      "frac": round(nbytes / 1e6 / t / HBM_PEAK_GBS, 4) if t > 0 else None}
        if k in traffic:
            kernels[k]["hbm_traffic_MB"] = round(traffic[k] * B / 1e6, 1)
    for k in ("PREPARE", "PACK", "SCAN", "BACKWARD_PREPARE", "BACKWARD_POST"):
        if r["per_step_ms"].get(k, 0.0) > 0:
            kernels[k] = {"ms": round(r["per_step_ms"][k], 5), "alg_MB": 0.0, "GBps": None, "frac": None}
    dominant = max(alg.keys(), key=lambda k: r["per_step_ms"].get(k, 0.0))
    dom_ms = r["per_launch_ms"][dominant]
    dom_launches = max(1.0, r["launches_per_step"].get(dominant, 1.0))
    dom_bytes = alg[dominant] / dom_launches  # (one launch takes up to four views of a call)
    achieved = dom_bytes / 1e6 / dom_ms if dom_ms > 0 else 0.0
    total_alg = sum(alg.values())

    view0 = scene.views[0]
    if backward:
        metric = f"fwd+bwd ms/frame (1080p, {N / 1e6:g}M pts, {L} layers" + (f", {B} views)" if B > 1 else ")")
    else:
        metric = f"fwd ms/frame (1080p, {N / 1e6:g}M pts, {L} layers)"
    if args.config == 3 and args.points is None:
        metric = "fwd+bwd ms/frame (1080p, 2M pts, 4 layers)"
    if args.config == 2 and args.points is None:
        metric = "fwd ms/frame (1080p, 2M pts, 4 layers)"
    result = {
        "metric": metric,
        "value": round(ms_step, 5),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "samples": args.samples,
        "ms_per_step": round(ms_step, 5),
        "ms_per_step_p10": round(r["step"]["p10"], 5),
        "ms_per_step_p90": round(r["step"]["p90"], 5),
        "ms_per_step_samples": r["step"]["samples"],
        "ms_per_step_host_clock": round(r["step"]["wall"], 5),
        "timing": f"median over {args.samples} groups of {args.steps} steps, HIP events on the launch stream, "
                  f"{args.warmup} warm-up steps before; host clock over all groups beside it",
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"BASELINE config {args.config} ({scene.name}): N={N} points, {view0.w}x{view0.h}, "
                        f"L={L} layers, K={K}, C={Cn}, B={B} view" + ("s" if B > 1 else "") + ", "
                        + ("forward+backward" if backward else "forward")
                        + f", point order {args.point_order}"
                        + {1: ", render_mode 1 (FULL_BLEND)", 2: ", render_mode 2 (FUZZY_BLEND, depth_accept_blend 0.01)",
                           3: ", render_mode 3 (BILINEAR_BLEND)"}[args.render_mode],
            "point_order": args.point_order, "render_mode": args.render_mode, "views": B,
            "fragments_per_layer": r["F_layers"], "fragments": F, "fragments_kept": Fk, "pixels": P * B,
            "workspace_MB": round(r["workspace_bytes"] / 1e6, 1),
        },
        "forward_ms": round(ms_fwd, 5),
        "backward_ms": round(ms_step - ms_fwd, 5) if backward else None,
        "kernels_note": ("the byte model counts every view's pass over the point arrays; the per-point backward kernel "
                         "takes the (up to four) views of a launch in one pass over them, so its rate against the model can "
                         "exceed what the memory delivers") if B > 1 else None,
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
            "traffic_source": traffic_source,
            "avg_launch_ms": round(dom_ms, 5),
            "algorithmic_bytes_per_launch": int(dom_bytes),
        },
        "kernels": kernels,
    }
    if "graph" in r:
        g = r["graph"]
        result["graph_replay"] = {"ms_per_step": round(g["median"], 5), "p10": round(g["p10"], 5),
                                  "p90": round(g["p90"], 5),
                                  "step_frac_of_hbm_peak": round(total_alg / 1e6 / g["median"] / HBM_PEAK_GBS, 4),
                                  "what": "the same forward+backward step captured once in a HIP graph and replayed"}

    if "kept_descriptors" in r:
        result["kept_descriptors"] = r["kept_descriptors"]

    if extras and not args.no_other_order:
        # VET hands the rasterizer Morton-ordered clouds with shuffled 256-point blocks (sorted by radius inside the
        # blocks) and appends new points unsorted while it trains; the generator's raw order is the worst case.
        others = []
        short = dict(steps=max(10, args.steps // 2), warmup=5, samples=3, profile=False, render_mode=args.render_mode)
        for order in ("vet_preprocess", "grown", "generated"):
            if order == args.point_order:
                continue
            sc2 = make(**dict(kw, point_order=order))
            r2 = run_scene(sc2, backward, **short)
            r2o = run_scene(sc2, backward, processing_order=True, **short)
            others.append({"point_order": order, "ms_per_step": round(r2["ms_step"], 5),
                           "forward_ms": round(r2["ms_fwd"], 5),
                           "with_processing_order": {"ms_per_step": round(r2o["ms_step"], 5),
                                                     "forward_ms": round(r2o["ms_fwd"], 5)}})
        result["other_point_orders"] = others
        r1o = run_scene(scene, backward, processing_order=True, **short)
        result["processing_order"] = {
            "what": "vetrast_forward_args.point_order = Morton order with shuffled 256-point blocks, built on the "
                    "device by the shim (ProcessingOrderOnDevice) once per 1000 forward calls; results are the same bits",
            "build_ms": round(r1o["order_build_ms"], 4),
            "headline_order_ms_per_step": round(r1o["ms_step"], 5), "headline_order_forward_ms": round(r1o["ms_fwd"], 5)}
        if args.config in (2, 3):
            # log-normal radii, blocks sorted by radius as SortBlocksByRadius(256) leaves them, radius drop-out on
            sc = make(**dict(kw, radius_spread=0.5))
            r3 = run_scene(sc, backward, drop_out_points_by_radius=1, **short)
            result["radius_dropout"] = {"point_order": args.point_order, "radius_spread": 0.5,
                                        "drop_out_radius_threshold": 0.6, "ms_per_step": round(r3["ms_step"], 5),
                                        "forward_ms": round(r3["ms_fwd"], 5), "fragments": r3["F"],
                                        "fragments_per_layer": r3["F_layers"]}

    if backward and extras:
        result["fused_steps"] = time_fused_steps(scene, args.render_mode, max(10, args.steps // 2), 3)
        result["shim_path"] = time_shim_path(scene, args.render_mode, max(10, args.steps // 2), 3)
    if args.calibration_kernel:
        from vet_amd.rasterizer import Rasterizer

        n = (scene.num_channels + 1) * scene.num_points + scene.num_channels
        p_, g_, m_, v_ = (torch.zeros(n, dtype=torch.float32, device="cuda") for _ in range(4))
        rast_c = Rasterizer()
        for k in range(3):
            rast_c.adam_step(p_, g_, m_, v_, k + 1, 1e-3)
        torch.cuda.synchronize()
        result["calibration_kernel"] = {"kernel": "adam_step_kernel", "elements": n, "read_bytes": 16 * n,
                                        "write_bytes": 12 * n}

    if extras and backward and args.config == 3:
        result["training_crops"] = time_training_crops(max(10, args.steps // 2), 3, args.render_mode)
        if args.render_mode == 1:
            # the same batch in the mode VET's shipped configuration trains in
            result["training_crops_bilinear"] = time_training_crops(max(10, args.steps // 2), 3, 3)
    if extras:
        result["lift_error"] = time_lift_error(scene, max(10, args.steps // 2), 0 if args.no_cpu_baseline else cpu_threads)

    if not args.no_cpu_baseline:
        from oracle import oracle_py

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

        ladder = sorted({t for t in (1, 2, 4, 8, 16, 32, 64, 128, 256) if t < cpu_threads} | {cpu_threads})
        by_threads = {}
        for t in ladder:
            runs = [cpu_step(t) for _ in range(1 if t == 1 else 3)]
            by_threads[t] = (float(np.median([x[0] for x in runs])), float(np.median([x[1] for x in runs])))
        multi_ms, multi_fwd = by_threads[cpu_threads]
        result["cpu_baseline"] = {
            "value": round(multi_ms, 2),
            "unit": "ms",
            "cores": cpu_threads,
            "kind": "port",
            "sample": f"the same frame (config {args.config}, all {N} points): CPU oracle, median of 3 runs on "
                      f"{cpu_threads} threads = every core a job may use on this box ({cores_visible} cores visible to "
                      f"the process, worker limit {cores_limit}); one run on 1 thread = {by_threads[1][0]:.1f} ms. "
                      f"The threaded oracle is bound by its atomics: its backward pass adds every fragment's gradient "
                      f"with an OpenMP atomic, as the reference's kernel does with a CUDA atomic, so it hardly scales "
                      f"with threads (ms_by_threads); only its forward pass ({multi_fwd:.0f} ms on {cpu_threads} "
                      f"threads) does",
            "single_thread_ms": round(by_threads[1][0], 2),
            "forward_ms": round(multi_fwd, 2),
            "cores_visible": cores_visible,
            "worker_limit": cores_limit,
            "ms_by_threads": {str(t): round(v[0], 2) for t, v in by_threads.items()},
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
