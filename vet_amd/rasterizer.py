"""Thin Python host over the C ABI (include/vetrast.h), with torch used only for device memory and streams.

This is what tests and bench.py drive. It adds no arithmetic of its own and has no CPU path: without a GPU and the
built HIP library every call raises.
"""
import ctypes as C
from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import torch

from . import abi
from .synthetic import Scene


def make_params(scene: Scene, **overrides) -> abi.Params:
    """RenderParams of the blending path with the defaults the benchmark configurations use."""
    p = abi.Params()
    p.num_texture_channels = scene.num_channels
    p.num_layers = scene.num_layers
    p.debug_max_list_length = scene.max_list_length
    p.use_environment_map = 0
    p.need_point_gradient = 0
    p.viewer_only = 0
    p.stability_cutoff_value = 10000.0
    p.drop_out_points_by_radius = 0
    p.drop_out_radius_threshold = 0.6
    p.output_background_mask = 0
    p.output_background_mask_value = 0.0
    p.check_normal = 0
    p.quirk_background_confidence_leak = 0
    p.point_gradient_normalization = 0
    p.K_gradient_factor = 0.5
    p.camera_gradient_normalization = 0
    p.render_mode = abi.RENDER_FULL_BLEND
    p.confidence_activation = 0
    p.confidence_scale = 10.0
    p.texture_abs = 0
    p.depth_accept_blend = 0.01
    p.allow_distortion = 0
    p.distortion_gradient_factor = 0.005
    for k, v in {**scene.params, **overrides}.items():
        if not hasattr(p, k):
            raise AttributeError(f"vetrast_params has no field {k}")
        if k == "expected_fragments":
            for l, x in enumerate(v):
                p.expected_fragments[l] = float(x)
            continue
        setattr(p, k, v)
    return p


def make_views(scene: Scene):
    arr = (abi.View * len(scene.views))()
    for i, v in enumerate(scene.views):
        arr[i].w, arr[i].h = v.w, v.h
        arr[i].image_index, arr[i].camera_index = v.image_index, v.camera_index
        arr[i].camera_model_type = v.camera_model_type
        arr[i].crop_transform = (C.c_float * 5)(*v.crop_transform)
        arr[i].crop_rotation = (C.c_float * 4)(*v.crop_rotation)
    return arr


def fill_forward_args(args: abi.ForwardArgs, scene: Scene, params: abi.Params, views, ptr):
    """Common part for host (oracle) and device callers; `ptr(name)` returns the address of an input array or None."""
    args.num_points = scene.num_points
    args.num_views = len(scene.views)
    args.num_poses = int(scene.poses_se3.shape[0])
    args.num_cameras = int(scene.intrinsics.shape[0])
    for name in ("position", "index", "texture", "confidence", "background", "dropout", "poses_se3", "intrinsics"):
        setattr(args, name, ptr(name))
    args.views = views
    args.params = params


def fill_lift_args(a, view, poses_se3, intrinsics, loss_image, border_pixels):
    """Scalar part of vetrast_lift_args shared by host and device callers; `view` is a synthetic.View."""
    a.num_poses, a.num_cameras = int(poses_se3.shape[0]), int(intrinsics.shape[0])
    a.view.w, a.view.h = view.w, view.h
    a.view.image_index, a.view.camera_index = view.image_index, view.camera_index
    a.view.camera_model_type = view.camera_model_type
    a.view.crop_transform = (C.c_float * 5)(*view.crop_transform)
    a.view.crop_rotation = (C.c_float * 4)(*view.crop_rotation)
    a.channels, a.height, a.width = (int(d) for d in loss_image.shape)
    a.border_pixels = border_pixels


@dataclass
class ForwardResult:
    out: List[torch.Tensor]
    out_mask: List[Optional[torch.Tensor]]
    workspace: torch.Tensor
    layout: abi.WorkspaceLayout
    args: abi.ForwardArgs
    keep: tuple  # objects that must outlive `args`
    out_weight: Optional[List[torch.Tensor]] = None  # [B,1,h,w] per layer, only with want_weight

    def _view_array(self, base, stride, b, dtype, count):
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        raw = self.workspace[base + stride * b: base + stride * b + nbytes]
        return raw.view(dtype)

    # The workspace numbers pixels tile by tile (16x16 tiles, see include/vetrast.h). The accessors below hand the lists
    # back in image order instead: layer after layer, row-major inside a layer, which is the order a reader expects and
    # the order the CPU check uses.
    def num_layers(self):
        return int(self.args.params.num_layers)

    def layer_bases(self):
        """Image-order pixel number of the first pixel of every layer, plus the total."""
        lay, run, bases = self.layout, 0, []
        for l in range(self.num_layers()):
            bases.append(run)
            run += int(lay.layer_w[l]) * int(lay.layer_h[l])
        return bases + [run]

    def total_pixels(self):
        return self.layer_bases()[-1]

    def device_pixels(self):
        return int(self.layout.layer_pixel_base[self.num_layers()])

    def pixel_map(self):
        """int64 [total_pixels]: workspace pixel number of every image-order pixel."""
        if getattr(self, "_pixel_map", None) is None:
            lay, parts = self.layout, []
            for l in range(self.num_layers()):
                w, h = int(lay.layer_w[l]), int(lay.layer_h[l])
                y, x = np.meshgrid(np.arange(h, dtype=np.int64), np.arange(w, dtype=np.int64), indexing="ij")
                tile = int(lay.layer_tile_base[l]) + (y // 16) * int(lay.layer_tiles_x[l]) + x // 16
                parts.append((tile * 256 + (y % 16) * 16 + x % 16).reshape(-1))
            self._pixel_map = np.concatenate(parts)
        return self._pixel_map

    def device_offsets(self, b=0):
        """int64 numpy copy of the list starts [device_pixels + 1] of view b, in workspace pixel order."""
        t = self._view_array(self.layout.offsets_base, self.layout.offsets_stride, b, torch.int32,
                             self.device_pixels() + 1)
        return t.cpu().numpy().astype(np.int64) & 0xFFFFFFFF

    def _gather_index(self, b):
        """(image-order exclusive scan [P+1], workspace position of every fragment in image order)."""
        dev = self.device_offsets(b)
        m = self.pixel_map()
        counts = dev[m + 1] - dev[m]
        off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
        src = np.repeat(dev[m] - off[:-1], counts) + np.arange(off[-1], dtype=np.int64)
        return off, src

    def offsets(self, b=0):
        """int64 exclusive scan [P+1] of the per-pixel fragment counts of view b, image order."""
        return self._gather_index(b)[0]

    def fragments(self, b=0):
        """uint64 fragment keys of view b, the lists concatenated in image order."""
        _, src = self._gather_index(b)
        t = self._view_array(self.layout.fragments_base, self.layout.fragments_stride, b, torch.int64,
                             int(self.layout.fragment_capacity))
        return t.cpu().numpy().view(np.uint64)[src]

    def transmittance(self, b=0):
        _, src = self._gather_index(b)
        t = self._view_array(self.layout.transmittance_base, self.layout.transmittance_stride, b, torch.float32,
                             int(self.layout.fragment_capacity))
        return t.cpu().numpy()[src]

    def kept(self, b=0):
        """int64 [total_pixels]: fragments of every pixel's list that took part in the blend, image order."""
        if int(self.args.params.render_mode) != abi.RENDER_BILINEAR_BLEND:  # not stored: min(count, K)
            counts, K = np.diff(self.offsets(b)), int(self.args.params.debug_max_list_length)
            return np.minimum(counts, K) if K > 0 else counts
        t = self._view_array(self.layout.kept_base, self.layout.kept_stride, b, torch.int32, self.device_pixels())
        return t.cpu().numpy().astype(np.int64)[self.pixel_map()]

    def weight(self, b=0):
        t = self._view_array(self.layout.weight_base, self.layout.weight_stride, b, torch.float32,
                             self.device_pixels())
        return t.cpu().numpy()[self.pixel_map()]


class DeviceScene:
    """Inputs of a Scene as torch tensors on the GPU."""

    def __init__(self, scene: Scene, device="cuda:0"):
        self.scene = scene
        self.device = torch.device(device)
        f = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(self.device)
        self.position = f(scene.position)
        self.index = f(scene.index)
        self.texture = f(scene.texture)
        self.confidence = f(scene.confidence)
        self.background = f(scene.background)
        self.dropout = f(scene.dropout)
        self.poses_se3 = f(scene.poses_se3)
        self.intrinsics = f(scene.intrinsics)

    def ptr(self, name):
        t = getattr(self, name)
        return None if t is None else t.data_ptr()


class Rasterizer:
    """Owns a vetrast context; forward/backward enqueue on torch's current stream."""

    def __init__(self):
        if not torch.cuda.is_available():
            raise RuntimeError("vet_amd.Rasterizer needs a GPU; there is no CPU path")
        self.lib = abi.load_library()
        h = C.c_void_p()
        abi.check(self.lib.vetrast_create(C.byref(h)), "create")
        self.ctx = h

    def __del__(self):
        try:
            if getattr(self, "ctx", None):
                self.lib.vetrast_destroy(self.ctx)
                self.ctx = None
        except Exception:
            pass

    @staticmethod
    def _stream():
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def layout(self, scene: Scene, render_mode=abi.RENDER_FULL_BLEND) -> abi.WorkspaceLayout:
        lay = abi.WorkspaceLayout()
        v = scene.views[0]
        abi.check(self.lib.vetrast_workspace_layout_for_mode(scene.num_points, len(scene.views), scene.num_layers, v.w,
                                                             v.h, render_mode, C.byref(lay)), "workspace_layout_for_mode")
        return lay

    def forward(self, dev: DeviceScene, params: abi.Params = None, save_for_backward=True, workspace=None,
                out=None, want_weight=False, point_order=None, packed=None) -> ForwardResult:
        """point_order: optional int32 device tensor [N], a permutation: the order the binning pass walks the points in.
        packed: optional float32 device tensor [N,8] from pack_descriptors: the call reads the descriptor records from
        it instead of interleaving them itself."""
        scene = dev.scene
        params = params or make_params(scene)
        lay = self.layout(scene, params.render_mode)
        if workspace is None:
            workspace = torch.empty(lay.total_bytes, dtype=torch.uint8, device=dev.device)
        B, Cn = len(scene.views), scene.num_channels
        sizes = scene.layer_sizes()
        if out is None:
            out = [torch.empty((B, Cn, h, w), dtype=torch.float32, device=dev.device) for (w, h) in sizes]
        masks = [None] * len(sizes)
        if params.output_background_mask:
            masks = [torch.empty((B, 1, h, w), dtype=torch.float32, device=dev.device) for (w, h) in sizes]
        args = abi.ForwardArgs()
        views = make_views(scene)
        fill_forward_args(args, scene, params, views, dev.ptr)
        args.save_for_backward = 1 if save_for_backward else 0
        for l in range(len(sizes)):
            args.out[l] = out[l].data_ptr()
            args.out_mask[l] = masks[l].data_ptr() if masks[l] is not None else None
        weights = None
        if want_weight:
            weights = [torch.empty((B, 1, h, w), dtype=torch.float32, device=dev.device) for (w, h) in sizes]
            for l in range(len(sizes)):
                args.out_weight[l] = weights[l].data_ptr()
        args.workspace = workspace.data_ptr()
        args.workspace_bytes = workspace.numel()
        if point_order is not None:
            assert point_order.dtype == torch.int32 and point_order.is_cuda and point_order.numel() == scene.num_points
            args.point_order = point_order.data_ptr()
        if packed is not None:
            assert packed.dtype == torch.float32 and packed.is_cuda and packed.is_contiguous()
            assert packed.numel() == 8 * scene.num_points
            args.packed_descriptors = packed.data_ptr()
        abi.check(self.lib.vetrast_forward(self.ctx, C.byref(args), self._stream()), "forward")
        return ForwardResult(out, masks, workspace, lay, args, (views, dev, params, point_order, packed), weights)

    def pack_descriptors(self, dev: DeviceScene, params: abi.Params, out=None) -> torch.Tensor:
        """The descriptor records [N,8] of the scene's texture and confidence under `params` (vetrast_pack_descriptors),
        for forward(..., packed=...)."""
        n = dev.scene.num_points
        assert self.lib.vetrast_packed_descriptor_bytes(n) == 32 * n
        if out is None:
            out = torch.empty((n, 8), dtype=torch.float32, device=dev.device)
        a = abi.PackArgs()
        a.num_points = n
        a.texture, a.confidence = dev.ptr("texture"), dev.ptr("confidence")
        C.memmove(C.byref(a.params), C.byref(params), C.sizeof(abi.Params))
        a.packed = out.data_ptr()
        abi.check(self.lib.vetrast_pack_descriptors(self.ctx, C.byref(a), self._stream()), "pack_descriptors")
        return out

    def backward(self, fwd: ForwardResult, grad_out: List[torch.Tensor], want_points=True, want_cameras=False,
                 **param_overrides):
        dev = fwd.keep[1]
        scene = dev.scene
        N, Cn = scene.num_points, scene.num_channels
        g = abi.BackwardArgs()
        C.memmove(C.byref(g.fwd), C.byref(fwd.args), C.sizeof(abi.ForwardArgs))
        for k, v in param_overrides.items():
            setattr(g.fwd.params, k, v)
        for l, t in enumerate(grad_out):
            assert t.is_contiguous() and t.dtype == torch.float32
            g.grad_out[l] = t.data_ptr()
        res = {
            "texture": torch.empty((Cn, N), dtype=torch.float32, device=dev.device),
            "confidence": torch.empty((N,), dtype=torch.float32, device=dev.device),
            "background": torch.empty((Cn,), dtype=torch.float32, device=dev.device),
        }
        g.grad_texture = res["texture"].data_ptr()
        g.grad_confidence = res["confidence"].data_ptr()
        g.grad_background = res["background"].data_ptr()
        if want_points:
            res["points"] = torch.empty((N, 4), dtype=torch.float32, device=dev.device)
            res["point_count"] = torch.empty((N,), dtype=torch.float32, device=dev.device)
            g.grad_points = res["points"].data_ptr()
            g.grad_point_count = res["point_count"].data_ptr()
        if want_cameras:
            F, ncam = int(scene.poses_se3.shape[0]), int(scene.intrinsics.shape[0])
            res["pose"] = torch.empty((F, 6), dtype=torch.float64, device=dev.device)
            res["pose_count"] = torch.empty((F,), dtype=torch.float32, device=dev.device)
            res["intrinsics"] = torch.empty((ncam, 13), dtype=torch.float32, device=dev.device)
            res["intrinsics_count"] = torch.empty((ncam,), dtype=torch.float32, device=dev.device)
            g.grad_pose = res["pose"].data_ptr()
            g.grad_pose_count = res["pose_count"].data_ptr()
            g.grad_intrinsics = res["intrinsics"].data_ptr()
            g.grad_intrinsics_count = res["intrinsics_count"].data_ptr()
        abi.check(self.lib.vetrast_backward(self.ctx, C.byref(g), self._stream()), "backward")
        # the argument block only holds raw pointers: whoever replays it (graph capture, timing loops) needs the
        # upstream gradients, the forward result and the gradient tensors to stay alive with it
        g._keepalive = (list(grad_out), fwd, res)
        res["_args"] = g
        return res

    def adam_step(self, param, grad, exp_avg, exp_avg_sq, step, lr, beta1=0.9, beta2=0.999, eps=1e-8,
                  weight_decay=0.0, zero_grad=False):
        """One fused Adam step in place on contiguous float32 CUDA tensors (vetrast_adam_step)."""
        a = abi.AdamArgs()
        for name, t in (("param", param), ("grad", grad), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
            assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == param.numel()
            setattr(a, name, t.data_ptr())
        a.n, a.step = param.numel(), step
        a.lr, a.beta1, a.beta2, a.eps, a.weight_decay, a.zero_grad = lr, beta1, beta2, eps, weight_decay, int(zero_grad)
        abi.check(self.lib.vetrast_adam_step(self.ctx, C.byref(a), self._stream()), "adam_step")

    def lift_error(self, cell_bb_min, cell_bb_length, cell_value, cell_access_count, view, poses_se3, intrinsics,
                   loss_image, border_pixels=abi.LIFT_BORDER_PIXELS, workspace=None, static_scratch=False):
        """Adds the error image of one view to the grid cells its pixels fall in, in place on cell_value (float32 [n]
        or [n,1]) and cell_access_count (int32) (vetrast_lift_error; the reference's FillSceneGridWithLoss). All
        arguments but `view` (a synthetic.View) are contiguous CUDA tensors. Returns the workspace, whose flag word
        `lift_flags` reads. With `static_scratch` the call goes to vetrast_lift_error_static, which takes no workspace
        (the scratch is an array inside the library) and allocates nothing; None is returned."""
        a = abi.LiftArgs()
        for name, t, dt in (("cell_bb_min", cell_bb_min, torch.float32), ("cell_bb_length", cell_bb_length, torch.float32),
                            ("cell_value", cell_value, torch.float32), ("cell_access_count", cell_access_count, torch.int32),
                            ("poses_se3", poses_se3, torch.float64), ("intrinsics", intrinsics, torch.float32),
                            ("loss_image", loss_image, torch.float32)):
            assert t.is_cuda and t.dtype == dt and t.is_contiguous(), name
            setattr(a, name, t.data_ptr())
        a.num_cells = cell_value.numel()
        assert cell_bb_min.numel() == 3 * a.num_cells and cell_bb_length.numel() == 3 * a.num_cells
        assert cell_access_count.numel() == a.num_cells and loss_image.dim() == 3
        fill_lift_args(a, view, poses_se3, intrinsics, loss_image, border_pixels)
        if static_scratch:
            abi.check(self.lib.vetrast_lift_error_static(self.ctx, C.byref(a), self._stream()), "lift_error_static")
            return None
        need = int(self.lib.vetrast_lift_workspace_bytes(a.num_cells))
        if workspace is None:
            workspace = torch.empty(max(need, 256), dtype=torch.uint8, device=loss_image.device)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        abi.check(self.lib.vetrast_lift_error(self.ctx, C.byref(a), self._stream()), "lift_error")
        return workspace

    @staticmethod
    def lift_flags(workspace):
        """Blocking: the flag word of a lift_error workspace (1: the camera row had non-zero distortion)."""
        return int(workspace[abi.LIFT_FLAGS_OFFSET:abi.LIFT_FLAGS_OFFSET + 4].view(torch.int32).item())

    def check_device_flags(self, fwd: ForwardResult):
        return self.lib.vetrast_query_device_flags(self.ctx, C.c_void_p(fwd.workspace.data_ptr()),
                                                   C.byref(fwd.layout), self._stream())

    # ---- per-kernel timing (the reference's timer_system) -------------------------------------------------------
    def set_profiling(self, on: bool):
        abi.check(self.lib.vetrast_set_profiling(self.ctx, 1 if on else 0), "set_profiling")

    def reset_scope_times(self):
        abi.check(self.lib.vetrast_reset_scope_times(self.ctx), "reset_scope_times")

    def scope_times(self):
        ms = (C.c_float * abi.SCOPE_COUNT)()
        n = (C.c_int32 * abi.SCOPE_COUNT)()
        abi.check(self.lib.vetrast_scope_times(self.ctx, ms, n), "scope_times")
        return {abi.SCOPE_NAMES[i]: (float(ms[i]), int(n[i])) for i in range(abi.SCOPE_COUNT)}
