"""ctypes wrapper of the CPU oracle (oracle/libvetrast_oracle.so) — TEST INFRASTRUCTURE ONLY.

Imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; the product (vet_amd/) never imports it.
The argument structs are the ctypes mirrors of include/vetrast.h from vet_amd.abi, filled with host pointers.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from vet_amd import abi
from vet_amd.rasterizer import fill_forward_args, fill_lift_args, make_params, make_views
from vet_amd.synthetic import Scene

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libvetrast_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-B", "libvetrast_oracle.so"], check=True)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} is missing: run `make -C oracle`")
        lib = C.CDLL(LIB_PATH)
        sizes = (C.c_uint64 * 4)()
        mirrors = [C.sizeof(t) for t in (abi.ForwardArgs, abi.BackwardArgs, abi.AdamArgs, abi.LiftArgs)]
        if not hasattr(lib, "vetref_struct_sizes") or lib.vetref_struct_sizes(sizes) != 0 or list(sizes) != mirrors:
            raise OSError(f"{LIB_PATH} was built from another version of include/vetrast.h: run `make -C oracle`")
        lib.vetref_forward.restype = C.c_int
        lib.vetref_forward.argtypes = [C.POINTER(abi.ForwardArgs), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_int]
        lib.vetref_backward.restype = C.c_int
        lib.vetref_backward.argtypes = [C.POINTER(abi.BackwardArgs), C.c_void_p, C.c_void_p, C.c_int]
        lib.vetref_prepare_view.restype = C.c_int
        lib.vetref_prepare_view.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        lib.vetref_project_point.restype = C.c_int
        lib.vetref_project_point.argtypes = [C.c_void_p, C.POINTER(abi.View), C.c_void_p, C.c_void_p]
        lib.vetref_sigmoid.restype = C.c_int
        lib.vetref_sigmoid.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_float]
        lib.vetref_adam_step.restype = C.c_int
        lib.vetref_adam_step.argtypes = [C.POINTER(abi.AdamArgs)]
        lib.vetref_lift_error.restype = C.c_int
        lib.vetref_lift_error.argtypes = [C.POINTER(abi.LiftArgs), C.c_int]
        _lib = lib
    return _lib


def _addr(a):
    return None if a is None else a.ctypes.data


class OracleForward:
    """Result of the oracle's forward pass (numpy arrays) plus everything backward needs."""

    def __init__(self, scene: Scene, params: abi.Params, num_threads=1):
        self.scene, self.params = scene, params
        self.views = make_views(scene)
        B, Cn, N, L = len(scene.views), scene.num_channels, scene.num_points, scene.num_layers
        self.sizes = scene.layer_sizes()
        self.P = sum(w * h for w, h in self.sizes)
        self.cap = N * L * (4 if params.render_mode == abi.RENDER_BILINEAR_BLEND else 1)
        self.out = [np.zeros((B, Cn, h, w), np.float32) for (w, h) in self.sizes]
        self.out_mask = [np.zeros((B, 1, h, w), np.float32) if params.output_background_mask else None
                         for (w, h) in self.sizes]
        self.offsets = np.zeros((B, self.P + 1), np.uint32)
        self.fragments = np.zeros((B, max(self.cap, 1)), np.uint64)
        self.transmittance = np.zeros((B, max(self.cap, 1)), np.float32)
        self.weight = np.zeros((B, self.P), np.float32)
        self.kept = np.zeros((B, self.P), np.uint32)  # fragments of every pixel that took part in the blend
        self.inputs = {k: (None if getattr(scene, k) is None else np.ascontiguousarray(getattr(scene, k)))
                       for k in ("position", "index", "texture", "confidence", "background", "dropout", "poses_se3",
                                 "intrinsics")}
        a = abi.ForwardArgs()
        fill_forward_args(a, scene, params, self.views, lambda n: _addr(self.inputs[n]))
        a.save_for_backward = 1
        for l in range(L):
            a.out[l] = _addr(self.out[l])
            a.out_mask[l] = _addr(self.out_mask[l])
        self.args = a
        self.status = load().vetref_forward(C.byref(a), _addr(self.offsets), _addr(self.fragments),
                                            _addr(self.transmittance), _addr(self.weight), _addr(self.kept),
                                            num_threads)

    def layer_base(self, l):
        return sum(w * h for w, h in self.sizes[:l])

    def pixel_list(self, b, l, x, y):
        q = self.layer_base(l) + y * self.sizes[l][0] + x
        o0, o1 = int(self.offsets[b, q]), int(self.offsets[b, q + 1])
        return self.fragments[b, o0:o1]


def forward(scene: Scene, params: abi.Params = None, num_threads=1, **overrides) -> OracleForward:
    params = params or make_params(scene, **overrides)
    res = OracleForward(scene, params, num_threads)
    if res.status != 0:
        raise abi.VetrastError(res.status, "oracle forward")
    return res


def backward(fwd: OracleForward, grad_out, want_points=True, want_cameras=False, num_threads=1, **param_overrides):
    scene = fwd.scene
    N, Cn = scene.num_points, scene.num_channels
    g = abi.BackwardArgs()
    C.memmove(C.byref(g.fwd), C.byref(fwd.args), C.sizeof(abi.ForwardArgs))
    for k, v in param_overrides.items():
        setattr(g.fwd.params, k, v)
    go = [np.ascontiguousarray(t, dtype=np.float32) for t in grad_out]
    for l, t in enumerate(go):
        g.grad_out[l] = _addr(t)
    res = {
        "texture": np.zeros((Cn, N), np.float32),
        "confidence": np.zeros((N,), np.float32),
        "background": np.zeros((Cn,), np.float32),
    }
    g.grad_texture = _addr(res["texture"])
    g.grad_confidence = _addr(res["confidence"])
    g.grad_background = _addr(res["background"])
    if want_points:
        res["points"] = np.zeros((N, 4), np.float32)
        res["point_count"] = np.zeros((N,), np.float32)
        g.grad_points = _addr(res["points"])
        g.grad_point_count = _addr(res["point_count"])
    if want_cameras:
        F, ncam = int(scene.poses_se3.shape[0]), int(scene.intrinsics.shape[0])
        res["pose"] = np.zeros((F, 6), np.float64)
        res["pose_count"] = np.zeros((F,), np.float32)
        res["intrinsics"] = np.zeros((ncam, 13), np.float32)
        res["intrinsics_count"] = np.zeros((ncam,), np.float32)
        g.grad_pose = _addr(res["pose"])
        g.grad_pose_count = _addr(res["pose_count"])
        g.grad_intrinsics = _addr(res["intrinsics"])
        g.grad_intrinsics_count = _addr(res["intrinsics_count"])
    st = load().vetref_backward(C.byref(g), _addr(fwd.offsets), _addr(fwd.fragments), num_threads)
    if st != 0:
        raise abi.VetrastError(st, "oracle backward")
    return res


def prepare_view(pose8, intrinsics13):
    """Camera constants of a view: [0:12] rotation rows with the translation in the fourth column, [12:17] fx fy cx cy
    s, [17:25] the distortion coefficients k1 k2 k3 k4 k5 k6 p1 p2, [25] 1 if any of them is not zero."""
    out = np.zeros(26, np.float32)
    p = np.ascontiguousarray(pose8, np.float64)
    k = np.ascontiguousarray(intrinsics13, np.float32)
    load().vetref_prepare_view(_addr(p), _addr(k), _addr(out))
    return out


def project_point(prepared26, view: abi.View, position4):
    out = np.zeros(4, np.float32)
    m = np.ascontiguousarray(prepared26, np.float32)
    assert m.size == 26
    p = np.ascontiguousarray(position4, np.float32)
    ok = load().vetref_project_point(_addr(m), C.byref(view), _addr(p), _addr(out))
    return bool(ok), out


def sigmoid(x, scale):
    """sigmoid(scale * x) in the canonical float32 arithmetic of the fused confidence activation."""
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    load().vetref_sigmoid(_addr(x), _addr(y), x.size, scale)
    return y


def adam_step(param, grad, exp_avg, exp_avg_sq, step, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0,
              zero_grad=False):
    """One Adam step in place on float32 numpy arrays."""
    a = abi.AdamArgs()
    for name, arr in (("param", param), ("grad", grad), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
        assert arr.dtype == np.float32 and arr.flags.c_contiguous
        setattr(a, name, _addr(arr))
    a.n, a.step = param.size, step
    a.lr, a.beta1, a.beta2, a.eps, a.weight_decay, a.zero_grad = lr, beta1, beta2, eps, weight_decay, int(zero_grad)
    st = load().vetref_adam_step(C.byref(a))
    if st != 0:
        raise abi.VetrastError(st, "oracle adam_step")


def lift_error(cell_bb_min, cell_bb_length, cell_value, cell_access_count, view, poses_se3, intrinsics, loss_image,
               border_pixels=abi.LIFT_BORDER_PIXELS, num_threads=1):
    """Error lifting on numpy arrays, in place on cell_value (float32 [n]) and cell_access_count (int32 [n])."""
    a = abi.LiftArgs()
    for name, arr, dt in (("cell_bb_min", cell_bb_min, np.float32), ("cell_bb_length", cell_bb_length, np.float32),
                          ("cell_value", cell_value, np.float32), ("cell_access_count", cell_access_count, np.int32),
                          ("poses_se3", poses_se3, np.float64), ("intrinsics", intrinsics, np.float32),
                          ("loss_image", loss_image, np.float32)):
        assert arr.dtype == dt and arr.flags.c_contiguous, name
        setattr(a, name, _addr(arr))
    a.num_cells = cell_value.size
    assert cell_bb_min.shape == (a.num_cells, 3) and cell_bb_length.shape == (a.num_cells, 3)
    fill_lift_args(a, view, poses_se3, intrinsics, loss_image, border_pixels)
    st = load().vetref_lift_error(C.byref(a), num_threads)
    if st != 0:
        raise abi.VetrastError(st, "oracle lift_error")
