"""Error behaviour and edge cases of the C ABI on the GPU: every bad call returns a status (nothing aborts), odd image
sizes, empty clouds, all points behind the camera, one-channel descriptors, five layers, viewer-only confidence cut,
dropout masks, HIP graph capture of a whole forward+backward."""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu


def _parity(scene, rasterizer, oracle, backward=True, **over):
    params = make_params(scene, **over)
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params)
    torch.cuda.synchronize()
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64))
        keep = kept_mask(off, params.debug_max_list_length)
        np.testing.assert_array_equal(res.fragments(b)[keep], ref.fragments[b, :int(off[-1])][keep])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    if backward:
        go = scene.grad_out()
        want = oracle.backward(ref, go)
        got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go])
        torch.cuda.synchronize()
        for key in ("texture", "confidence", "points"):
            assert max_rel_err(got[key].cpu().numpy(), want[key]) <= 1e-4, key
        # the oracle adds the background gradient in float32 in pixel order, which is the less accurate of the two sums
        # when most pixels are empty; the exact value is checked where a closed form exists
        assert max_rel_err(got["background"].cpu().numpy(), want["background"]) <= 2e-3
        return res, ref, got
    return res, ref, None


def test_odd_sizes_and_five_layers(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=9000, w=83, h=61, num_layers=5, K=6, seed=51)
    assert scene.layer_sizes() == [(83, 61), (41, 30), (20, 15), (10, 7), (5, 3)]
    _parity(scene, rasterizer, oracle, need_point_gradient=1)


@pytest.mark.parametrize("channels", [1, 2, 3])
def test_fewer_channels(channels, rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=4000, K=5, channels=channels, seed=52 + channels)
    _parity(scene, rasterizer, oracle, need_point_gradient=1)


def test_no_point_in_front_of_the_camera(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=500, seed=56)
    scene.position[:, 2] = -5.0
    res, ref, got = _parity(scene, rasterizer, oracle, need_point_gradient=1)
    assert int(res.offsets(0)[-1]) == 0
    for o in res.out:  # every pixel shows the background
        np.testing.assert_array_equal(o.cpu().numpy()[0, :, 0, 0], scene.background)
    # ... so the background gradient is the plain sum of the incoming gradients
    exact = sum(g.astype(np.float64).sum(axis=(0, 2, 3)) for g in scene.grad_out())
    assert max_rel_err(got["background"].cpu().numpy(), exact) <= 1e-5
    assert not got["texture"].any() and not got["confidence"].any() and not got["points"].any()


def test_viewer_only_confidence_cut_and_dropout_mask(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=5000, K=8, seed=57, num_views=2)
    rng = np.random.default_rng(1)
    scene.dropout = (rng.random((2, scene.num_points)) < 0.3).astype(np.float32)
    res, ref, _ = _parity(scene, rasterizer, oracle, backward=False, viewer_only=1, stability_cutoff_value=0.4)
    visible = int(ref.offsets[0, -1])
    assert 0 < visible < 0.6 * scene.num_points * scene.num_layers


def test_single_point_cloud(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=1, seed=58)
    scene.position[0, :3] = (0.0, 0.0, 0.5)
    _parity(scene, rasterizer, oracle, need_point_gradient=1)


def test_bad_calls_return_status_codes(rasterizer):
    scene = synthetic.tiny_scene(num_points=200, seed=59)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev)
    lib, ctx, stream = rasterizer.lib, rasterizer.ctx, rasterizer._stream()

    def call_with(mutate):
        a = abi.ForwardArgs()
        C.memmove(C.byref(a), C.byref(res.args), C.sizeof(abi.ForwardArgs))
        mutate(a)
        return lib.vetrast_forward(ctx, C.byref(a), stream)

    assert call_with(lambda a: None) == abi.OK
    assert call_with(lambda a: setattr(a, "workspace_bytes", 1024)) == abi.ERR_WORKSPACE_SMALL
    assert call_with(lambda a: setattr(a, "workspace", a.workspace + 8)) == abi.ERR_INVALID_ARG
    assert call_with(lambda a: setattr(a, "position", None)) == abi.ERR_INVALID_ARG
    assert call_with(lambda a: setattr(a.params, "num_layers", 6)) == abi.ERR_INVALID_ARG
    assert call_with(lambda a: setattr(a.params, "num_texture_channels", 5)) == abi.ERR_INVALID_ARG
    assert call_with(lambda a: setattr(a.params, "check_normal", 1)) == abi.ERR_UNSUPPORTED
    assert call_with(lambda a: setattr(a, "num_views", 0)) == abi.ERR_INVALID_ARG

    views = (abi.View * 1)()
    C.memmove(views, res.args.views, C.sizeof(abi.View))
    views[0].camera_model_type = abi.CAMERA_OCAM
    assert call_with(lambda a: setattr(a, "views", views)) == abi.ERR_UNSUPPORTED
    views[0].camera_model_type = abi.CAMERA_PINHOLE_DISTORTION
    views[0].image_index = 7
    assert call_with(lambda a: setattr(a, "views", views)) == abi.ERR_INVALID_ARG

    g = abi.BackwardArgs()
    C.memmove(C.byref(g.fwd), C.byref(res.args), C.sizeof(abi.ForwardArgs))
    assert lib.vetrast_backward(ctx, C.byref(g), stream) == abi.ERR_INVALID_ARG  # no gradient buffers
    torch.cuda.synchronize()


def test_nonzero_distortion_raises_the_device_flag(rasterizer):
    scene = synthetic.tiny_scene(num_points=200, seed=60)
    scene.intrinsics[0, 6] = 0.05
    res = rasterizer.forward(DeviceScene(scene))
    assert rasterizer.check_device_flags(res) == abi.ERR_BAD_INPUT_DATA
    scene.intrinsics[0, 6] = 0.0
    res = rasterizer.forward(DeviceScene(scene))
    assert rasterizer.check_device_flags(res) == abi.OK


@pytest.mark.parametrize("mode,K", [(abi.RENDER_FULL_BLEND, 16), (abi.RENDER_FUZZY_BLEND, -1), (abi.RENDER_BILINEAR_BLEND, 16)],
                         ids=["full", "fuzzy_no_cut", "bilinear"])
def test_forward_backward_can_be_captured_in_a_hip_graph(mode, K, rasterizer, oracle):
    """The library only launches kernels (no memsets, allocations or host reads), so a whole step replays from a
    graph; every replay is compared with the eager result, with eager work in between. (FUZZY_BLEND without a list cut
    also launches the kernel that walks the lists too long for the dense layout.)"""
    scene = synthetic.config2(num_points=60_000, w=480, h=270, K=K)
    params = make_params(scene, need_point_gradient=1, render_mode=mode, depth_accept_blend=0.05)
    dev = DeviceScene(scene)
    eager = rasterizer.forward(dev, params)
    go = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    eager_g = rasterizer.backward(eager, go)
    torch.cuda.synchronize()
    want_out = [o.clone() for o in eager.out]
    want_g = {k: v.clone() for k, v in eager_g.items() if k != "_args"}

    lib, ctx = rasterizer.lib, rasterizer.ctx
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            abi.check(lib.vetrast_forward(ctx, C.byref(eager.args), s), "forward (capture)")
            abi.check(lib.vetrast_backward(ctx, C.byref(eager_g["_args"]), s), "backward (capture)")
    for replay in range(3):
        for o in eager.out:
            o.zero_()
        for k, v in eager_g.items():
            if k != "_args":
                v.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager.out, want_out):
            assert torch.equal(a, b), f"replay {replay}"
        for k, v in want_g.items():
            assert torch.equal(eager_g[k], v), (k, replay)
        # eager work between replays
        again = rasterizer.forward(dev, params)
        torch.cuda.synchronize()
        assert torch.equal(again.out[0], want_out[0])


@pytest.mark.parametrize("K", [16, 0])
def test_cluster_far_denser_than_the_layer_average(K, rasterizer, oracle):
    """All points inside a 3x3 pixel patch of a 96x64 image: the bins that hold them are thousands of times fuller than
    the host-side estimate they were sized for, so they take the path that streams a bin from memory, sorts lists of
    thousands of keys in place and blends one thread per pixel."""
    scene = synthetic.tiny_scene(num_points=30_000, w=96, h=64, num_layers=3, K=K, seed=61)
    scene.position[:, 0] *= 0.02
    scene.position[:, 1] *= 0.02
    res, ref, _ = _parity(scene, rasterizer, oracle, backward=(K > 0), need_point_gradient=1)
    counts = np.diff(res.offsets(0))
    assert counts.max() > 2500 and (counts > 0).sum() < 40


def test_more_views_than_one_preparation_launch_holds(rasterizer, oracle):
    """18 views: the view constants are prepared 16 per launch, the second launch must not reset what the first wrote."""
    print("[case] 18 views", flush=True)
    scene = synthetic.tiny_scene(num_points=1500, K=6, seed=53, num_views=18)
    params = make_params(scene, need_point_gradient=1)
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_cameras=True)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_cameras=True)
    torch.cuda.synchronize()
    for key in ("texture", "confidence", "background", "points", "pose"):
        assert max_rel_err(got[key].cpu().numpy(), want[key]) <= 1e-4, key


_LENGTHS_IN_ONE_SMALL_BIN = [1, 2, 63, 64, 65, 127, 128, 129]   # 579 keys: the bin is built in LDS
_LENGTHS_IN_ONE_FULL_BIN = [200, 255, 256, 257]                  # 968 keys, still in LDS, one list beyond a wave's registers
_LENGTHS_APART = [300, 511, 512, 513, 700, 1023, 1024, 1025, 1500, 4097]  # each makes its bin stream from memory


@pytest.mark.parametrize("K", [0, 100, 16])
@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND])
def test_list_lengths_around_every_sorting_limit(K, mode, rasterizer, oracle):
    """Pixels that receive exactly 63, 64, 65, ..., 1025, 4097 points: one length either side of every limit between
    the sorting methods (one wave's network, two or four keys per lane in registers, the workgroup's sort in LDS, the
    in-place sort in memory), in bins built in LDS and in bins streamed from memory. A quarter of the points share their
    depth with another point of the same pixel, so the order inside ties is checked as well."""
    print(f"[case] list lengths around the sorting limits K={K} mode={mode}", flush=True)
    w, h = 64, 32
    where = [((2 + i, 1), n) for i, n in enumerate(_LENGTHS_IN_ONE_SMALL_BIN)]
    where += [((34 + i, 17), n) for i, n in enumerate(_LENGTHS_IN_ONE_FULL_BIN)]
    where += [((4 + 6 * (i % 5) + 32 * (i // 5 % 2), 9 + 16 * (i // 5 % 2)), n) for i, n in enumerate(_LENGTHS_APART)]
    total = sum(n for _, n in where)
    scene = synthetic.tiny_scene(num_points=total, w=w, h=h, num_layers=1, K=K, seed=97)
    rng = np.random.default_rng(97)
    fx, cx, cy = 0.45 * w, w / 2.0, h / 2.0
    first = 0
    for (px, py), n in where:
        z = rng.uniform(-0.4, 1.4, size=n)
        z[n // 4 * 3:] = z[: n - n // 4 * 3]           # depth ties inside the list
        z = z.astype(np.float32).astype(np.float64)
        scene.position[first:first + n, 0] = ((px - cx) * (z + 2.0) / fx).astype(np.float32)
        scene.position[first:first + n, 1] = ((py - cy) * (z + 2.0) / fx).astype(np.float32)
        scene.position[first:first + n, 2] = z.astype(np.float32)
        first += n
    order = rng.permutation(total)                     # list places do not follow the point order
    scene.position = np.ascontiguousarray(scene.position[order])
    res, ref, _ = _parity(scene, rasterizer, oracle, backward=(K > 0), need_point_gradient=1, render_mode=mode,
                          depth_accept_blend=0.05)
    counts = np.diff(res.offsets(0)).reshape(h, w)
    for (px, py), n in where:
        assert counts[py, px] == n, (px, py, n, counts[py, px])
    assert counts.sum() == total


def test_two_contexts_on_two_streams_do_not_disturb_each_other(rasterizer, oracle):
    """There is no process-global state (the reference keeps its parameters in __constant__ symbols,
    src/lib/rendering/RenderForward.cu:22-27): two contexts with their own workspaces, driven from two streams at the same
    time, on different scenes and in different modes, give what each gives alone, frame after frame."""
    from vet_amd.rasterizer import Rasterizer

    print("[case] two contexts on two streams", flush=True)
    scene_a = synthetic.config2(num_points=150_000, w=640, h=360)
    scene_b = synthetic.tiny_scene(num_points=60_000, w=320, h=200, num_layers=4, K=-1, seed=77)
    other = Rasterizer()
    jobs = []
    for rast, scene, over in ((rasterizer, scene_a, {}), (other, scene_b, {"render_mode": abi.RENDER_BILINEAR_BLEND})):
        params = make_params(scene, need_point_gradient=1, **over)
        dev = DeviceScene(scene)
        res = rast.forward(dev, params)
        go = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
        grads = rast.backward(res, go)
        torch.cuda.synchronize()
        want_out = [o.clone() for o in res.out]
        want_g = {k: v.clone() for k, v in grads.items() if k != "_args"}
        jobs.append((rast, res, grads, want_out, want_g, torch.cuda.Stream(), go))  # go: the calls hold its pointers
    for frame in range(4):
        for rast, res, grads, _, _, stream, _ in jobs:
            for o in res.out:
                o.zero_()
            for k, v in grads.items():
                if k != "_args":
                    v.fill_(float("nan"))
        torch.cuda.synchronize()
        for _ in range(3):  # several frames in flight on either stream
            for rast, res, grads, _, _, stream, _ in jobs:
                s = C.c_void_p(stream.cuda_stream)
                abi.check(rast.lib.vetrast_forward(rast.ctx, C.byref(res.args), s), "forward")
                abi.check(rast.lib.vetrast_backward(rast.ctx, C.byref(grads["_args"]), s), "backward")
        torch.cuda.synchronize()
        for rast, res, grads, want_out, want_g, _, _ in jobs:
            for a, b in zip(res.out, want_out):
                assert torch.equal(a, b), f"frame {frame}"
            for k, v in want_g.items():
                assert torch.equal(grads[k], v), (k, frame)


@pytest.mark.parametrize("mode", ["full", "fuzzy_no_cut", "bilinear"])
def test_empty_cloud(rasterizer, mode):
    """num_points = 0 (the buffers exist, they are just not read): every pixel shows the background, the background
    gradient is the plain sum of the incoming gradients, nothing else is touched or launched on the points."""
    print(f"[case] empty cloud, {mode}", flush=True)
    scene = synthetic.tiny_scene(num_points=8, w=40, h=24, num_layers=3, seed=58)
    dev = DeviceScene(scene)
    over = {"full": {}, "bilinear": {"render_mode": abi.RENDER_BILINEAR_BLEND},
            "fuzzy_no_cut": {"render_mode": abi.RENDER_FUZZY_BLEND, "depth_accept_blend": 0.05, "debug_max_list_length": -1}}[mode]
    params = make_params(scene, need_point_gradient=1, **over)
    full = rasterizer.forward(dev, params)  # sizes the workspace and the outputs
    torch.cuda.synchronize()
    args = full.args
    args.num_points = 0
    for o in full.out:
        o.fill_(float("nan"))
    abi.check(rasterizer.lib.vetrast_forward(rasterizer.ctx, C.byref(args), None), "forward, no points")
    torch.cuda.synchronize()
    for o in full.out:
        got = o.cpu().numpy()
        assert np.all(got == scene.background.reshape(1, -1, 1, 1))
    g = abi.BackwardArgs()
    C.memmove(C.byref(g.fwd), C.byref(args), C.sizeof(abi.ForwardArgs))
    go = [torch.from_numpy(x).cuda() for x in scene.grad_out()]
    for l, t in enumerate(go):
        g.grad_out[l] = t.data_ptr()
    gb = torch.full((scene.num_channels,), float("nan"), device="cuda")
    gt = torch.zeros((scene.num_channels, 8), device="cuda")
    gc = torch.zeros((8,), device="cuda")
    g.grad_texture, g.grad_confidence, g.grad_background = gt.data_ptr(), gc.data_ptr(), gb.data_ptr()
    abi.check(rasterizer.lib.vetrast_backward(rasterizer.ctx, C.byref(g), None), "backward, no points")
    torch.cuda.synchronize()
    exact = sum(x.astype(np.float64).sum(axis=(0, 2, 3)) for x in scene.grad_out())
    assert max_rel_err(gb.cpu().numpy(), exact) <= 1e-5
    assert not gt.any() and not gc.any()


@pytest.mark.parametrize("num_poses", [2, 40, 3000])
def test_camera_accumulators_are_cleared(rasterizer, oracle, num_poses):
    """The pose and intrinsics gradients are sums over the views of a call and are cleared inside the call: by the first
    per-pixel kernel where they are small, by a fill kernel of their own where they are not (3 000 pose rows). The call
    is replayed onto outputs full of NaN; rows no view uses must come back as exact zeros."""
    print(f"[case] camera accumulators, {num_poses} pose rows", flush=True)
    scene = synthetic.tiny_scene(num_points=4000, num_views=2, seed=61)
    have = scene.poses_se3.shape[0]
    if num_poses > have:
        scene.poses_se3 = np.ascontiguousarray(np.concatenate(
            [scene.poses_se3, np.tile(scene.poses_se3[:1], (num_poses - have, 1))]))
    params = make_params(scene, need_point_gradient=1)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    grad_out = scene.grad_out()
    got = rasterizer.backward(res, [torch.from_numpy(x).cuda() for x in grad_out], want_cameras=True)
    torch.cuda.synchronize()
    for key in ("pose", "pose_count", "intrinsics", "intrinsics_count"):
        got[key].fill_(float("nan"))
    abi.check(rasterizer.lib.vetrast_backward(rasterizer.ctx, C.byref(got["_args"]), None), "backward again")
    torch.cuda.synchronize()
    want = oracle.backward(oracle.forward(scene, params), grad_out, want_points=True, want_cameras=True)
    used = sorted({v.image_index for v in scene.views})
    pose = got["pose"].cpu().numpy()
    assert np.isfinite(pose).all() and np.isfinite(got["intrinsics"].cpu().numpy()).all()
    unused = np.setdiff1d(np.arange(pose.shape[0]), used)
    assert not pose[unused].any() and not got["pose_count"].cpu().numpy()[unused].any()
    np.testing.assert_array_equal(got["pose_count"].cpu().numpy(), want["pose_count"])
    np.testing.assert_array_equal(got["intrinsics_count"].cpu().numpy(), want["intrinsics_count"])
    assert max_rel_err(pose, want["pose"]) <= 1e-3
    assert max_rel_err(got["intrinsics"].cpu().numpy(), want["intrinsics"]) <= 1e-3
