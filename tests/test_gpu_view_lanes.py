"""GPU tests of calls with several views, whose views share the library's launches.

Up to four views of a call go through every kernel together: one launch per kernel for such a round, each view on a lane
(its own copy of the scratch that one view needs); further views follow in rounds; the per-point backward kernel adds
a round's views up inside its threads. None of that may show in the results: the cases here
hold calls of 2 to 9 views (short rounds, exact rounds, several rounds) against the oracle in all three render modes
with camera gradients, drop-out masks and an index indirection, compare a call of many views with the same views given
one per call, capture such a call in a HIP graph and replay it, and run two contexts on two streams at once.
Counterpart of the per-view host loop, src/lib/rendering/PointRenderer.cu:771-931 (forward) and :1185-1249 (backward).
"""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, Rasterizer, make_params

pytestmark = pytest.mark.gpu
MODES = [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND, abi.RENDER_BILINEAR_BLEND]


def _scene(num_views, seed, num_points=5000, **kw):
    scene = synthetic.tiny_scene(num_points=num_points, w=96, h=64, num_layers=3, K=8, seed=seed, num_views=num_views, **kw)
    return scene


@pytest.mark.parametrize("render_mode", MODES)
@pytest.mark.parametrize("num_views", [2, 3, 4, 5, 9])
def test_many_views_match_the_oracle(render_mode, num_views, rasterizer, oracle):
    print(f"[case] view lanes: {num_views} views, render mode {render_mode}", flush=True)
    scene = _scene(num_views, 80 + num_views)
    rng = np.random.default_rng(num_views)
    scene.dropout = (rng.uniform(size=(num_views, scene.num_points)) < 0.2).astype(np.float32)
    if num_views == 5:
        scene.index = rng.integers(0, 1200, size=scene.num_points).astype(np.int32)
    params = make_params(scene, need_point_gradient=1, render_mode=render_mode, depth_accept_blend=0.05,
                         quirk_background_confidence_leak=1 if render_mode == abi.RENDER_FULL_BLEND else 0)
    res = rasterizer.forward(DeviceScene(scene), params)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0 and res.layout.view_lanes == min(num_views, 4)
    ref = oracle.forward(scene, params)
    for b in range(num_views):
        np.testing.assert_array_equal(res.offsets(b), ref.offsets[b].astype(np.int64))
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    go = scene.grad_out()
    want = oracle.backward(ref, go, want_cameras=True)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go], want_cameras=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in ("texture", "confidence", "background", "points", "pose", "intrinsics"):
        g, w = got[key].cpu().numpy(), want[key]
        if key == "confidence" and params.quirk_background_confidence_leak:
            # Row 0 also takes the leak term of every view: a float32 sum over all pixels of terms of both signs, added
            # in arrival order on the oracle's side. It is held to a looser bar, against the scale of the whole tensor.
            assert abs(float(g.ravel()[0]) - float(w.ravel()[0])) <= 5e-3 * float(np.abs(w).max()), "leak row"
            g, w = g.ravel()[1:], w.ravel()[1:]
        err = max_rel_err(g, w)
        # (pose and intrinsics: one sum over all fragments of a view, of both signs, in float32 and arrival order on
        # the oracle's side, hierarchical and in double here)
        assert err <= (3e-4 if key in ("pose", "intrinsics") else 1e-4), (key, err)
    assert np.abs(want["pose"]).sum() > 0 and got["pose_count"].cpu().numpy().min() > 0


@pytest.mark.parametrize("render_mode", MODES)
@pytest.mark.parametrize("num_views", [1, 3, 6])
def test_hints_that_switch_the_record_layout_change_nothing(render_mode, num_views, rasterizer, oracle):
    """Where the caller expects its views to see a small part of the cloud (vetrast_params.expected_fragments), the
    backward pass keeps a point's gradient records next to each other instead of layer after layer. The same call
    without hints, with hints that say "most of the cloud" and with hints that say "next to nothing" (which also makes
    the bins overflow): images the same bits, gradients against the oracle and against each other."""
    scene = _scene(num_views, 60 + num_views)
    go = scene.grad_out()
    results = []
    for hint in (0.0, 0.9 * scene.num_points, 25.0):
        params = make_params(scene, need_point_gradient=1, render_mode=render_mode, depth_accept_blend=0.05)
        for l in range(scene.num_layers):
            params.expected_fragments[l] = hint
        res = rasterizer.forward(DeviceScene(scene), params)
        got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go], want_cameras=True)
        torch.cuda.synchronize()
        results.append((res, got, params))
    ref = oracle.forward(scene, results[0][2])
    want = oracle.backward(ref, go, want_cameras=True)
    for res, got, _ in results:
        for l in range(scene.num_layers):
            np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
        for key in ("texture", "confidence", "background", "points", "pose", "intrinsics"):
            err = max_rel_err(got[key].cpu().numpy(), want[key])
            assert err <= (3e-4 if key in ("pose", "intrinsics") else 1e-4), (key, err)
    # one record per fragment whatever the layout: the per-point sums are the same additions in the same order
    for key in ("texture", "confidence", "points", "point_count"):
        assert torch.equal(results[0][1][key], results[2][1][key]), key


@pytest.mark.parametrize("max_list_length", [-1, 48])
def test_uncut_fuzzy_lists_of_several_views(max_list_length, rasterizer, oracle):
    """FUZZY_BLEND without a cut (or a cut beyond what the dense backward kernel takes): lists of more than 32 fragments
    go to the kernel that gives a wave to each list, whose grid already uses y for its replicas (the view is z there),
    and the replicas' background rows are folded per view. Five views = a round of four and a round of one."""
    scene = _scene(5, 70, num_points=20_000)
    scene.max_list_length = max_list_length
    params = make_params(scene, need_point_gradient=1, render_mode=abi.RENDER_FUZZY_BLEND, depth_accept_blend=0.05)
    assert params.debug_max_list_length == max_list_length
    res = rasterizer.forward(DeviceScene(scene), params)
    go = scene.grad_out()
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go], want_cameras=True)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    ref = oracle.forward(scene, params)
    lengths = np.diff(ref.offsets[4].astype(np.int64))
    assert lengths.max() > 64  # long lists exist, in the last view too
    want = oracle.backward(ref, go, want_cameras=True)
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    for key in ("texture", "confidence", "background", "points", "pose", "intrinsics"):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        assert err <= (3e-4 if key in ("pose", "intrinsics") else 1e-4), (key, err)


@pytest.mark.parametrize("render_mode", [abi.RENDER_FULL_BLEND, abi.RENDER_BILINEAR_BLEND])
def test_views_that_see_little_interleave_the_rows_they_need(render_mode, rasterizer, oracle):
    """With hints that say "a small part of the cloud" (and neither texture index nor processing order) every view's
    scatter pass interleaves the descriptor rows of the points it sees instead of the first view's taking all rows.
    Five crops (two rounds) into a workspace filled with NaN bit patterns beforehand: whatever row a fragment or a
    gradient needs has been written by this call; rows of points that no view sees stay untouched."""
    scene = synthetic.tiny_scene(num_points=6000, w=96, h=64, num_layers=3, K=8, seed=99)
    scene.views = [synthetic.ViewSpec(32, 24, image_index=0, crop_transform=(1.0, 1.0, -float(ox), -float(oy), 0.0))
                   for (ox, oy) in ((0, 0), (40, 10), (64, 40), (20, 30), (50, 0))]
    params = make_params(scene, need_point_gradient=1, render_mode=render_mode)
    for l in range(scene.num_layers):
        params.expected_fragments[l] = 40.0
    dev = DeviceScene(scene)
    first = rasterizer.forward(dev, params)  # (for the size of the workspace)
    workspace = torch.full_like(first.workspace, 0xFF)
    res = rasterizer.forward(dev, params, workspace=workspace)
    go = scene.grad_out()
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go])
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    ref = oracle.forward(scene, params)
    want = oracle.backward(ref, go)
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    for key in ("texture", "confidence", "background", "points"):
        assert max_rel_err(got[key].cpu().numpy(), want[key]) <= 1e-4, key
    rows = res.workspace[res.layout.packed_base:res.layout.packed_base + 32 * scene.num_points].view(torch.float32)
    rows = rows.reshape(scene.num_points, 8).cpu().numpy()
    written = ~np.isnan(rows[:, 0])
    assert 0 < written.sum() < scene.num_points  # some rows, not all of them
    np.testing.assert_array_equal(rows[written, :scene.num_channels], scene.texture.T[written])
    seen = np.zeros(scene.num_points, dtype=bool)
    for b in range(len(scene.views)):
        frag = res.fragments(b)
        ids = (frag & np.uint64(0xFFFFFFFF)).astype(np.int64)
        if render_mode == abi.RENDER_BILINEAR_BLEND:
            ids >>= 2
        seen[ids[: int(res.offsets(b)[-1])]] = True
    assert not (seen & ~written).any()


def test_a_call_of_many_views_equals_its_views_one_by_one(rasterizer):
    """Seven views in one call against seven calls of one view: images and lists bit for bit, and the gradients of the
    big call equal the sum of the single calls' gradients to rounding (the rows are added in view order either way)."""
    scene = _scene(7, 90, num_points=8000)
    params = make_params(scene, need_point_gradient=1)
    dev = DeviceScene(scene)
    go = scene.grad_out()
    res = rasterizer.forward(dev, params)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go], want_cameras=True)
    torch.cuda.synchronize()
    sums = None
    for b in range(7):
        import copy

        one = copy.copy(scene)
        one.views = [scene.views[b]]
        r1 = rasterizer.forward(DeviceScene(one), make_params(one, need_point_gradient=1))
        g1 = rasterizer.backward(r1, [torch.from_numpy(np.ascontiguousarray(g[b:b + 1])).cuda() for g in go],
                                 want_cameras=True)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(r1.offsets(0), res.offsets(b))
        m = kept_mask(res.offsets(b), params.debug_max_list_length)
        np.testing.assert_array_equal(r1.fragments(0)[m], res.fragments(b)[m])
        for l in range(scene.num_layers):
            assert torch.equal(r1.out[l][0], res.out[l][b])
        vals = {k: g1[k].double().cpu().numpy() for k in ("texture", "confidence", "background", "points", "pose")}
        sums = vals if sums is None else {k: sums[k] + vals[k] for k in vals}
    for k, v in sums.items():
        assert max_rel_err(got[k].cpu().numpy(), v) <= 1e-4, k  # (float32 results of seven calls summed in double)


@pytest.mark.parametrize("render_mode", [abi.RENDER_FULL_BLEND, abi.RENDER_BILINEAR_BLEND])
def test_a_call_of_several_rounds_replays_from_a_hip_graph(render_mode, rasterizer):
    """Six views (a round of four and a round of two) with camera gradients, captured on a side stream: every replay
    gives the bits of the eager call, with eager calls in between."""
    scene = _scene(6, 95, num_points=20_000)
    params = make_params(scene, need_point_gradient=1, render_mode=render_mode)
    dev = DeviceScene(scene)
    eager = rasterizer.forward(dev, params)
    go = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    eager_g = rasterizer.backward(eager, go, want_cameras=True)
    torch.cuda.synchronize()
    want_out = [o.clone() for o in eager.out]
    want_g = {k: v.clone() for k, v in eager_g.items() if k != "_args"}
    # a context whose very first calls are the captured ones (it must not have to create anything while it is captured)
    fresh = Rasterizer()
    lib, ctx = fresh.lib, fresh.ctx
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
        again = rasterizer.forward(dev, params)  # eager work between replays, in the same workspace
        torch.cuda.synchronize()
        assert torch.equal(again.out[0], want_out[0])


def test_two_contexts_with_lanes_on_two_streams(oracle):
    """Two contexts issue calls of five views on two caller streams at the same time (each call has its own workspace)."""
    scenes = [_scene(5, 97), _scene(5, 98)]
    rasts = [Rasterizer(), Rasterizer()]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    devs = [DeviceScene(s) for s in scenes]
    results = [None, None]
    torch.cuda.synchronize()
    for rep in range(3):
        for k in range(2):
            with torch.cuda.stream(streams[k]):
                results[k] = rasts[k].forward(devs[k], make_params(scenes[k]))
    torch.cuda.synchronize()
    for k in range(2):
        ref = oracle.forward(scenes[k], make_params(scenes[k]))
        for l in range(scenes[k].num_layers):
            np.testing.assert_array_equal(results[k].out[l].cpu().numpy(), ref.out[l])
