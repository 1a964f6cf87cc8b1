"""Pins the oracle's BILINEAR_BLEND mode (render_mode 3) against what the mathematics fixes.

The reference holds no test, vector or fixture for this mode either. What pins it: brute-force binning of the 2x2
splat, the closed forms of bilinear weights (they sum to one; a point on a pixel centre has weight one there), an
independent float64 compositing model with its own textbook projection, and central differences of that model. The
position gradient is analytic in this mode (the derivative of the bilinear weights), so finite differences pin it,
unlike the heuristic of the other mode.
"""
import numpy as np
import pytest

from tests.test_oracle_pinning import project64
from vet_amd import abi, synthetic
from vet_amd.rasterizer import make_params

MODE = dict(render_mode=abi.RENDER_BILINEAR_BLEND)


def _scene(num_points=150, seed=31, K=-1, w=24, h=16, layers=3, channels=4):
    s = synthetic.tiny_scene(num_points=num_points, w=w, h=h, num_layers=layers, K=K, seed=seed, channels=channels)
    return s


def _uv64(scene, i, l, b=0):
    v = scene.views[b]
    ip, z = project64(scene.position[i], scene.poses_se3[v.image_index], scene.intrinsics[v.camera_index][:5],
                      np.asarray(v.crop_transform, np.float64), np.asarray(v.crop_rotation, np.float64), v.w, v.h)
    return ip * 0.5 ** l, z


def _weights64(uv):
    s = uv - np.floor(uv)
    return np.array([(1 - s[0]) * (1 - s[1]), s[0] * (1 - s[1]), (1 - s[0]) * s[1], s[0] * s[1]])


def _lists(fwd, b=0):
    """{(l, x, y): [(point id, corner)]} of all pixels, in the oracle's sorted order, cut to K."""
    K = fwd.params.debug_max_list_length
    res = {}
    for l, (w, h) in enumerate(fwd.sizes):
        for y in range(h):
            for x in range(w):
                lst = fwd.pixel_list(b, l, x, y)
                n = len(lst) if K <= 0 else min(K, len(lst))
                res[(l, x, y)] = [(int(k & 0xFFFFFFFF) >> 2, int(k & 3)) for k in lst[:n]]
    return res


def test_binning_is_the_2x2_splat_by_brute_force(oracle):
    scene = _scene(num_points=400, seed=32)
    # the oracle floors the float32 position: drop the (rare) points this float64 check cannot place for certain
    sizes = scene.layer_sizes()
    clear = [i for i in range(scene.num_points)
             if all(np.min(np.abs(_uv64(scene, i, l)[0] - np.round(_uv64(scene, i, l)[0]))) > 1e-4 for l in range(len(sizes)))]
    assert len(clear) > 390
    scene.position = np.ascontiguousarray(scene.position[clear])
    scene.texture = np.ascontiguousarray(scene.texture[:, clear])
    scene.confidence = np.ascontiguousarray(scene.confidence[clear])
    fwd = oracle.forward(scene, **MODE)
    want = {}
    for i in range(scene.num_points):
        for l, (w, h) in enumerate(fwd.sizes):
            uv, z = _uv64(scene, i, l)
            if z <= 0:
                continue
            x0, y0 = int(np.floor(uv[0])), int(np.floor(uv[1]))
            for dy in (0, 1):
                for dx in (0, 1):
                    x, y = x0 + dx, y0 + dy
                    if 0 <= x < w and 0 <= y < h:
                        want.setdefault((l, x, y), set()).add((i, dy * 2 + dx))
    got = {k: set(v) for k, v in _lists(fwd).items() if v}
    assert got == want
    # lists are sorted by (depth, id, corner)
    for (l, x, y), lst in _lists(fwd).items():
        keys = fwd.pixel_list(0, l, x, y)
        assert np.all(keys[:-1] < keys[1:])


def test_weights_of_a_point_sum_to_one_and_a_centred_point_fills_one_pixel(oracle):
    """Descriptor 1, confidence c, black background, one point: the 2x2 pixels hold c * weight, which adds up to c;
    a point exactly on a pixel centre gives c there and 0 in the three others (still four fragments)."""
    scene = _scene(num_points=1, layers=1)
    scene.texture[:] = 1.0
    scene.background[:] = 0.0
    scene.confidence[:] = 0.75
    f = float(scene.intrinsics[0, 0])
    cx, cy = float(scene.intrinsics[0, 2]), float(scene.intrinsics[0, 3])
    z = float(scene.poses_se3[0, 6])
    for target in ((7.3, 5.6), (10.0, 8.0), (3.999, 4.001)):
        scene.position[0, :3] = ((target[0] - cx) / f * (z + 0.5), (target[1] - cy) / f * (z + 0.5), 0.5)
        fwd = oracle.forward(scene, **MODE)
        img = fwd.out[0][0, 0].astype(np.float64)
        uv, _ = _uv64(scene, 0, 0)
        assert np.allclose(uv, target, atol=1e-4)
        assert int(fwd.offsets[0, -1]) == 4
        assert abs(img.sum() - 0.75) < 1e-6
        x0, y0 = int(np.floor(uv[0])), int(np.floor(uv[1]))
        wts = _weights64(uv)
        for k in range(4):
            assert abs(img[y0 + k // 2, x0 + k % 2] - 0.75 * wts[k]) < 2e-4  # uv itself is only float32-accurate
        if target == (10.0, 8.0):
            assert abs(img[8, 10] - 0.75) < 1e-5 and np.count_nonzero(img) == 1


def _blend64(scene, lists, l_x_y, use_env, cutoff=True):
    """Independent float64 compositing of one pixel. Returns colour, final T, number of fragments that took part and
    the smallest distance of any running T from the 0.001 cut (to tell robust cases from borderline ones)."""
    l = l_x_y[0]
    T, out, used, margin = 1.0, np.zeros(scene.num_channels), 0, 1.0
    for (i, corner) in lists[l_x_y]:
        uv, _ = _uv64(scene, i, l)
        alpha = _weights64(uv)[corner] * float(scene.confidence[i])
        out += T * alpha * scene.texture[:, i].astype(np.float64)
        T *= 1.0 - alpha
        used += 1
        margin = min(margin, abs(T - 0.001))
        if cutoff and T < 0.001:
            break
    if not use_env and T >= 0.001:
        out += T * scene.background.astype(np.float64)
    return out, T, used, margin


@pytest.mark.parametrize("use_env", [0, 1])
def test_blend_matches_float64_compositing_with_the_early_exit(oracle, use_env):
    scene = _scene(num_points=2500, seed=33, K=-1)
    scene.confidence[:] = np.clip(scene.confidence * 1.6, 0, 0.98)  # opaque enough for the cut to trigger
    fwd = oracle.forward(scene, use_environment_map=use_env, **MODE)
    lists = _lists(fwd)
    cut_pixels = 0
    for l, (w, h) in enumerate(fwd.sizes):
        base = fwd.layer_base(l)
        for y in range(h):
            for x in range(w):
                want, T, used, margin = _blend64(scene, lists, (l, x, y), use_env)
                if margin < 1e-5:
                    continue  # float32 and float64 may disagree on which side of 0.001 this pixel falls
                assert int(fwd.kept[0, base + y * w + x]) == used
                cut_pixels += used < len(lists[(l, x, y)])
                assert np.allclose(fwd.out[l][0, :, y, x], want, rtol=2e-4, atol=2e-5)
                assert abs(float(fwd.weight[0, base + y * w + x]) - T) < 1e-5
    assert cut_pixels > 20, "the scene must exercise the early exit"


def _loss64(scene, lists, kept, grad_out, use_env, sizes):
    """sum(out * grad_out) of the float64 model with the lists and the number of blended fragments frozen."""
    total = 0.0
    for (l, x, y), lst in lists.items():
        T, out = 1.0, np.zeros(scene.num_channels)
        n = kept[(l, x, y)]
        for (i, corner) in lst[:n]:
            uv, _ = _uv64(scene, i, l)
            alpha = _weights64(uv)[corner] * float(scene.confidence[i])
            out += T * alpha * scene.texture[:, i].astype(np.float64)
            T *= 1.0 - alpha
        if not use_env and (n == len(lst) or T >= 0.001) and T >= 0.001:
            out += T * scene.background.astype(np.float64)
        total += float((out * grad_out[l][0, :, y, x]).sum())
    return total


@pytest.mark.parametrize("use_env", [0, 1])
def test_gradients_match_central_differences(oracle, use_env):
    """Descriptor, confidence, background and POSITION gradients against central differences of the float64 model.
    The reference only forms confidence and position gradients at pixels more than 2 away from the border
    (src/lib/rendering/RenderBackward.cu:3044), so the upstream gradient is zero in that rim."""
    scene = _scene(num_points=260, seed=34, K=6, w=20, h=14, layers=2)
    scene.position = scene.position.astype(np.float64).astype(np.float32)
    fwd = oracle.forward(scene, use_environment_map=use_env, need_point_gradient=1, **MODE)
    rng = np.random.default_rng(5)
    grad_out = []
    for (w, h) in fwd.sizes:
        g = rng.standard_normal((1, scene.num_channels, h, w)).astype(np.float32)
        g[:, :, :3, :] = 0
        g[:, :, -3:, :] = 0
        g[:, :, :, :3] = 0
        g[:, :, :, -3:] = 0
        grad_out.append(g)
    got = oracle.backward(fwd, grad_out, want_points=True)
    lists = _lists(fwd)
    kept = {}
    for l, (w, h) in enumerate(fwd.sizes):
        for y in range(h):
            for x in range(w):
                kept[(l, x, y)] = int(fwd.kept[0, fwd.layer_base(l) + y * w + x])
    go64 = [g.astype(np.float64) for g in grad_out]

    def loss():
        return _loss64(scene, lists, kept, go64, use_env, fwd.sizes)

    def fd(arr, idx, eps):
        old = arr[idx]
        arr[idx] = old + eps
        hi = loss()
        arr[idx] = old - eps
        lo = loss()
        arr[idx] = old
        return (hi - lo) / (2 * eps)

    visible = sorted({i for lst in lists.values() for (i, _) in lst})
    probe = visible[:: max(1, len(visible) // 12)][:12]
    tex64 = scene.texture.astype(np.float64)
    conf64 = scene.confidence.astype(np.float64)
    pos64 = scene.position.astype(np.float64)
    bg64 = scene.background.astype(np.float64)
    scene.texture, scene.confidence, scene.position, scene.background = tex64, conf64, pos64, bg64
    scale = max(1.0, float(np.abs(got["confidence"]).max()))
    for i in probe:
        assert abs(fd(scene.confidence, i, 1e-6) - got["confidence"][i]) <= 2e-3 * scale, ("confidence", i)
        for c in range(scene.num_channels):
            assert abs(fd(scene.texture, (c, i), 1e-6) - got["texture"][c, i]) <= 2e-3 * scale, ("texture", c, i)
    pscale = max(1.0, float(np.abs(got["points"]).max()))
    checked = 0
    for i in probe:
        # a finite step must not carry the point over a pixel border in any layer
        ok = all(np.min(np.abs(_uv64(scene, i, l)[0] - np.round(_uv64(scene, i, l)[0]))) > 5e-3 for l in range(len(fwd.sizes)))
        if not ok:
            continue
        for k in range(3):
            assert abs(fd(scene.position, (i, k), 1e-5) - got["points"][i, k]) <= 3e-3 * pscale, ("position", i, k)
        checked += 1
    assert checked >= 6
    if not use_env:
        for c in range(scene.num_channels):
            assert abs(fd(scene.background, c, 1e-6) - got["background"][c]) <= 2e-3 * max(1.0, abs(got["background"][c]))
    # one count per fragment that received a position gradient
    interior = 0
    for (l, x, y), lst in lists.items():
        w, h = fwd.sizes[l]
        if min(x, y, w - 1 - x, h - 1 - y) > 2:
            interior += kept[(l, x, y)]
    assert got["point_count"].sum() == interior


def test_confidence_gradient_skips_the_rim_but_descriptor_gradient_does_not(oracle):
    """Literal behaviour: with an upstream gradient only in the rim (distance from the border <= 2) the descriptor and
    background gradients are non-zero while confidence and position gradients stay exactly zero."""
    scene = _scene(num_points=600, seed=35, K=8)
    fwd = oracle.forward(scene, need_point_gradient=1, **MODE)
    grad_out = []
    for (w, h) in fwd.sizes:
        g = np.ones((1, scene.num_channels, h, w), np.float32)
        g[:, :, 3:-3, 3:-3] = 0
        grad_out.append(g)
    got = oracle.backward(fwd, grad_out, want_points=True)
    assert np.abs(got["texture"]).sum() > 0 and np.abs(got["background"]).sum() > 0
    assert not got["confidence"].any() and not got["points"].any()
    assert got["point_count"].sum() > 0  # interior fragments are still counted, their gradient is just zero


def test_pose_count_grows_by_one_per_fragment_in_this_mode(oracle):
    scene = _scene(num_points=300, seed=36, K=8)
    fwd = oracle.forward(scene, need_point_gradient=1, **MODE)
    grad_out = [np.ones((1, scene.num_channels, h, w), np.float32) for (w, h) in fwd.sizes]
    got = oracle.backward(fwd, grad_out, want_points=True, want_cameras=True)
    n = float(got["point_count"].sum())
    assert n > 0 and got["pose_count"][0] == n  # +1 per fragment (RenderBackward.cu:3146)
    assert abs(got["intrinsics_count"][0] - n / 1024.0) < 1e-3  # +1/1024 per fragment (:3174)


def test_threaded_oracle_agrees(oracle):
    scene = _scene(num_points=3000, seed=37, K=8)
    a = oracle.forward(scene, need_point_gradient=1, **MODE)
    b = oracle.forward(scene, need_point_gradient=1, num_threads=4, **MODE)
    assert np.array_equal(a.offsets, b.offsets) and np.array_equal(a.kept, b.kept)
    for x, y in zip(a.out, b.out):
        assert np.array_equal(x, y)
    go = [np.random.default_rng(1).standard_normal(o.shape).astype(np.float32) for o in a.out]
    ga = oracle.backward(a, go)
    gb = oracle.backward(b, go, num_threads=4)
    for k in ("texture", "confidence", "points"):
        assert np.allclose(ga[k], gb[k], rtol=1e-4, atol=1e-5 * max(1.0, np.abs(ga[k]).max()))


@pytest.mark.parametrize("use_env", [0, 1])
def test_suffix_sum_model_of_the_backward_pass_agrees_on_short_lists(oracle, use_env):
    """The O(n) float64 model that the GPU test of long lists is checked against (tests/helpers.py) gives what the
    oracle's literal O(n^2) loop gives (RenderBackward.cu:2987-3012), early exit, texture index and rim included."""
    from tests.helpers import bilinear_backward_model, max_rel_err

    scene = _scene(num_points=1500, seed=36, K=-1)
    scene.confidence[:] = np.clip(scene.confidence * 1.6, 0, 0.98)  # so that the 0.001 cut triggers
    rng = np.random.default_rng(8)
    scene.index = rng.integers(0, 400, size=scene.num_points).astype(np.int32)
    fwd = oracle.forward(scene, use_environment_map=use_env, need_point_gradient=1, **MODE)
    grad_out = scene.grad_out()
    got = oracle.backward(fwd, grad_out, want_points=True)
    want = bilinear_backward_model(oracle, fwd, grad_out, use_env=bool(use_env))
    full = np.diff(fwd.offsets[0].astype(np.int64))
    assert (fwd.kept[0] < full).sum() > 20, "the early exit must be exercised"
    np.testing.assert_array_equal(got["point_count"], want["point_count"])
    for key in ("texture", "confidence", "points") + (() if use_env else ("background",)):
        assert max_rel_err(got[key], want[key]) <= 1e-4, key
