"""Pins the CPU oracle against what the mathematics fixes, independently of the oracle's own formulas.

The reference ships no tests, golden vectors or fixtures for this path, and it cannot be built here, so every piece
of the oracle is checked against something a plausible mistake (dropped term, wrong sign or index, transposed
operand) would break: a double-precision textbook pinhole model and scipy's quaternion routine, brute-force binning,
Python's own sort, closed forms of the blend, central differences of an independent float64 blend, finite-difference
Jacobians of the projection.
"""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

from vet_amd import abi, synthetic
from vet_amd.rasterizer import make_params, make_views


# ---------------------------------------------------------------------------------------------------------------------
# independent float64 models
# ---------------------------------------------------------------------------------------------------------------------
def project64(p, pose8, K5, crop5, rot4, w, h):
    """Textbook pinhole with zero distortion in float64 (the reference's own host restatement:
    src/lib/data/SceneData.cpp:28-36 and :1020-1049), then crop transform and rotation about (w//2, h//2)."""
    R = Rotation.from_quat(pose8[:4]).as_matrix()
    v = R @ np.asarray(p[:3], dtype=np.float64) + pose8[4:7]
    n = v[:2] / v[2]
    u = K5[0] * n[0] + K5[4] * n[1] + K5[2]
    vv = K5[1] * n[1] + K5[3]
    x = crop5[0] * u + crop5[4] * vv + crop5[2]
    y = crop5[1] * vv + crop5[3]
    c = np.array([w // 2, h // 2], dtype=np.float64)
    M = np.array([[rot4[0], rot4[1]], [rot4[2], rot4[3]]], dtype=np.float64)
    ip = M @ (np.array([x, y]) - c) + c
    return ip, v[2]


def blend64(tex, conf, bg, ids, use_env):
    """Front-to-back alpha compositing of one sorted list, float64. Returns colour [C] and final transmittance."""
    T = 1.0
    out = np.zeros(tex.shape[0])
    for i in ids:
        out += T * conf[i] * tex[:, i]
        T *= 1.0 - conf[i]
    if not use_env:
        out += T * bg
    return out, T


def lists_of(fwd, b=0):
    """{(layer, x, y): [point ids front to back]} for all non-empty pixels of the oracle result, cut to K."""
    K = fwd.params.debug_max_list_length
    res = {}
    for l, (w, h) in enumerate(fwd.sizes):
        for y in range(h):
            for x in range(w):
                lst = fwd.pixel_list(b, l, x, y)
                n = len(lst) if K <= 0 else min(K, len(lst))
                res[(l, x, y)] = [int(k & 0xFFFFFFFF) for k in lst[:n]]
    return res


# ---------------------------------------------------------------------------------------------------------------------
# projection
# ---------------------------------------------------------------------------------------------------------------------
def test_pose_conversion_matches_scipy(oracle):
    rng = np.random.default_rng(0)
    for _ in range(20):
        q = rng.normal(size=4)
        q /= np.linalg.norm(q)
        pose = np.concatenate([q, rng.normal(size=3), [0.0]])
        k = np.zeros(13, np.float32)
        k[:5] = [500, 510, 320, 240, 0.5]
        m = oracle.prepare_view(pose, k)
        R = np.array([m[0:3], m[4:7], m[8:11]], dtype=np.float64)
        np.testing.assert_allclose(R, Rotation.from_quat(q).as_matrix(), atol=1e-7)
        np.testing.assert_allclose([m[3], m[7], m[11]], pose[4:7], rtol=1e-7)
        np.testing.assert_array_equal(m[12:17], k[:5])


def test_projection_matches_textbook_pinhole(oracle):
    rng = np.random.default_rng(1)
    worst = 0.0
    for trial in range(200):
        q = rng.normal(size=4)
        q /= np.linalg.norm(q)
        pose = np.concatenate([q, rng.normal(size=3), [0.0]])
        k = np.zeros(13, np.float32)
        k[:5] = [400 + 300 * rng.random(), 400 + 300 * rng.random(), 300 + 50 * rng.random(), 200 + 50 * rng.random(),
                 rng.normal() * 2]
        view = abi.View()
        view.w, view.h = 640, 480
        ang = rng.normal() * 0.3
        crop = [0.5 + rng.random(), 0.5 + rng.random(), rng.normal() * 20, rng.normal() * 20, rng.normal() * 0.1]
        rot = [np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang)]
        view.crop_transform = (abi.C.c_float * 5)(*crop)
        view.crop_rotation = (abi.C.c_float * 4)(*rot)
        p = np.array([*rng.normal(size=3) * 2, 0.05], dtype=np.float32)
        m = oracle.prepare_view(pose, k)
        ok, got = oracle.project_point(m, view, p)
        crop32 = np.array(crop, np.float32).astype(np.float64)
        rot32 = np.array(rot, np.float32).astype(np.float64)
        ip, z = project64(p.astype(np.float64), pose, k[:5].astype(np.float64), crop32, rot32, 640, 480)
        assert ok == (z > 0)
        if not ok:
            continue
        if z < 0.05:
            continue  # near the camera plane float32 cancellation dominates
        assert got[2] == pytest.approx(z, rel=1e-5, abs=1e-5)
        scale = max(1.0, abs(ip[0]), abs(ip[1]))
        err = max(abs(got[0] - ip[0]), abs(got[1] - ip[1])) / scale
        worst = max(worst, err * z)  # error grows like 1/z
        assert err * min(z, 1.0) < 2e-4
        radius = k[0] * np.float32(crop[0]) * p[3] / z
        assert got[3] == pytest.approx(radius, rel=1e-5)
    assert worst > 0  # the loop did compare something


def test_points_behind_the_camera_are_rejected(oracle):
    pose = np.array([0, 0, 0, 1, 0, 0, 0, 0], dtype=np.float64)
    k = np.zeros(13, np.float32)
    k[:5] = [100, 100, 50, 50, 0]
    m = oracle.prepare_view(pose, k)
    view = make_views(synthetic.tiny_scene())[0]
    for z, want in ((1.0, True), (0.0, False), (-1.0, False), (1e-30, True)):
        ok, _ = oracle.project_point(m, view, np.array([0.1, 0.1, z, 0.01], np.float32))
        assert ok == want


# ---------------------------------------------------------------------------------------------------------------------
# count / scan / fill / sort
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("overrides", [{}, {"drop_out_points_by_radius": 1}], ids=["plain", "radius_dropout"])
def test_binning_matches_brute_force(oracle, overrides):
    scene = synthetic.tiny_scene(num_points=1500, w=24, h=16, num_layers=3, K=-1, seed=5, num_views=2)
    rng = np.random.default_rng(3)
    scene.dropout = (rng.random((2, scene.num_points)) < 0.2).astype(np.float32)
    params = make_params(scene, **overrides)
    fwd = oracle.forward(scene, params)
    views = make_views(scene)
    total_pairs = 0
    for b in range(2):
        m = oracle.prepare_view(scene.poses_se3[scene.views[b].image_index], scene.intrinsics[0])
        expected = {}
        for i in range(scene.num_points):
            if scene.dropout[b, i] == 1:
                continue
            ok, pr = oracle.project_point(m, views[b], scene.position[i])
            if not ok:
                continue
            ip = pr[:2].astype(np.float32).copy()
            radius = np.float32(pr[3])
            for l, (w, h) in enumerate(scene.layer_sizes()):
                if params.drop_out_points_by_radius and radius < np.float32(params.drop_out_radius_threshold):
                    break
                px, py = np.rint(ip)  # numpy rint is round-half-even, like __float2int_rn
                if 0 <= px < w and 0 <= py < h:
                    expected.setdefault((l, int(px), int(py)), []).append((float(pr[2]), i))
                ip = ip * np.float32(0.5)
                radius = radius * np.float32(0.5)
        for l, (w, h) in enumerate(fwd.sizes):
            for y in range(h):
                for x in range(w):
                    got = fwd.pixel_list(b, l, x, y)
                    want = sorted(expected.get((l, x, y), []))  # Python's tuple order: depth, then id
                    assert len(got) == len(want), (b, l, x, y)
                    got_pairs = [(float(np.uint32(k >> 32).view(np.float32)), int(k & 0xFFFFFFFF)) for k in got]
                    assert got_pairs == want
                    total_pairs += len(want)
        assert int(fwd.offsets[b, -1]) == sum(len(v) for v in expected.values())
    assert total_pairs > 2000
    # the scan is an exclusive prefix sum starting at zero
    assert np.all(fwd.offsets[:, 0] == 0) and np.all(np.diff(fwd.offsets.astype(np.int64), axis=1) >= 0)


def test_equal_depths_are_ordered_by_point_id(oracle):
    scene = synthetic.tiny_scene(num_points=64, K=-1, seed=2)
    scene.position[:, :3] = scene.position[0, :3]  # every point at the same place: same pixel, same depth
    fwd = oracle.forward(scene)
    lists = [v for v in lists_of(fwd).values() if v]
    assert len(lists) == scene.num_layers
    for ids in lists:
        assert ids == list(range(64))


# ---------------------------------------------------------------------------------------------------------------------
# blend
# ---------------------------------------------------------------------------------------------------------------------
def _single_pixel_scene(confs, texs, K=-1, channels=4):
    """All points on the optical axis at increasing depth: one list in the centre pixel of an 8x8 image."""
    n = len(confs)
    s = synthetic.tiny_scene(num_points=max(n, 1), w=8, h=8, num_layers=1, K=K, channels=channels, seed=1)
    s.position[:, 0] = 0
    s.position[:, 1] = 0
    s.position[:, 2] = np.arange(max(n, 1), dtype=np.float32)
    s.confidence[:] = np.asarray(confs, np.float32) if n else 0
    s.texture[:, :] = np.asarray(texs, np.float32).T if n else 0
    if n == 0:
        s.position[:, 2] = -10  # behind the camera: no fragment at all
    return s


def test_blend_closed_forms(oracle):
    bg = None
    # empty pixel -> background, weight 1
    s = _single_pixel_scene([], [])
    f = oracle.forward(s)
    bg = s.background
    np.testing.assert_array_equal(f.out[0][0, :, 4, 4], bg)
    assert np.all(f.weight == 1.0)
    # one fragment: c*t + (1-c)*bg
    s = _single_pixel_scene([0.3], [[1.0, 2.0, -3.0, 0.5]])
    f = oracle.forward(s)
    want = 0.3 * np.array([1.0, 2.0, -3.0, 0.5]) + 0.7 * s.background.astype(np.float64)
    np.testing.assert_allclose(f.out[0][0, :, 4, 4], want, rtol=1e-6)
    assert f.weight[0, 4 * 8 + 4] == pytest.approx(0.7, rel=1e-6)
    # n equal fragments: t*(1-(1-c)^n) + (1-c)^n * bg
    n, c = 7, 0.2
    t = np.array([0.5, -1.0, 2.0, 1.5])
    s = _single_pixel_scene([c] * n, [t] * n)
    f = oracle.forward(s)
    want = t * (1 - (1 - c) ** n) + (1 - c) ** n * s.background.astype(np.float64)
    np.testing.assert_allclose(f.out[0][0, :, 4, 4], want, rtol=2e-6)
    # an opaque fragment hides everything behind it, a transparent one changes nothing
    s = _single_pixel_scene([0.0, 1.0, 0.5], [[9, 9, 9, 9], [1, 2, 3, 4], [7, 7, 7, 7]])
    f = oracle.forward(s)
    np.testing.assert_array_equal(f.out[0][0, :, 4, 4], np.array([1, 2, 3, 4], np.float32))
    assert f.weight[0, 4 * 8 + 4] == 0.0
    # with an environment map the background is not blended
    f = oracle.forward(_single_pixel_scene([0.3], [[1.0, 2.0, -3.0, 0.5]]), use_environment_map=1)
    np.testing.assert_allclose(f.out[0][0, :, 4, 4], 0.3 * np.array([1.0, 2.0, -3.0, 0.5]), rtol=1e-6)
    # top-K cut: only the K nearest fragments are blended
    s = _single_pixel_scene([0.5, 0.5, 0.5], [[1, 1, 1, 1], [2, 2, 2, 2], [4, 4, 4, 4]], K=2)
    f = oracle.forward(s)
    want = 0.5 * 1 + 0.25 * 2 + 0.25 * s.background.astype(np.float64)
    np.testing.assert_allclose(f.out[0][0, :, 4, 4], want, rtol=1e-6)


def test_blend_is_a_partition_of_unity(oracle):
    scene = synthetic.tiny_scene(num_points=4000, K=6, seed=8)
    scene.texture[:] = 1.0
    scene.background[:] = 1.0
    f = oracle.forward(scene)
    for o in f.out:
        np.testing.assert_allclose(o, 1.0, atol=2e-6)


def test_blend_matches_float64_compositing(oracle):
    scene = synthetic.tiny_scene(num_points=2500, K=5, seed=6, channels=3)
    f = oracle.forward(scene)
    lists = lists_of(f)
    tex, conf, bg = (a.astype(np.float64) for a in (scene.texture, scene.confidence, scene.background))
    for (l, x, y), ids in lists.items():
        want, T = blend64(tex, conf, bg, ids, use_env=False)
        np.testing.assert_allclose(f.out[l][0, :, y, x], want, rtol=1e-5, atol=1e-6)
        assert f.weight[0, f.layer_base(l) + y * f.sizes[l][0] + x] == pytest.approx(T, rel=1e-5, abs=1e-7)
        # stored transmittance in front of every kept fragment
        q = f.layer_base(l) + y * f.sizes[l][0] + x
        o = int(f.offsets[0, q])
        Ti = 1.0
        for r, i in enumerate(ids):
            assert f.transmittance[0, o + r] == pytest.approx(Ti, rel=1e-5, abs=1e-7)
            Ti *= 1 - conf[i]


def test_background_mask(oracle):
    s = _single_pixel_scene([1.0], [[1, 2, 3, 4]])
    f = oracle.forward(s, output_background_mask=1, output_background_mask_value=0.25)
    m = f.out_mask[0][0, 0]
    assert m[4, 4] == 0.25  # weight == 0 there: CreateMask writes the background value (PointRenderer.cu:216-235)
    assert np.all(np.delete(m.reshape(-1), 4 * 8 + 4) == 1.0)


# ---------------------------------------------------------------------------------------------------------------------
# value gradients: central differences of the independent float64 blend with the lists frozen
# ---------------------------------------------------------------------------------------------------------------------
def _loss64(tex, conf, bg, lists, grad_out, use_env):
    total = 0.0
    for (l, x, y), ids in lists.items():
        out, _ = blend64(tex, conf, bg, ids, use_env)
        total += float(np.dot(out, grad_out[l][0, :, y, x].astype(np.float64)))
    return total


@pytest.mark.parametrize("use_env", [0, 1])
def test_value_gradients_match_central_differences(oracle, use_env):
    scene = synthetic.tiny_scene(num_points=500, w=12, h=8, num_layers=2, K=4, seed=10)
    f = oracle.forward(scene, use_environment_map=use_env)
    grad_out = scene.grad_out()
    g = oracle.backward(f, grad_out, want_points=False)
    lists = lists_of(f)
    tex, conf, bg = (a.astype(np.float64) for a in (scene.texture, scene.confidence, scene.background))
    used = sorted({i for ids in lists.values() for i in ids})
    rng = np.random.default_rng(4)
    eps = 1e-4
    scale_t = np.abs(g["texture"]).max()
    scale_c = np.abs(g["confidence"]).max()
    for i in rng.choice(used, size=25, replace=False):
        for ci in range(tex.shape[0]):
            tp, tm = tex.copy(), tex.copy()
            tp[ci, i] += eps
            tm[ci, i] -= eps
            fd = (_loss64(tp, conf, bg, lists, grad_out, use_env) - _loss64(tm, conf, bg, lists, grad_out, use_env)) / (2 * eps)
            assert g["texture"][ci, i] == pytest.approx(fd, rel=2e-3, abs=2e-4 * scale_t)
        cp, cm = conf.copy(), conf.copy()
        cp[i] += eps
        cm[i] -= eps
        fd = (_loss64(tex, cp, bg, lists, grad_out, use_env) - _loss64(tex, cm, bg, lists, grad_out, use_env)) / (2 * eps)
        assert g["confidence"][i] == pytest.approx(fd, rel=2e-3, abs=2e-4 * scale_c)
    for ci in range(tex.shape[0]):
        bp, bm = bg.copy(), bg.copy()
        bp[ci] += eps
        bm[ci] -= eps
        fd = (_loss64(tex, conf, bp, lists, grad_out, use_env) - _loss64(tex, conf, bm, lists, grad_out, use_env)) / (2 * eps)
        assert g["background"][ci] == pytest.approx(fd, rel=2e-3, abs=1e-3)
    # points that never made it into a kept list get no gradient
    unused = np.setdiff1d(np.arange(scene.num_points), used)
    assert np.all(g["texture"][:, unused] == 0) and np.all(g["confidence"][unused] == 0)


def test_gradient_of_a_constant_upstream_sums_to_the_pixel_count(oracle):
    """With upstream gradient 1 everywhere, sum_points d tex[ci] + d bg[ci] = number of pixels (partition of unity)."""
    scene = synthetic.tiny_scene(num_points=3000, K=6, seed=12)
    f = oracle.forward(scene)
    ones = [np.ones_like(o) for o in f.out]
    g = oracle.backward(f, ones, want_points=False)
    pixels = sum(w * h for w, h in f.sizes)
    for ci in range(scene.num_channels):
        assert g["texture"][ci].astype(np.float64).sum() + g["background"][ci] == pytest.approx(pixels, rel=1e-5)


def test_background_confidence_leak_switch(oracle):
    """The reference adds the background element's alpha gradient to confidence row 0 (RenderBackward.cu:1157)."""
    scene = synthetic.tiny_scene(num_points=800, K=4, seed=13)
    f = oracle.forward(scene)
    go = scene.grad_out()
    off = oracle.backward(f, go, want_points=False)
    on = oracle.backward(f, go, want_points=False, quirk_background_confidence_leak=1)
    np.testing.assert_array_equal(on["confidence"][1:], off["confidence"][1:])
    np.testing.assert_array_equal(on["texture"], off["texture"])
    leak = 0.0
    bg = scene.background.astype(np.float64)
    for l, (w, h) in enumerate(f.sizes):
        T = f.weight[0, f.layer_base(l):f.layer_base(l) + w * h].reshape(h, w).astype(np.float64)
        leak += float((T * np.tensordot(bg, go[l][0].astype(np.float64), axes=(0, 0))).sum())
    assert on["confidence"][0] - off["confidence"][0] == pytest.approx(leak, rel=1e-4)


# ---------------------------------------------------------------------------------------------------------------------
# position gradient
# ---------------------------------------------------------------------------------------------------------------------
def test_position_gradient_chain_and_counts(oracle):
    """g_point = J^T dR/dp with J the finite-difference Jacobian of the float64 projection at the layer's scale, and
    dR/dp the neighbour-difference heuristic evaluated by hand from the forward image and the upstream gradient."""
    scene = synthetic.tiny_scene(num_points=700, w=24, h=16, num_layers=2, K=3, seed=17)
    ang = 0.2
    scene.views[0].crop_transform = (1.1, 0.9, 1.5, -2.0, 0.05)
    scene.views[0].crop_rotation = (np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang))
    scene.intrinsics[0, 4] = 0.3
    q = np.array([0.05, -0.03, 0.02, 1.0])
    scene.poses_se3[0, :4] = q / np.linalg.norm(q)
    params = make_params(scene, need_point_gradient=1)
    f = oracle.forward(scene, params)
    go = scene.grad_out()
    g = oracle.backward(f, go)
    lists = lists_of(f)
    tex = scene.texture.astype(np.float64)
    v = scene.views[0]
    crop32 = np.array(v.crop_transform, np.float32).astype(np.float64)
    rot32 = np.array(v.crop_rotation, np.float32).astype(np.float64)
    K5 = scene.intrinsics[0, :5].astype(np.float64)
    want = np.zeros((scene.num_points, 3))
    count = np.zeros(scene.num_points)
    Cn = scene.num_channels
    for (l, x, y), ids in lists.items():
        w, h = f.sizes[l]
        if min(x, y, w - 1 - x, h - 1 - y) <= 2:
            continue
        I, G = f.out[l][0].astype(np.float64), go[l][0].astype(np.float64)
        for i in ids:
            t = tex[:, i]
            dx = 0.5 * (-(t - I[:, y, x - 1]) * G[:, y, x - 1] + (t - I[:, y, x + 1]) * G[:, y, x + 1]).sum() / Cn
            dy = 0.5 * (-(t - I[:, y - 1, x]) * G[:, y - 1, x] + (t - I[:, y + 1, x]) * G[:, y + 1, x]).sum() / Cn
            p = scene.position[i].astype(np.float64)
            J = np.zeros((2, 3))
            for k in range(3):
                e = np.zeros(4)
                e[k] = 1e-6
                ip1, _ = project64(p + e, scene.poses_se3[0], K5, crop32, rot32, v.w, v.h)
                ip0, _ = project64(p - e, scene.poses_se3[0], K5, crop32, rot32, v.w, v.h)
                J[:, k] = (ip1 - ip0) / 2e-6
            want[i] += (0.5 ** l) * (J.T @ np.array([dx, dy]))
            count[i] += 1
    np.testing.assert_array_equal(g["point_count"], count.astype(np.float32))
    assert count.sum() > 100
    scale = np.abs(want).max()
    np.testing.assert_allclose(g["points"][:, :3], want, rtol=2e-3, atol=2e-4 * scale)
    assert np.all(g["points"][:, 3] == 0)


@pytest.mark.parametrize("mode", ["full", "fuzzy"])
def test_position_heuristic_on_a_case_worked_out_by_hand(mode, oracle):
    """Literal numbers, not a second copy of the formula: two fragments in the centre pixel of a 7x7 image, their four
    neighbours with known colours and upstream gradients (RenderBackward.cu:1346-1377; :729-1080 for FUZZY_BLEND)."""
    from tests.helpers import check_hand_case, hand_case

    scene, grad_out, expected = hand_case()
    extra = dict(render_mode=abi.RENDER_FUZZY_BLEND, depth_accept_blend=0.01) if mode == "fuzzy" else {}
    f = oracle.forward(scene, make_params(scene, need_point_gradient=1, **extra))
    g = oracle.backward(f, grad_out)
    check_hand_case(f.out[0], g["points"], g["point_count"], expected[mode])


def test_point_gradient_normalization_modes(oracle):
    scene = synthetic.tiny_scene(num_points=900, K=4, seed=18)
    f = oracle.forward(scene, need_point_gradient=1)
    go = scene.grad_out()
    raw = oracle.backward(f, go)
    n1 = oracle.backward(f, go, point_gradient_normalization=1)
    n2 = oracle.backward(f, go, point_gradient_normalization=2)
    cnt = raw["point_count"]
    safe = np.where(cnt > 0, cnt, 1).astype(np.float32)
    np.testing.assert_array_equal(n1["points"][:, :3], raw["points"][:, :3] / safe[:, None])
    # literal reference: the [N,4] buffer walked as N vec3 (PointRenderer.cu:1278-1279)
    flat = raw["points"].reshape(-1).copy()
    for i in range(scene.num_points):
        if cnt[i] > 0:
            flat[3 * i:3 * i + 3] /= cnt[i]
    np.testing.assert_array_equal(n2["points"].reshape(-1), flat)


# ---------------------------------------------------------------------------------------------------------------------
# error behaviour and threads
# ---------------------------------------------------------------------------------------------------------------------
def test_oracle_rejects_what_it_cannot_pin(oracle):
    scene = synthetic.tiny_scene()
    scene.intrinsics[0, 5] = 0.1  # k1 != 0: saiga's distortion model is not available
    with pytest.raises(abi.VetrastError) as e:
        oracle.forward(scene)
    assert e.value.status == abi.ERR_BAD_INPUT_DATA
    scene = synthetic.tiny_scene()
    scene.views[0].camera_model_type = abi.CAMERA_OCAM
    with pytest.raises(abi.VetrastError) as e:
        oracle.forward(scene)
    assert e.value.status == abi.ERR_UNSUPPORTED
    with pytest.raises(abi.VetrastError) as e:
        oracle.forward(synthetic.tiny_scene(), check_normal=1)
    assert e.value.status == abi.ERR_UNSUPPORTED


def test_threaded_oracle_agrees_with_single_thread(oracle):
    scene = synthetic.config2(num_points=40_000, w=480, h=270)
    a = oracle.forward(scene, num_threads=1)
    b = oracle.forward(scene, num_threads=4)
    np.testing.assert_array_equal(a.offsets, b.offsets)
    np.testing.assert_array_equal(a.fragments, b.fragments)
    for x, y in zip(a.out, b.out):
        np.testing.assert_array_equal(x, y)
    go = scene.grad_out()
    ga = oracle.backward(a, go, need_point_gradient=1)
    gb = oracle.backward(b, go, num_threads=4, need_point_gradient=1)
    for k in ("texture", "confidence", "points"):
        np.testing.assert_allclose(ga[k], gb[k], rtol=1e-4, atol=1e-5 * np.abs(ga[k]).max())


# ---------------------------------------------------------------------------------------------------------------------
# pose and intrinsics gradients
# ---------------------------------------------------------------------------------------------------------------------
def project64_camera(p, R, t, K5, crop5, rot4, w, h):
    v = R @ np.asarray(p[:3], dtype=np.float64) + t
    n = v[:2] / v[2]
    u = K5[0] * n[0] + K5[4] * n[1] + K5[2]
    vv = K5[1] * n[1] + K5[3]
    x = crop5[0] * u + crop5[4] * vv + crop5[2]
    y = crop5[1] * vv + crop5[3]
    c = np.array([w // 2, h // 2], dtype=np.float64)
    M = np.array([[rot4[0], rot4[1]], [rot4[2], rot4[3]]], dtype=np.float64)
    return M @ (np.array([x, y]) - c) + c


def test_pose_and_intrinsics_gradients(oracle):
    """Camera gradients = sum over fragments of J^T dR/dp, with J the finite-difference Jacobian of the float64
    projection with respect to (a) the se3 tangent applied on the left, pose <- exp(tangent) * pose, as ApplyTangent does
    (src/lib/rendering/PointRenderer.cu:1325-1341), order (translation, rotation), and (b) fx, fy, cx, cy (skew zeroed,
    scaled by K_gradient_factor). Counts grow by 1/1024 per fragment."""
    scene = synthetic.tiny_scene(num_points=500, w=24, h=16, num_layers=2, K=3, seed=19)
    ang = -0.15
    scene.views[0].crop_transform = (1.05, 0.95, 0.5, 1.0, 0.02)
    scene.views[0].crop_rotation = (np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang))
    scene.intrinsics[0, 4] = 0.2
    q = np.array([0.03, 0.04, -0.02, 1.0])
    scene.poses_se3[0, :4] = q / np.linalg.norm(q)
    params = make_params(scene, need_point_gradient=1, K_gradient_factor=0.5)
    f = oracle.forward(scene, params)
    go = scene.grad_out()
    g = oracle.backward(f, go, want_cameras=True)
    lists = lists_of(f)
    tex = scene.texture.astype(np.float64)
    v = scene.views[0]
    crop32 = np.array(v.crop_transform, np.float32).astype(np.float64)
    rot32 = np.array(v.crop_rotation, np.float32).astype(np.float64)
    K5 = scene.intrinsics[0, :5].astype(np.float64)
    R0 = Rotation.from_quat(scene.poses_se3[0, :4]).as_matrix()
    t0 = scene.poses_se3[0, 4:7].copy()
    want_pose, want_k, n_frag = np.zeros(6), np.zeros(5), 0
    Cn = scene.num_channels
    eps = 1e-6
    for (l, x, y), ids in lists.items():
        w, h = f.sizes[l]
        if min(x, y, w - 1 - x, h - 1 - y) <= 2:
            continue
        I, G = f.out[l][0].astype(np.float64), go[l][0].astype(np.float64)
        for i in ids:
            t = tex[:, i]
            dx = 0.5 * (-(t - I[:, y, x - 1]) * G[:, y, x - 1] + (t - I[:, y, x + 1]) * G[:, y, x + 1]).sum() / Cn
            dy = 0.5 * (-(t - I[:, y - 1, x]) * G[:, y - 1, x] + (t - I[:, y + 1, x]) * G[:, y + 1, x]).sum() / Cn
            grad = (0.5 ** l) * np.array([dx, dy])
            p = scene.position[i].astype(np.float64)
            for k in range(6):
                xi = np.zeros(6)
                ips = []
                for sgn in (+1, -1):
                    xi[:] = 0
                    xi[k] = sgn * eps
                    Rw = Rotation.from_rotvec(xi[3:]).as_matrix()
                    ips.append(project64_camera(p, Rw @ R0, Rw @ t0 + xi[:3], K5, crop32, rot32, v.w, v.h))
                want_pose[k] += grad @ ((ips[0] - ips[1]) / (2 * eps))
            for k in range(4):  # fx, fy, cx, cy; the skew column is zeroed by the reference
                Kp, Km = K5.copy(), K5.copy()
                h_k = 1e-4
                Kp[k] += h_k
                Km[k] -= h_k
                d = project64_camera(p, R0, t0, Kp, crop32, rot32, v.w, v.h) - project64_camera(p, R0, t0, Km, crop32, rot32, v.w, v.h)
                want_k[k] += 0.5 * (grad @ (d / (2 * h_k)))
            n_frag += 1
    assert n_frag > 100
    assert g["pose_count"][0] == pytest.approx(n_frag / 1024.0, rel=1e-5)
    assert g["intrinsics_count"][0] == pytest.approx(n_frag / 1024.0, rel=1e-5)
    np.testing.assert_allclose(g["pose"][0], want_pose, rtol=2e-3, atol=2e-4 * np.abs(want_pose).max())
    np.testing.assert_allclose(g["intrinsics"][0, :5], want_k, rtol=2e-3, atol=2e-4 * np.abs(want_k).max())
    assert np.all(g["intrinsics"][0, 4:] == 0)
    # normalisation: every row divided by its count (1024 x the mean over fragments)
    gn = oracle.backward(f, go, want_cameras=True, camera_gradient_normalization=1)
    np.testing.assert_allclose(gn["pose"][0], g["pose"][0] / g["pose_count"][0], rtol=1e-6)
    np.testing.assert_allclose(gn["intrinsics"][0], g["intrinsics"][0] / g["intrinsics_count"][0], rtol=1e-6)
