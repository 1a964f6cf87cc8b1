"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same seeded inputs.

Bars: per-pixel counts, scan and the kept part of every fragment list bit-exact; blended features within 1e-5
relative (they are in fact computed in the same operation order, the test also reports exact equality); gradients
within 1e-4 relative (atomic accumulation order differs).
"""
import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu

FEATURE_TOL = 1e-5
GRAD_TOL = 1e-4


def _scenes():
    yield "tiny_K4", synthetic.tiny_scene(), {}
    yield "tiny_dense_K4", synthetic.tiny_scene(num_points=6000, K=4), {}
    yield "tiny_dense_nocut", synthetic.tiny_scene(num_points=6000, K=-1, seed=9), {}
    yield "tiny_dense_K16_3ch", synthetic.tiny_scene(num_points=5000, K=16, channels=3, seed=11), {}
    yield "tiny_long_lists_K16", synthetic.tiny_scene(num_points=40000, K=16, seed=12), {}
    yield "tiny_long_lists_nocut", synthetic.tiny_scene(num_points=40000, K=0, seed=13), {}
    yield "tiny_2views_envmap", synthetic.tiny_scene(num_points=3000, K=8, num_views=2, seed=14), {"use_environment_map": 1}
    yield "tiny_radius_dropout", synthetic.tiny_scene(num_points=3000, K=8, seed=15), {"drop_out_points_by_radius": 1}
    yield "config1", synthetic.config1(), {}
    yield "config2_200k", synthetic.config2(num_points=200_000), {}


SCENES = list(_scenes())


def _check_forward(scene, overrides, rasterizer, oracle):
    params = make_params(scene, **overrides)
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    K = params.debug_max_list_length
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64), err_msg="scan / per-pixel counts differ")
        total = int(off[-1])
        keep = kept_mask(off, K)
        got = res.fragments(b)
        np.testing.assert_array_equal(got[keep], ref.fragments[b, :total][keep], err_msg="fragment lists differ")
        np.testing.assert_array_equal(res.transmittance(b)[keep], ref.transmittance[b, :total][keep])
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    exact = True
    for l in range(scene.num_layers):
        got = res.out[l].cpu().numpy()
        assert max_rel_err(got, ref.out[l]) <= FEATURE_TOL
        exact &= bool(np.array_equal(got, ref.out[l]))
    return ref, dev, res, exact


@pytest.mark.parametrize("name,scene,overrides", SCENES, ids=[s[0] for s in SCENES])
def test_forward_matches_oracle(name, scene, overrides, rasterizer, oracle):
    print(f"[case] forward {name} N={scene.num_points}", flush=True)
    _, _, _, exact = _check_forward(scene, overrides, rasterizer, oracle)
    assert exact, "blend is computed in the oracle's operation order and should agree bit for bit"


@pytest.mark.parametrize("name,scene,overrides", SCENES, ids=[s[0] for s in SCENES])
def test_backward_matches_oracle(name, scene, overrides, rasterizer, oracle):
    print(f"[case] backward {name} N={scene.num_points}", flush=True)
    overrides = dict(overrides, need_point_gradient=1)
    ref, dev, res, _ = _check_forward(scene, overrides, rasterizer, oracle)
    grad_out = scene.grad_out()
    ref_g = oracle.backward(ref, grad_out)
    got_g = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got_g["point_count"].cpu().numpy(), ref_g["point_count"])
    for key in ("texture", "confidence", "background", "points"):
        err = max_rel_err(got_g[key].cpu().numpy(), ref_g[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= GRAD_TOL, key


@pytest.mark.parametrize("mode", ["full", "fuzzy"])
def test_position_heuristic_on_a_case_worked_out_by_hand(mode, rasterizer):
    """The literal expectations of tests/helpers.py::hand_case, no oracle in between
    (RenderBackward.cu:1346-1377; :729-1080 for FUZZY_BLEND)."""
    from tests.helpers import check_hand_case, hand_case

    scene, grad_out, expected = hand_case()
    extra = dict(render_mode=abi.RENDER_FUZZY_BLEND, depth_accept_blend=0.01) if mode == "fuzzy" else {}
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, make_params(scene, need_point_gradient=1, **extra))
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    check_hand_case(res.out[0].cpu().numpy(), got["points"].cpu().numpy(), got["point_count"].cpu().numpy(),
                    expected[mode])


@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND, abi.RENDER_BILINEAR_BLEND])
def test_processing_order_changes_nothing(mode, rasterizer):
    """vetrast_forward_args.point_order only tells the binning pass in which order to walk the points: lists, outputs
    and gradients are the same bits for any permutation (several views, radius drop-out on; no texture index, whose
    shared rows are summed with float atomics in arrival order)."""
    scene = synthetic.tiny_scene(num_points=7000, K=8, seed=41, num_views=2)
    rng = np.random.default_rng(11)
    params = make_params(scene, need_point_gradient=1, render_mode=mode, drop_out_points_by_radius=1)
    dev = DeviceScene(scene)
    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    plain = rasterizer.forward(dev, params)
    plain_g = {k: v.clone() for k, v in rasterizer.backward(plain, grad_out).items() if k != "_args"}
    for perm in (rng.permutation(scene.num_points), np.arange(scene.num_points)[::-1].copy()):
        order = torch.from_numpy(perm.astype(np.int32)).cuda()
        res = rasterizer.forward(dev, params, point_order=order)
        got = rasterizer.backward(res, grad_out)
        torch.cuda.synchronize()
        for b in range(2):
            np.testing.assert_array_equal(res.offsets(b), plain.offsets(b))
            np.testing.assert_array_equal(res.kept(b), plain.kept(b))
        for a, b in zip(res.out, plain.out):
            assert torch.equal(a, b)
        for k, v in plain_g.items():
            assert torch.equal(got[k], v), k


@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_BILINEAR_BLEND])
def test_expected_fragments_hint_changes_nothing(mode, rasterizer):
    """vetrast_params.expected_fragments only sizes the pixel bins: a crop that sees a part of the cloud gives the same
    lists, images and gradients with the true counts, with counts far too small (records overflow their bins' rooms
    and take the log path) and with counts far too large as with none."""
    scene = synthetic.config2(num_points=120_000, w=480, h=270, K=8)
    scene.views = [synthetic.ViewSpec(128, 96, crop_transform=(1.0, 1.0, -170.0, -90.0, 0.0)),
                   synthetic.ViewSpec(128, 96, crop_transform=(1.0, 1.0, -20.0, -150.0, 0.0))]
    dev = DeviceScene(scene)
    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    plain = rasterizer.forward(dev, make_params(scene, need_point_gradient=1, render_mode=mode))
    plain_g = {k: v.clone() for k, v in rasterizer.backward(plain, grad_out).items() if k != "_args"}
    off, bases = plain.offsets(0), plain.layer_bases()
    true_counts = [float(off[bases[l + 1]] - off[bases[l]]) for l in range(scene.num_layers)]
    assert 0 < sum(true_counts) < 0.5 * scene.num_points * scene.num_layers, "the crop must see a part of the cloud only"
    for hint in (true_counts, [1.0] * 4, [c * 50 for c in true_counts], [true_counts[0], 0.0, 3.0, 0.0]):
        res = rasterizer.forward(dev, make_params(scene, need_point_gradient=1, render_mode=mode, expected_fragments=hint))
        got = rasterizer.backward(res, grad_out)
        torch.cuda.synchronize()
        assert rasterizer.check_device_flags(res) == 0
        for b in range(2):
            np.testing.assert_array_equal(res.offsets(b), plain.offsets(b))
            kept = kept_mask(plain.offsets(b), scene.max_list_length)  # what lies behind the cut is in no particular order
            np.testing.assert_array_equal(res.fragments(b)[kept], plain.fragments(b)[kept])
        for a, b in zip(res.out, plain.out):
            assert torch.equal(a, b)
        for k, v in plain_g.items():
            assert torch.equal(got[k], v), k


def _backward_pair(scene, overrides, rasterizer, oracle, want_points=True):
    ref, dev, res, _ = _check_forward(scene, overrides, rasterizer, oracle)
    grad_out = scene.grad_out()
    ref_g = oracle.backward(ref, grad_out, want_points=want_points)
    got_g = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_points=want_points)
    torch.cuda.synchronize()
    return ref_g, {k: v.cpu().numpy() for k, v in got_g.items() if k != "_args"}


def test_backward_with_texture_index_indirection(rasterizer, oracle):
    """Several points share a descriptor row (t_index); descriptor/confidence gradients add up per row."""
    scene = synthetic.tiny_scene(num_points=5000, K=8, seed=21)
    rng = np.random.default_rng(5)
    scene.index = rng.integers(0, 700, size=scene.num_points).astype(np.int32)
    ref_g, got_g = _backward_pair(scene, {"need_point_gradient": 1}, rasterizer, oracle)
    np.testing.assert_array_equal(got_g["point_count"], ref_g["point_count"])
    for key in ("texture", "confidence", "background", "points"):
        assert max_rel_err(got_g[key], ref_g[key]) <= GRAD_TOL, key
    assert np.all(got_g["texture"][:, 700:] == 0)


@pytest.mark.parametrize("mode", [1, 2])
def test_point_gradient_normalization_modes(mode, rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=4000, K=8, seed=22)
    ref_g, got_g = _backward_pair(scene, {"need_point_gradient": 1, "point_gradient_normalization": mode}, rasterizer,
                                  oracle)
    assert max_rel_err(got_g["points"], ref_g["points"]) <= GRAD_TOL


def test_background_confidence_leak_switch(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=2000, K=8, seed=23)
    ref_g, got_g = _backward_pair(scene, {"quirk_background_confidence_leak": 1}, rasterizer, oracle)
    off_ref, _ = _backward_pair(scene, {}, rasterizer, oracle)
    assert abs(ref_g["confidence"][0] - off_ref["confidence"][0]) > 1e-3, "the switch must change row 0"
    assert max_rel_err(got_g["confidence"], ref_g["confidence"]) <= GRAD_TOL


def test_backward_without_point_gradient(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=2000, K=8, seed=24)
    ref_g, got_g = _backward_pair(scene, {"need_point_gradient": 0}, rasterizer, oracle, want_points=False)
    assert "points" not in got_g
    for key in ("texture", "confidence", "background"):
        assert max_rel_err(got_g[key], ref_g[key]) <= GRAD_TOL, key


def test_backward_is_reproducible(rasterizer):
    """No float atomics on the descriptor/confidence/position gradients: two runs agree bit for bit."""
    scene = synthetic.config2(num_points=100_000)
    dev = DeviceScene(scene)
    params = make_params(scene, need_point_gradient=1)
    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    runs = []
    for _ in range(2):
        res = rasterizer.forward(dev, params)
        g = rasterizer.backward(res, grad_out)
        torch.cuda.synchronize()
        runs.append({k: v.cpu().numpy() for k, v in g.items() if k != "_args"})
    for key in ("texture", "confidence", "points", "point_count"):
        np.testing.assert_array_equal(runs[0][key], runs[1][key])


@pytest.mark.parametrize("normalize", [0, 1])
def test_pose_and_intrinsics_gradients(normalize, rasterizer, oracle):
    """Camera gradients: per-workgroup sums in double on the GPU against the oracle's per-fragment accumulation."""
    scene = synthetic.tiny_scene(num_points=6000, K=8, seed=41, num_views=3)
    scene.views[2].image_index = 0  # two views share a pose row: their sums add up
    over = {"need_point_gradient": 1, "camera_gradient_normalization": normalize}
    ref, dev, res, _ = _check_forward(scene, over, rasterizer, oracle)
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_cameras=True)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_cameras=True)
    torch.cuda.synchronize()
    np.testing.assert_allclose(got["pose_count"].cpu().numpy(), want["pose_count"], rtol=1e-6)
    np.testing.assert_allclose(got["intrinsics_count"].cpu().numpy(), want["intrinsics_count"], rtol=1e-6)
    assert want["pose_count"][0] > want["pose_count"][1] > 0 and want["pose_count"][2] == 0
    for key in ("pose", "intrinsics", "points", "texture"):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= GRAD_TOL, key


def test_camera_gradients_without_point_gradient_buffer(rasterizer, oracle):
    scene = synthetic.tiny_scene(num_points=3000, K=8, seed=42)
    ref, dev, res, _ = _check_forward(scene, {"need_point_gradient": 1}, rasterizer, oracle)
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_points=False, want_cameras=True)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_points=False, want_cameras=True)
    torch.cuda.synchronize()
    assert max_rel_err(got["pose"].cpu().numpy(), want["pose"]) <= GRAD_TOL
    assert max_rel_err(got["intrinsics"].cpu().numpy(), want["intrinsics"]) <= GRAD_TOL


@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND, abi.RENDER_BILINEAR_BLEND])
def test_per_pixel_weight_output(mode, rasterizer, oracle):
    """The optional out_weight tensors: the transmittance behind the last blended fragment of every pixel in image order
    (the `weight` tensor of the reference's layer cache), 1 where no point landed, for every view and layer."""
    print(f"[case] per-pixel weight output mode={mode}", flush=True)
    scene = synthetic.tiny_scene(num_points=2500, K=6, seed=71, w=37, h=21, num_layers=3, num_views=2)
    scene.confidence[::4] = 1.0
    params = make_params(scene, render_mode=mode, depth_accept_blend=0.05)
    ref = oracle.forward(scene, params)
    res = rasterizer.forward(DeviceScene(scene), params, want_weight=True)
    torch.cuda.synchronize()
    assert res.out_weight is not None and len(res.out_weight) == scene.num_layers
    for b in range(len(scene.views)):
        got = np.concatenate([w[b].cpu().numpy().ravel() for w in res.out_weight])
        np.testing.assert_array_equal(got, ref.weight[b])
        assert (got == 1.0).any() and (got < 1.0).any()
