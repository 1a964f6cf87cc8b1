"""GPU parity of BILINEAR_BLEND (render_mode 3): the HIP path through the C ABI against the CPU oracle.

Bars as for the other mode: per-pixel counts and the blended part of every fragment list bit-exact, stored
transmittances, weights and blended features bit-exact (same operation order), gradients within 1e-4 relative.
"""
import numpy as np
import pytest
import torch

from tests.helpers import bilinear_backward_model, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu
MODE = dict(render_mode=abi.RENDER_BILINEAR_BLEND)


def _opaque(scene, factor=1.6):
    scene.confidence[:] = np.clip(scene.confidence * factor, 0, 0.98)  # so that the 0.001 cut triggers
    return scene


def _scenes():
    yield "tiny_K4", synthetic.tiny_scene(), {}
    yield "tiny_dense_K16", _opaque(synthetic.tiny_scene(num_points=6000, K=16, seed=71)), {}
    yield "tiny_dense_nocut_3ch", _opaque(synthetic.tiny_scene(num_points=5000, K=-1, channels=3, seed=72)), {}
    yield "tiny_long_lists", _opaque(synthetic.tiny_scene(num_points=40000, K=0, seed=73), 1.0), {}
    yield "tiny_2views_envmap", synthetic.tiny_scene(num_points=3000, K=8, num_views=2, seed=74), {"use_environment_map": 1}
    yield "tiny_radius_dropout", synthetic.tiny_scene(num_points=3000, K=8, seed=75), {"drop_out_points_by_radius": 1}
    yield "odd_size_5_layers", synthetic.tiny_scene(num_points=9000, w=83, h=61, num_layers=5, K=6, seed=76), {}
    yield "config1", synthetic.config1(), {}
    yield "config2_200k", synthetic.config2(num_points=200_000), {}


SCENES = list(_scenes())


def _blended_mask(off, kept):
    """True for the fragments of every list that took part in the blend (the first kept[q] of each)."""
    counts = np.diff(off)
    rank = np.arange(off[-1], dtype=np.int64) - np.repeat(off[:-1], counts)
    return rank < np.repeat(kept, counts)


def _check_forward(scene, overrides, rasterizer, oracle):
    params = make_params(scene, **{**overrides, **MODE})
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    saturated = 0
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64), err_msg="per-pixel counts differ")
        total = int(off[-1])
        kept = res.kept(b)
        np.testing.assert_array_equal(kept, ref.kept[b].astype(np.int64), err_msg="blended fragment counts differ")
        K = params.debug_max_list_length
        saturated += int((kept < (np.minimum(np.diff(off), K) if K > 0 else np.diff(off))).sum())
        m = _blended_mask(off, kept)
        np.testing.assert_array_equal(res.fragments(b)[m], ref.fragments[b, :total][m], err_msg="fragment lists differ")
        np.testing.assert_array_equal(res.transmittance(b)[m], ref.transmittance[b, :total][m])
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    return ref, dev, res, saturated


@pytest.mark.parametrize("name,scene,overrides", SCENES, ids=[s[0] for s in SCENES])
def test_forward_matches_oracle(name, scene, overrides, rasterizer, oracle):
    _, _, _, saturated = _check_forward(scene, overrides, rasterizer, oracle)
    if "nocut" in name or "long" in name:
        assert saturated > 50, "the scene must exercise the early exit"


def test_mode_3_needs_the_bigger_workspace(rasterizer):
    scene = synthetic.tiny_scene(num_points=500)
    dev = DeviceScene(scene)
    small = torch.empty(rasterizer.layout(scene).total_bytes, dtype=torch.uint8, device="cuda")
    with pytest.raises(abi.VetrastError) as e:
        rasterizer.forward(dev, make_params(scene, **MODE), workspace=small)
    assert e.value.status == abi.ERR_WORKSPACE_SMALL
    for mode in (0, 4):  # FUZZY_DT is not built; 4 does not exist
        with pytest.raises(abi.VetrastError) as e:
            rasterizer.forward(dev, make_params(scene, render_mode=mode))
        assert e.value.status == abi.ERR_UNSUPPORTED


GRAD_TOL = 1e-4


@pytest.mark.parametrize("name,scene,overrides", SCENES, ids=[s[0] for s in SCENES])
def test_backward_matches_oracle(name, scene, overrides, rasterizer, oracle):
    print(f"[case] bilinear backward {name} N={scene.num_points}", flush=True)
    ref, dev, res, _ = _check_forward(scene, dict(overrides, need_point_gradient=1), rasterizer, oracle)
    grad_out = scene.grad_out()
    if name == "tiny_long_lists":
        # lists of hundreds of fragments: the oracle's literal O(n^2) loop takes minutes, so the expectation comes from
        # the O(n) float64 suffix-sum model, which tests/test_oracle_bilinear.py pins against the oracle on short lists
        ref_g = bilinear_backward_model(oracle, ref, grad_out)
    else:
        ref_g = oracle.backward(ref, grad_out)
    got_g = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got_g["point_count"].cpu().numpy(), ref_g["point_count"])
    for key in ("texture", "confidence", "background", "points"):
        err = max_rel_err(got_g[key].cpu().numpy(), ref_g[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= GRAD_TOL, key


def test_backward_with_index_views_and_cameras(rasterizer, oracle):
    """Texture index indirection, two views, pose and intrinsics gradients (the pose count grows by 1 per fragment in
    this mode, the intrinsics count by 1/1024)."""
    scene = synthetic.tiny_scene(num_points=4000, K=8, seed=77, num_views=2)
    rng = np.random.default_rng(6)
    scene.index = rng.integers(0, 900, size=scene.num_points).astype(np.int32)
    ref, dev, res, _ = _check_forward(scene, {"need_point_gradient": 1}, rasterizer, oracle)
    grad_out = scene.grad_out()
    ref_g = oracle.backward(ref, grad_out, want_cameras=True)
    got_g = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_cameras=True)
    torch.cuda.synchronize()
    got = {k: v.cpu().numpy() for k, v in got_g.items() if k != "_args"}
    np.testing.assert_array_equal(got["point_count"], ref_g["point_count"])
    for key in ("texture", "confidence", "background", "points", "pose", "intrinsics"):
        assert max_rel_err(got[key], ref_g[key]) <= GRAD_TOL, key
    np.testing.assert_allclose(got["pose_count"], ref_g["pose_count"], rtol=1e-6)
    np.testing.assert_allclose(got["intrinsics_count"], ref_g["intrinsics_count"], rtol=1e-4)
    assert got["pose_count"][0] > 100


def test_backward_is_reproducible_and_linear(rasterizer):
    scene = synthetic.config2(num_points=100_000, w=480, h=270)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, make_params(scene, need_point_gradient=1, **MODE))
    go = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    a = {k: v.clone() for k, v in rasterizer.backward(res, go).items() if k != "_args"}
    b = {k: v.clone() for k, v in rasterizer.backward(res, go).items() if k != "_args"}
    c = {k: v.clone() for k, v in rasterizer.backward(res, [2.0 * g for g in go]).items() if k != "_args"}
    for k in a:
        assert torch.equal(a[k], b[k]), k
        if k != "point_count":
            assert torch.equal(c[k], 2.0 * a[k]), k


@pytest.mark.parametrize("shipped", [False, True], ids=["K16", "no_cut_radius_dropout"])
def test_config3_full_size(shipped, rasterizer, oracle):
    """BASELINE config 3 (2 M points, 1080p, 4 layers, K = 16) in BILINEAR_BLEND: 15 M fragments; and the same scene
    with the settings VET ships (configs/config.ini: no cut, points dropped by radius): 6.9 M fragments."""
    print(f"[case] bilinear config 3, 2M points, 1080p, forward+backward, shipped settings={shipped}", flush=True)
    scene = synthetic.config3(K=-1) if shipped else synthetic.config3()
    params = make_params(scene, need_point_gradient=1, drop_out_points_by_radius=1 if shipped else 0, **MODE)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    ref = oracle.forward(scene, params, num_threads=16)
    off = res.offsets(0)
    np.testing.assert_array_equal(off, ref.offsets[0].astype(np.int64))
    if not shipped:
        assert off[-1] > 3.9 * 3_800_000  # four fragments per visible (point, layer) but for the image border
    kept = res.kept(0)
    np.testing.assert_array_equal(kept, ref.kept[0].astype(np.int64))
    m = _blended_mask(off, kept)
    np.testing.assert_array_equal(res.fragments(0)[m], ref.fragments[0, :int(off[-1])][m])
    np.testing.assert_array_equal(res.weight(0), ref.weight[0])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    grad_out = scene.grad_out()
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    want = oracle.backward(ref, grad_out, num_threads=16)
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in ("texture", "confidence", "points"):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= GRAD_TOL, key
    # background: against the float64 sum over the pixels whose blend reached the background (T >= 0.001)
    bg64 = np.zeros(scene.num_channels)
    for l, (w, h) in enumerate(scene.layer_sizes()):
        T = ref.weight[0, ref.layer_base(l):ref.layer_base(l) + w * h].astype(np.float64).reshape(h, w)
        T = np.where(T >= 0.001, T, 0.0)
        bg64 += (grad_out[l][0].astype(np.float64) * T[None]).sum(axis=(1, 2))
    assert max_rel_err(got["background"].cpu().numpy(), bg64) <= 1e-4
