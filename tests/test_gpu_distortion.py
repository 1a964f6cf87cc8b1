"""GPU parity of the opt-in lens distortion (vetrast_params.allow_distortion) against the oracle.

Parity with the reference itself is unpinned for cameras with distortion (tests/test_oracle_distortion.py says why and
what pins the oracle instead); this file holds the HIP path to the oracle: lists and images bit-exact, gradients
(descriptors, confidence, points, poses, all thirteen intrinsics columns) within 1e-4.
"""
import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu


def _distorted_scene(**kw):
    scene = synthetic.tiny_scene(**kw)
    for c in range(scene.intrinsics.shape[0]):
        scene.intrinsics[c, 5:] = [0.15, -0.04, 0.006, 0.05, -0.012, 0.002, 0.004, -0.003]
    return scene


@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND, abi.RENDER_BILINEAR_BLEND])
def test_forward_and_backward_match_the_oracle(mode, rasterizer, oracle):
    scene = _distorted_scene(num_points=6000, K=8, seed=51, num_views=2)
    ang = 0.1
    scene.views[1].crop_transform = (1.1, 0.9, 1.5, -2.0, 0.05)
    scene.views[1].crop_rotation = (np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang))
    params = make_params(scene, need_point_gradient=1, render_mode=mode, allow_distortion=1, distortion_gradient_factor=0.25)
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    for b in range(2):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64))
        if mode != abi.RENDER_BILINEAR_BLEND:
            m = kept_mask(off, scene.max_list_length)
            np.testing.assert_array_equal(res.fragments(b)[m], ref.fragments[b, :int(off[-1])][m])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    # the distortion did move things: the same scene without it has other lists
    flat = synthetic.tiny_scene(num_points=6000, K=8, seed=51, num_views=2)
    flat.views = scene.views
    assert not np.array_equal(oracle.forward(flat, make_params(flat, render_mode=mode)).offsets, ref.offsets)

    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_cameras=True)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_cameras=True)
    torch.cuda.synchronize()
    got = {k: v.cpu().numpy() for k, v in got.items() if k != "_args"}
    np.testing.assert_array_equal(got["point_count"], want["point_count"])
    for key in ("texture", "confidence", "background", "points", "pose", "intrinsics"):
        assert max_rel_err(got[key], want[key]) <= 1e-4, key
    assert np.abs(want["intrinsics"][:, 5:]).min() > 0, "every distortion column carries a gradient"
    np.testing.assert_allclose(got["intrinsics_count"], want["intrinsics_count"], rtol=1e-4)


def test_without_the_switch_the_camera_is_refused(rasterizer):
    scene = _distorted_scene(num_points=500, seed=52)
    res = rasterizer.forward(DeviceScene(scene))
    assert rasterizer.check_device_flags(res) == abi.ERR_BAD_INPUT_DATA
    res = rasterizer.forward(DeviceScene(scene), make_params(scene, allow_distortion=1))
    assert rasterizer.check_device_flags(res) == abi.OK


def test_zero_coefficients_with_the_switch_on_are_the_plain_camera(rasterizer, oracle):
    """All coefficients zero, switch on: the same images and the same gradients bit for bit as with the switch off (the
    distortion Jacobian is exactly the identity there), except the eight distortion columns of the intrinsics gradient,
    which hold J_dis_dis^T (src/lib/rendering/PointRendererHelper.h:346-368) and are not zero: checked against the
    oracle, whose values tests/test_oracle_distortion.py pins against central differences."""
    scene = synthetic.tiny_scene(num_points=4000, K=8, seed=53)
    dev = DeviceScene(scene)
    go = scene.grad_out()
    grad_out = [torch.from_numpy(g).cuda() for g in go]
    plain = rasterizer.forward(dev, make_params(scene, need_point_gradient=1))
    plain_g = {k: v.clone() for k, v in rasterizer.backward(plain, grad_out, want_cameras=True).items() if k != "_args"}
    params = make_params(scene, need_point_gradient=1, allow_distortion=1)
    on = rasterizer.forward(dev, params)
    on_g = rasterizer.backward(on, grad_out, want_cameras=True)
    torch.cuda.synchronize()
    for a, b in zip(plain.out, on.out):
        assert torch.equal(a, b)
    for k, v in plain_g.items():
        if k == "intrinsics":
            assert torch.equal(on_g[k][:, :5], v[:, :5]), k
            assert not v[:, 5:].any()
        else:
            assert torch.equal(on_g[k], v), k
    want = oracle.backward(oracle.forward(scene, params), go, want_cameras=True)
    got = on_g["intrinsics"].cpu().numpy()
    assert np.abs(got[0, 5:]).min() > 0
    assert max_rel_err(got[:, 5:], want["intrinsics"][:, 5:]) <= 1e-4


def test_through_the_shim(oracle):
    from vet_amd import torch_ops

    scene = _distorted_scene(num_points=3000, K=8, seed=54)
    params = make_params(scene, need_point_gradient=1, allow_distortion=1, distortion_gradient_factor=0.005)
    ref = oracle.forward(scene, params)
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_cameras=True)
    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    views = [(v.w, v.h, v.image_index, v.camera_index, v.camera_model_type, *v.crop_transform, *v.crop_rotation) for v in scene.views]
    args = lambda intr: (cu(scene.texture), cu(scene.background), cu(scene.position, True),
                         torch.zeros((1, 6), dtype=torch.float64, device="cuda"), intr, cu(scene.confidence.reshape(1, -1)),
                         cu(scene.poses_se3), None, views, scene.num_layers)
    common = dict(train=False, use_environment_map=0, need_point_gradient=1, drop_out_points_by_radius=0,
                  debug_max_list_length=scene.max_list_length, camera_gradient_normalization=0,
                  point_gradient_normalization=0, quirk_background_confidence_leak=0)
    with pytest.raises(RuntimeError, match="distortion"):
        torch_ops.blend_point_cloud(*args(cu(scene.intrinsics)), **common)
    intrinsics = cu(scene.intrinsics, True)
    outs = torch_ops.blend_point_cloud(*args(intrinsics), allow_distortion=1, **common)
    for l, o in enumerate(outs):
        np.testing.assert_array_equal(o.detach().cpu().numpy(), ref.out[l])
    torch.autograd.backward(outs, [torch.from_numpy(g).cuda() for g in grad_out])
    assert max_rel_err(intrinsics.grad.cpu().numpy(), want["intrinsics"]) <= 1e-4
    assert np.abs(intrinsics.grad.cpu().numpy()[:, 5:]).min() > 0
