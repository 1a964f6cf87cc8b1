"""Calls with several views that each see a part of an ordered cloud, as a training batch of crops does: lists, images
and gradients against the oracle, with crops inside the image, a rotated and scaled crop across the image border, an
empty crop, a camera with the whole cloud behind it and one that stands inside the cloud; and every view rendered alone
against the same view in the batch, in both orders of the batch.
"""
import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params
from vet_amd.synthetic import ViewSpec

pytestmark = pytest.mark.gpu


def _quat_y(angle):
    return [0.0, np.sin(angle / 2), 0.0, np.cos(angle / 2)]


def _scene(K):
    scene = synthetic.config2(num_points=150_000, w=480, h=270, K=K)
    ang = 0.4
    rot = (np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang))
    # poses (rotation, then the translation added in view space): 0 the scene's own; 1 the whole cloud behind the
    # camera plane; 2 inside the cloud, turned by 70 degrees (boxes on both sides of the camera plane); 3 shifted sideways
    poses = np.repeat(scene.poses_se3[:1], 4, axis=0).copy()
    poses[1, 4:7] = [0.0, 0.0, -20.0]
    poses[2, :4] = _quat_y(np.deg2rad(70.0))
    poses[2, 4:7] = [0.3, -0.2, 0.5]
    poses[3, 4:7] = poses[0, 4:7] + [1.5, 0.5, 0.0]
    scene.poses_se3 = poses
    scene.views = [
        ViewSpec(128, 96, image_index=0, crop_transform=(1.0, 1.0, -170.0, -90.0, 0.0)),
        ViewSpec(128, 96, image_index=0, crop_transform=(1.0, 1.0, -20.0, -150.0, 0.0)),
        ViewSpec(128, 96, image_index=0, crop_transform=(1.3, 0.8, -300.0, -60.0, 0.02), crop_rotation=rot),
        ViewSpec(128, 96, image_index=0, crop_transform=(1.0, 1.0, -5000.0, -90.0, 0.0)),   # sees nothing
        ViewSpec(128, 96, image_index=1, crop_transform=(1.0, 1.0, -170.0, -90.0, 0.0)),    # the cloud behind it
        ViewSpec(128, 96, image_index=2, crop_transform=(0.5, 0.5, -60.0, -20.0, 0.0)),     # inside the cloud
        ViewSpec(128, 96, image_index=3, crop_transform=(1.0, 1.0, -100.0, -100.0, 0.0), crop_rotation=rot),
    ]
    return scene


@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND, abi.RENDER_BILINEAR_BLEND],
                         ids=["full", "fuzzy", "bilinear"])
@pytest.mark.parametrize("dropout_by_radius", [0, 1])
def test_later_views_match_oracle(mode, dropout_by_radius, rasterizer, oracle):
    print(f"[case] batch of partial views mode={mode} radius drop-out={dropout_by_radius}", flush=True)
    scene = _scene(K=8)
    rng = np.random.default_rng(3)
    scene.dropout = (rng.random((len(scene.views), scene.num_points)) < 0.2).astype(np.float32)
    if dropout_by_radius:
        scene.position[:, 3] = (scene.position[:, 3] * rng.uniform(0.2, 3.0, scene.num_points)).astype(np.float32)
    params = make_params(scene, render_mode=mode, need_point_gradient=1, depth_accept_blend=0.05,
                         drop_out_points_by_radius=dropout_by_radius, drop_out_radius_threshold=0.6)
    ref = oracle.forward(scene, params, num_threads=8)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    seen = []
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64), err_msg=f"view {b}")
        total = int(off[-1])
        seen.append(total)
        keep = kept_mask(off, params.debug_max_list_length)
        np.testing.assert_array_equal(res.fragments(b)[keep], ref.fragments[b, :total][keep], err_msg=f"view {b}")
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    print("  fragments per view", seen, flush=True)
    assert seen[3] == 0 and seen[4] == 0 and min(seen[0], seen[1], seen[2], seen[5], seen[6]) > 0
    assert max(seen) < 0.5 * scene.num_points * scene.num_layers * (4 if mode == abi.RENDER_BILINEAR_BLEND else 1)
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_cameras=True, num_threads=8)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_cameras=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    # The oracle adds the intrinsics terms of ~10^5 fragments up in float32, as the reference does; that sum alone moves
    # by up to 4e-4 with the order of the additions (its own results for 1, 3 and 8 threads), the library's is in
    # float64.
    for key, tol in (("texture", 1e-4), ("confidence", 1e-4), ("background", 1e-4), ("points", 1e-4), ("pose", 1e-4),
                     ("intrinsics", 1e-3)):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= tol, key


@pytest.mark.parametrize("mode", [abi.RENDER_FULL_BLEND, abi.RENDER_BILINEAR_BLEND], ids=["full", "bilinear"])
def test_view_order_and_single_view_calls_agree(mode, rasterizer):
    """Every view rendered in a call of its own gives the lists and images it gives as a later view of the batch, and as
    an earlier view of the batch in reverse order."""
    scene = _scene(K=-1)
    views = list(scene.views)
    params = make_params(scene, render_mode=mode)
    batch = rasterizer.forward(DeviceScene(scene), params)
    scene.views = views[::-1]
    reverse = rasterizer.forward(DeviceScene(scene), params)
    torch.cuda.synchronize()
    B = len(views)
    for b, view in enumerate(views):
        scene.views = [view]
        one = rasterizer.forward(DeviceScene(scene), make_params(scene, render_mode=mode))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(one.offsets(0), batch.offsets(b))
        np.testing.assert_array_equal(one.offsets(0), reverse.offsets(B - 1 - b))
        np.testing.assert_array_equal(one.fragments(0), batch.fragments(b))
        np.testing.assert_array_equal(one.fragments(0), reverse.fragments(B - 1 - b))
        for l in range(scene.num_layers):
            assert torch.equal(one.out[l][0], batch.out[l][b])
            assert torch.equal(one.out[l][0], reverse.out[l][B - 1 - b])
