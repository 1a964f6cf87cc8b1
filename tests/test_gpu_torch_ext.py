"""The libtorch shim (PointRender autograd Function with the reference's argument order) against the oracle.

This is the check the reference's authors sketched in their disabled A/B harness (src/lib/models/Pipeline.cpp:167-219):
render, reduce the outputs to a scalar, call backward, compare the gradients of the scene tensors.
"""
import numpy as np
import pytest
import torch

from tests.helpers import max_rel_err
from vet_amd import synthetic
from vet_amd.rasterizer import make_params

pytestmark = pytest.mark.gpu


def _views(scene):
    return [(v.w, v.h, v.image_index, v.camera_index, v.camera_model_type, *v.crop_transform, *v.crop_rotation)
            for v in scene.views]


@pytest.mark.parametrize("render_mode", [1, 2, 3], ids=["full_blend", "fuzzy_blend", "bilinear_blend"])
@pytest.mark.parametrize("literal", [True, False], ids=["reference_literal", "clean"])
def test_autograd_matches_oracle(literal, render_mode, oracle):
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=5000, K=8, seed=31, num_views=2)
    quirks = dict(quirk_background_confidence_leak=1 if literal else 0,
                  point_gradient_normalization=2 if literal else 0,
                  camera_gradient_normalization=1 if literal else 0, render_mode=render_mode)
    params = make_params(scene, need_point_gradient=1, **quirks)
    ref = oracle.forward(scene, params)
    grad_out = scene.grad_out()
    ref_g = oracle.backward(ref, grad_out, want_cameras=True)

    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    texture, background = cu(scene.texture, True), cu(scene.background, True)
    points, confidence = cu(scene.position, True), cu(scene.confidence.reshape(1, -1), True)
    tangents = torch.zeros((scene.poses_se3.shape[0], 6), dtype=torch.float64, device="cuda", requires_grad=True)
    intrinsics = cu(scene.intrinsics, True)
    outs = torch_ops.blend_point_cloud(texture, background, points, tangents, intrinsics, confidence,
                                       cu(scene.poses_se3), None, _views(scene), scene.num_layers, train=False,
                                       use_environment_map=0, need_point_gradient=1, drop_out_points_by_radius=0,
                                       debug_max_list_length=scene.max_list_length, **quirks)
    assert len(outs) == scene.num_layers
    loss = 0
    for l, o in enumerate(outs):
        assert tuple(o.shape) == ref.out[l].shape
        np.testing.assert_array_equal(o.detach().cpu().numpy(), ref.out[l])
        loss = loss + (o * torch.from_numpy(grad_out[l]).cuda()).sum()
    loss.backward()
    assert max_rel_err(texture.grad.cpu().numpy(), ref_g["texture"]) <= 1e-4
    assert max_rel_err(confidence.grad.cpu().numpy().reshape(-1), ref_g["confidence"]) <= 1e-4
    assert max_rel_err(background.grad.cpu().numpy(), ref_g["background"]) <= 1e-4
    assert max_rel_err(points.grad.cpu().numpy(), ref_g["points"]) <= 1e-4
    # pose tangents [F,6] float64 and intrinsics [Ncam,13]: fx, fy, cx, cy columns (skew and distortion stay zero)
    assert tangents.grad.dtype == torch.float64
    assert max_rel_err(tangents.grad.cpu().numpy(), ref_g["pose"]) <= 1e-4
    assert max_rel_err(intrinsics.grad.cpu().numpy(), ref_g["intrinsics"]) <= 1e-4
    assert np.all(intrinsics.grad.cpu().numpy()[:, 4:] == 0)


def test_no_grad_call_and_masks(oracle):
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=3000, K=8, seed=32)
    params = make_params(scene, output_background_mask=1, output_background_mask_value=0.25)
    ref = oracle.forward(scene, params)
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    with torch.no_grad():
        outs = torch_ops.blend_point_cloud(cu(scene.texture), cu(scene.background), cu(scene.position),
                                           torch.zeros((1, 6), dtype=torch.float64, device="cuda"),
                                           cu(scene.intrinsics), cu(scene.confidence.reshape(1, -1)),
                                           cu(scene.poses_se3), None, _views(scene), scene.num_layers,
                                           use_environment_map=0, drop_out_points_by_radius=0,
                                           debug_max_list_length=scene.max_list_length, output_background_mask=1,
                                           output_background_mask_value=0.25)
    L = scene.num_layers
    assert len(outs) == 2 * L
    for l in range(L):
        np.testing.assert_array_equal(outs[l].cpu().numpy(), ref.out[l])
        np.testing.assert_array_equal(outs[L + l].cpu().numpy(), ref.out_mask[l])


def test_training_step_on_raw_tensors_with_fused_steps(oracle):
    """What one VET iteration does around the rasterizer, on the raw tensors: sigmoid on confidence_raw and abs on
    texture_raw fused into the render call, autograd back to the raw tensors, then MyAdam.step + zero_grad. Compared
    with the unfused formulation in torch (sigmoid/abs as tensor ops, torch.optim.Adam)."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=4000, K=8, seed=33)
    rng = np.random.default_rng(2)
    conf_raw = (0.2 * rng.standard_normal(scene.num_points)).astype(np.float32).reshape(1, -1)
    tex_raw = rng.standard_normal(scene.texture.shape).astype(np.float32)
    bg_raw = np.array([0.2, -0.5, 0.7, -0.3], np.float32)
    grad_out = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    common = dict(use_environment_map=0, need_point_gradient=0, drop_out_points_by_radius=0,
                  debug_max_list_length=scene.max_list_length, quirk_background_confidence_leak=0,
                  point_gradient_normalization=0)

    def render(texture, background, confidence, **extra):
        points = cu(scene.position)
        tangents = torch.zeros((scene.poses_se3.shape[0], 6), dtype=torch.float64, device="cuda")
        outs = torch_ops.blend_point_cloud(texture, background, points, tangents, cu(scene.intrinsics), confidence,
                                           cu(scene.poses_se3), None, _views(scene), scene.num_layers, train=False,
                                           **common, **extra)
        return sum((o * g).sum() for o, g in zip(outs, grad_out))

    # fused: raw tensors in, raw gradients out, fused Adam
    f = [cu(tex_raw, True), cu(bg_raw, True), cu(conf_raw, True)]
    opt_f = torch_ops.MyAdam([([f[0]], 0.01), ([f[1]], 0.004), ([f[2]], 0.002)])
    # unfused: the same with tensor ops
    u = [cu(tex_raw, True), cu(bg_raw, True), cu(conf_raw, True)]
    opt_u = torch.optim.Adam([{"params": [u[0]], "lr": 0.01}, {"params": [u[1]], "lr": 0.004},
                              {"params": [u[2]], "lr": 0.002}])
    for it in range(3):
        loss_f = render(f[0], f[1], f[2], fused_confidence_scale=10.0, fused_texture_abs=1)
        loss_f.backward()
        loss_u = render(torch.abs(u[0]), torch.abs(u[1]), torch.sigmoid(10.0 * u[2]))
        loss_u.backward()
        assert abs(loss_f.item() - loss_u.item()) <= 1e-4 * max(1.0, abs(loss_u.item()))
        for a, b in zip(f, u):
            assert max_rel_err(a.grad.cpu().numpy(), b.grad.cpu().numpy()) <= 1e-4
        opt_f.step(zero_grad=True)
        opt_u.step()
        opt_u.zero_grad()
        for a, b in zip(f, u):
            assert not a.grad.any()
            assert max_rel_err(a.detach().cpu().numpy(), b.detach().cpu().numpy()) <= 1e-4, it


def test_fill_scene_grid_with_loss_through_the_shim(oracle):
    """The reference's calling sequence (src/lib/apps/train.cpp:1069-1078 with NeuralPointCloudCuda.h:42-52): reset the
    cell values, lift |target - output| of every view of the batch, normalise by the access count."""
    from vet_amd import torch_ops

    print("[case] torch_ext fill_scene_grid_with_loss", flush=True)
    scene = synthetic.tiny_scene(num_points=500, w=160, h=120, num_views=2, seed=31)
    mn, ln = synthetic.cell_grid(scene.position[:, :3], 0.3)
    n = len(mn)
    loss = [np.abs(synthetic.error_image(40 + b, 3, 120, 160)) for b in range(2)]
    want_v, want_c = np.zeros(n, np.float32), np.zeros(n, np.int32)
    for b in range(2):
        oracle.lift_error(mn, ln, want_v, want_c, scene.views[b], scene.poses_se3, scene.intrinsics, loss[b])
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    value = torch.zeros((n, 1), dtype=torch.float32, device="cuda")       # ResetCellValues
    count = torch.zeros((n, 1), dtype=torch.int32, device="cuda")
    d_mn, d_ln, d_pose, d_intr = dev(mn), dev(ln), dev(scene.poses_se3), dev(scene.intrinsics)
    for b in range(2):
        torch_ops.fill_scene_grid_with_loss(b, d_mn, d_ln, value, count, _views(scene), d_pose, d_intr, dev(loss[b]))
    torch.cuda.synchronize()
    assert want_c.sum() > 1000
    np.testing.assert_array_equal(count.cpu().numpy().ravel(), want_c)
    np.testing.assert_allclose(value.cpu().numpy().ravel(), want_v, rtol=1e-6)
    normalised = value / torch.where(count != 0, count, torch.ones_like(count))   # NormalizeBBCellValue
    np.testing.assert_allclose(normalised.cpu().numpy().ravel(), want_v / np.maximum(want_c, 1), rtol=1e-6)


def test_render_module_glue_super_sampling_and_mask_channel(oracle):
    """PointRenderModuleImpl::forward (src/lib/rendering/RenderModule.cpp:45-245) around the rasterizer: with
    super_sampling the views are rendered at twice the size (crop transform scaled by 2) and 2x2 blocks averaged; the
    masks come back detached and, with cat_masks_to_color, as an extra image channel. Checked against the oracle
    rendering the doubled views, pooled by hand, and against autograd through the pooling."""
    from vet_amd import torch_ops
    from vet_amd.synthetic import ViewSpec

    scene = synthetic.tiny_scene(num_points=3000, K=8, seed=33, w=32, h=24, num_layers=3)
    big = synthetic.tiny_scene(num_points=3000, K=8, seed=33, w=32, h=24, num_layers=3)
    big.views = [ViewSpec(64, 48, crop_transform=(2.0, 2.0, 0.0, 0.0, 0.0))]
    params = make_params(big, output_background_mask=1, output_background_mask_value=0.25, need_point_gradient=0)
    ref = oracle.forward(big, params)
    pool = lambda a: a.reshape(a.shape[0], a.shape[1], a.shape[2] // 2, 2, a.shape[3] // 2, 2).mean(axis=(3, 5))

    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    texture, confidence = cu(scene.texture, True), cu(scene.confidence.reshape(1, -1), True)
    views = _views(scene)
    outs = torch_ops.blend_point_cloud(texture, cu(scene.background), cu(scene.position),
                                       torch.zeros((1, 6), dtype=torch.float64, device="cuda"), cu(scene.intrinsics),
                                       confidence, cu(scene.poses_se3), None, views, scene.num_layers, train=True,
                                       use_environment_map=0, drop_out_points_by_radius=0, need_point_gradient=0,
                                       debug_max_list_length=scene.max_list_length, output_background_mask=1,
                                       output_background_mask_value=0.25, quirk_background_confidence_leak=0,
                                       super_sampling=1, cat_masks_to_color=1)
    L = scene.num_layers
    assert len(outs) == 2 * L
    for l, (w, h) in enumerate(scene.layer_sizes()):
        img, mask = outs[l], outs[L + l]
        assert tuple(img.shape) == (1, scene.num_channels + 1, h, w) and tuple(mask.shape) == (1, 1, h, w)
        assert not mask.requires_grad
        np.testing.assert_allclose(img[:, :-1].detach().cpu().numpy(), pool(ref.out[l]), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(mask.cpu().numpy(), pool(ref.out_mask[l]), rtol=1e-6)
        np.testing.assert_array_equal(img[:, -1:].detach().cpu().numpy(), mask.cpu().numpy())
    # gradients flow through the pooling into the rasterizer: upstream gradient g on the pooled image is g / 4 on
    # each of the four pixels it averages
    grad_small = [np.random.default_rng(5 + l).normal(size=(1, scene.num_channels, h, w)).astype(np.float32)
                  for l, (w, h) in enumerate(scene.layer_sizes())]
    loss = sum((outs[l][:, :-1] * cu(grad_small[l])).sum() for l in range(L))
    loss.backward()
    grad_big = [np.repeat(np.repeat(g, 2, axis=2), 2, axis=3) * np.float32(0.25) for g in grad_small]
    want = oracle.backward(ref, grad_big, want_points=False)
    assert max_rel_err(texture.grad.cpu().numpy(), want["texture"]) <= 1e-4
    assert max_rel_err(confidence.grad.cpu().numpy().ravel(), want["confidence"]) <= 1e-4
    assert views == _views(scene), "the views are restored after the call"


@pytest.mark.parametrize("cat_env_to_color", [0, 1])
def test_render_module_environment_map_branch(cat_env_to_color, oracle):
    """The environment-map branch of PointRenderModuleImpl::forward (src/lib/rendering/RenderModule.cpp:129-202) with the
    map behind a callback: the callback sees, per layer and view, the transmittance left behind the points (the oracle's
    per-pixel weight, bit for bit); what it returns is appended as channels, or added where that weight is at most
    0.001 (the reference's no_envmap_at_points masking, literally). Gradients reach the map's own parameter and, through
    the rasterizer, the descriptors."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=4000, K=-1, seed=35, w=40, h=24, num_layers=3, num_views=2)
    scene.confidence[::3] = 1.0  # opaque points: pixels whose weight falls to exactly 0
    params = make_params(scene, output_background_mask=1, use_environment_map=1, need_point_gradient=0)
    ref = oracle.forward(scene, params)
    sizes = scene.layer_sizes()
    B, L, Cn = len(scene.views), scene.num_layers, scene.num_channels

    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    texture, confidence = cu(scene.texture, True), cu(scene.confidence.reshape(1, -1), True)
    sky = torch.tensor([0.3, -0.2, 0.7, 1.1], device="cuda")[:Cn].clone().requires_grad_(True)
    seen = {}

    def environment(layers):
        assert len(layers) == L and all(len(per_view) == B for per_view in layers)
        seen["layers"] = [[t.clone() for t in per_view] for per_view in layers]
        # a "map" that is one colour, weighted by what the points let through plus a constant
        return [torch.cat(per_view, 0) * sky.view(1, -1, 1, 1) + 0.5 * sky.view(1, -1, 1, 1) for per_view in layers]

    outs = torch_ops.blend_point_cloud(texture, cu(scene.background), cu(scene.position),
                                       torch.zeros((B, 6), dtype=torch.float64, device="cuda"), cu(scene.intrinsics),
                                       confidence, cu(scene.poses_se3), None, _views(scene), L, train=True,
                                       environment=environment, use_environment_map=1, drop_out_points_by_radius=0,
                                       need_point_gradient=0, debug_max_list_length=scene.max_list_length,
                                       output_background_mask=1, quirk_background_confidence_leak=0,
                                       cat_env_to_color=cat_env_to_color)
    assert len(outs) == 2 * L
    first = 0
    some_opaque = False
    for l, (w, h) in enumerate(sizes):
        weight = np.stack([ref.weight[b][first:first + w * h].reshape(1, h, w) for b in range(B)])
        first += w * h
        for b in range(B):
            np.testing.assert_array_equal(seen["layers"][l][b].cpu().numpy(), weight[b:b + 1])
        env = weight * sky.detach().cpu().numpy().reshape(1, -1, 1, 1) + 0.5 * sky.detach().cpu().numpy().reshape(1, -1, 1, 1)
        got = outs[l].detach().cpu().numpy()
        if cat_env_to_color:
            assert got.shape == (B, 2 * Cn, h, w)
            np.testing.assert_array_equal(got[:, :Cn], ref.out[l])
            np.testing.assert_allclose(got[:, Cn:], env, rtol=1e-6, atol=1e-7)
        else:
            masking = np.where(weight > 0.001, 0.0, 1.0).astype(np.float32)
            some_opaque |= bool(masking.any()) and not bool(masking.all())
            np.testing.assert_allclose(got, ref.out[l] + masking * env, rtol=1e-6, atol=1e-7)
    assert cat_env_to_color or some_opaque, "the scene must have pixels on both sides of the masking threshold"
    sum(o.sum() for o in outs[:L]).backward()
    assert sky.grad is not None and float(sky.grad.abs().sum()) > 0
    want = oracle.backward(ref, [np.ones_like(o) for o in ref.out], want_points=False)
    assert max_rel_err(texture.grad.cpu().numpy(), want["texture"]) <= 1e-4
    assert max_rel_err(confidence.grad.cpu().numpy().ravel(), want["confidence"]) <= 1e-4


def _plain_call(scene, torch_ops, texture=None, confidence=None, intrinsics=None, train=False, **extra):
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    B = scene.poses_se3.shape[0]
    return torch_ops.blend_point_cloud(cu(scene.texture) if texture is None else texture, cu(scene.background),
                                       cu(scene.position), torch.zeros((B, 6), dtype=torch.float64, device="cuda"),
                                       cu(scene.intrinsics) if intrinsics is None else intrinsics,
                                       cu(scene.confidence.reshape(1, -1)) if confidence is None else confidence,
                                       cu(scene.poses_se3), None, _views(scene), scene.num_layers, train=train,
                                       use_environment_map=0, drop_out_points_by_radius=0, need_point_gradient=0,
                                       debug_max_list_length=scene.max_list_length, quirk_background_confidence_leak=0,
                                       **extra)


def test_cameras_with_distortion_are_refused_by_the_shim():
    """Non-zero distortion coefficients (columns 5..12 of the intrinsics) must not render as an undistorted pinhole
    through the drop-in seam: BlendPointCloud and FillSceneGridWithLoss throw. A tensor the cache has not seen is read
    back (blocking) and refused before anything renders. A tensor it knows is never read back again: when it changes in
    place, the call that follows renders, the status word that call raised on the device travels to the host behind it,
    and the next call throws."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=1000, K=8, seed=36)
    fresh = torch.from_numpy(scene.intrinsics.copy()).cuda()
    fresh[0, 7] = 1e-3
    with pytest.raises(RuntimeError, match="distortion"):
        _plain_call(scene, torch_ops, intrinsics=fresh)  # unknown tensor: refused at once

    intr = torch.from_numpy(scene.intrinsics.copy()).cuda()
    outs = _plain_call(scene, torch_ops, intrinsics=intr)  # zero coefficients: fine
    assert len(outs) == scene.num_layers
    intr[0, 7] = 1e-3  # k3, changed in place: same storage, new version
    assert len(_plain_call(scene, torch_ops, intrinsics=intr)) == scene.num_layers  # not read back: renders, flagged
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="distortion"):
        _plain_call(scene, torch_ops, intrinsics=intr)
    mn, ln = synthetic.cell_grid(scene.position[:, :3], 0.5)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    value = torch.zeros((len(mn), 1), device="cuda")
    count = torch.zeros((len(mn), 1), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="distortion"):  # after a refusal the tensor itself is checked again
        torch_ops.fill_scene_grid_with_loss(0, dev(mn), dev(ln), value, count, _views(scene), dev(scene.poses_se3), intr,
                                            torch.zeros((3, scene.views[0].h, scene.views[0].w), device="cuda"))
    assert int(count.sum()) == 0
    intr[0, 7] = 0.0
    assert len(_plain_call(scene, torch_ops, intrinsics=intr)) == scene.num_layers

    # a write that leaves the tensor's version counter alone (as one through a raw pointer does) is found by the
    # look at the status word that every 64th call asks for
    with torch.autograd._unsafe_preserve_version_counter(intr):
        intr[0, 5] = 2e-3
    with pytest.raises(RuntimeError, match="distortion"):
        for _ in range(70):
            _plain_call(scene, torch_ops, intrinsics=intr)
            torch.cuda.synchronize()
    intr[0, 5] = 0.0
    assert len(_plain_call(scene, torch_ops, intrinsics=intr)) == scene.num_layers


def test_add_depth_to_network_appends_a_zero_channel(oracle):
    """The blend modes never write the depth tensors (src/lib/rendering/PointRenderer.cu:1061-1066 hands out the zero-filled
    buffers); PointRenderModuleImpl::forward appends them to the images as a channel (RenderModule.cpp:223-232), behind
    the masks' channel position: images [B,C+1,h,w] with a zero last channel, masks unchanged, gradients as without."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=3000, K=8, seed=37, num_views=2)
    params = make_params(scene, output_background_mask=1, output_background_mask_value=0.5, need_point_gradient=0)
    ref = oracle.forward(scene, params)
    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    texture, confidence = cu(scene.texture, True), cu(scene.confidence.reshape(1, -1), True)
    outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence, train=True, add_depth_to_network=1,
                       output_background_mask=1, output_background_mask_value=0.5)
    L, Cn = scene.num_layers, scene.num_channels
    assert len(outs) == 2 * L
    for l in range(L):
        img = outs[l].detach().cpu().numpy()
        assert img.shape[1] == Cn + 1
        np.testing.assert_array_equal(img[:, :Cn], ref.out[l])
        assert not img[:, Cn:].any()
        np.testing.assert_array_equal(outs[L + l].cpu().numpy(), ref.out_mask[l])
    grad_out = scene.grad_out()
    sum((outs[l][:, :Cn] * cu(grad_out[l])).sum() + outs[l][:, Cn:].sum() for l in range(L)).backward()
    want = oracle.backward(ref, grad_out, want_points=False)
    assert max_rel_err(texture.grad.cpu().numpy(), want["texture"]) <= 1e-4
    assert max_rel_err(confidence.grad.cpu().numpy().ravel(), want["confidence"]) <= 1e-4


def test_training_steps_share_one_workspace():
    """The workspace a training forward saves for its backward pass is taken again by the next step once the graph of
    the step before is gone; while a graph is alive its workspace is left alone."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=2000, K=8, seed=38)
    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    texture = cu(scene.texture, True)
    seen = []
    for it in range(3):
        outs = _plain_call(scene, torch_ops, texture=texture, train=True)
        seen.append(torch_ops.train_workspace_info())
        sum(o.sum() for o in outs).backward()
        del outs
    assert seen[0][0] != 0 and seen[0] == seen[1] == seen[2]
    first_grad = texture.grad.clone()
    # two graphs alive at once: the second call must not write into the first one's workspace
    a = _plain_call(scene, torch_ops, texture=texture, train=True)
    ptr_a = torch_ops.train_workspace_info()[0]
    b = _plain_call(scene, torch_ops, texture=texture, train=True)
    ptr_b = torch_ops.train_workspace_info()[0]
    assert ptr_a != ptr_b
    texture.grad = None
    sum(o.sum() for o in a).backward()
    np.testing.assert_array_equal(texture.grad.cpu().numpy() * 3, first_grad.cpu().numpy())  # same gradient each step
    texture.grad = None
    sum(o.sum() for o in b).backward()
    np.testing.assert_array_equal(texture.grad.cpu().numpy() * 3, first_grad.cpu().numpy())


def test_the_cache_keeps_a_processing_order_and_results_do_not_depend_on_it():
    """The shim builds a Morton order on the device for the binning pass, rebuilds it when the number of points changes
    and after `refresh` forward calls, and can be told not to; outputs and gradients are the same bits either way."""
    from vet_amd import torch_ops

    scene = synthetic.config2(num_points=30_000, w=320, h=180, point_order="grown")
    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    grads = [torch.from_numpy(g).cuda() for g in scene.grad_out()]

    def run():
        texture, confidence = cu(scene.texture, True), cu(scene.confidence.reshape(1, -1), True)
        points = cu(scene.position, True)
        B = scene.poses_se3.shape[0]
        outs = torch_ops.blend_point_cloud(texture, cu(scene.background), points,
                                           torch.zeros((B, 6), dtype=torch.float64, device="cuda"), cu(scene.intrinsics),
                                           confidence, cu(scene.poses_se3), None, _views(scene), scene.num_layers,
                                           train=True, use_environment_map=0, need_point_gradient=1,
                                           drop_out_points_by_radius=0, debug_max_list_length=scene.max_list_length)
        torch.autograd.backward(outs, grads)
        return [o.detach().clone() for o in outs], [texture.grad, confidence.grad, points.grad]

    try:
        torch_ops.set_point_order_refresh(0)
        plain_out, plain_grad = run()
        assert torch_ops.point_order() is None
        torch_ops.set_point_order_refresh(3)
        out1, grad1 = run()
        first = torch_ops.point_order()
        assert first is not None and first.dtype == torch.int32 and first.numel() == scene.num_points
        assert torch.equal(torch.sort(first.long()).values, torch.arange(scene.num_points, device="cuda"))
        ptr = first.data_ptr()
        run()
        run()
        assert torch_ops.point_order().data_ptr() == ptr, "kept for `refresh` calls"
        run()
        assert torch.equal(torch_ops.point_order(), first), "rebuilt from the same positions: the same order"
        for a, b in zip(plain_out + plain_grad, out1 + grad1):
            assert torch.equal(a, b)
        # fewer points: a new order of the new length
        scene.position, scene.texture, scene.confidence = scene.position[:20_000], scene.texture[:, :20_000].copy(), \
            scene.confidence[:20_000]
        run()
        assert torch_ops.point_order().numel() == 20_000
    finally:
        torch_ops.set_point_order_refresh(1000)


def test_a_cloud_in_preprocessed_order_goes_without_the_order_array():
    """The cache compares how far apart the 64 points of a wave lie in array order and in the order it has built; a
    cloud that comes in the order of VET's preprocessing (src/lib/data/SceneData.cpp:105-106) is as good as it is, so
    its calls are not handed the array; one in the generator's raw order is."""
    from vet_amd import torch_ops

    try:
        torch_ops.set_point_order_refresh(1000)
        for order, used in (("vet_preprocess", False), ("generated", True), ("grown", True), ("vet_preprocess", False)):
            # (2 000 points on each of the generator's 200 surfaces: a run of 64 of them spans its whole surface)
            scene = synthetic.config2(num_points=400_000, w=320, h=180, point_order=order)
            assert len(_plain_call(scene, torch_ops)) == scene.num_layers
            assert torch_ops.point_order() is not None and torch_ops.point_order_in_use() == used, order
            scene = synthetic.config2(num_points=409_600, w=320, h=180, point_order=order)  # another size: rebuilt
            _plain_call(scene, torch_ops)
            assert torch_ops.point_order_in_use() == used, order
    finally:
        torch_ops.set_point_order_refresh(1000)


def test_the_cache_sizes_bins_from_the_fragment_counts_of_earlier_calls():
    """Crops that see a part of the cloud: the shim reads the per-layer fragment counts of a call back without blocking
    and sizes the bins of later calls with them; images and gradients are the same bits with and without."""
    from vet_amd import torch_ops

    scene = synthetic.config2(num_points=60_000, w=480, h=270, K=8)
    scene.views = [synthetic.ViewSpec(128, 96, crop_transform=(1.0, 1.0, -170.0, -90.0, 0.0))]
    cu = lambda a, rg=False: torch.from_numpy(np.ascontiguousarray(a)).cuda().requires_grad_(rg)
    grads = [torch.from_numpy(g).cuda() for g in scene.grad_out()]

    def run(history):
        texture, confidence = cu(scene.texture, True), cu(scene.confidence.reshape(1, -1), True)
        outs = torch_ops.blend_point_cloud(texture, cu(scene.background), cu(scene.position),
                                           torch.zeros((1, 6), dtype=torch.float64, device="cuda"), cu(scene.intrinsics),
                                           confidence, cu(scene.poses_se3), None, _views(scene), scene.num_layers,
                                           train=True, use_environment_map=0, need_point_gradient=0,
                                           drop_out_points_by_radius=0, debug_max_list_length=scene.max_list_length,
                                           size_bins_from_history=1 if history else 0)
        torch.autograd.backward(outs, grads)
        torch.cuda.synchronize()
        return [o.detach().clone() for o in outs] + [texture.grad, confidence.grad]

    plain = run(False)
    first = run(True)   # nothing known yet: schedules the read-back
    second = run(True)  # the copy has landed (run() synchronises): bins sized from it
    hist = torch_ops.fragment_history()
    assert len(hist) == scene.num_layers and 0 < sum(hist) < 0.5 * scene.num_points * scene.num_layers
    for a, b, c in zip(plain, first, second):
        assert torch.equal(a, b) and torch.equal(a, c)


@pytest.mark.parametrize("render_mode", [1, 3], ids=["full_blend", "bilinear_blend"])
def test_adapter_templates_render_like_the_binding(render_mode):
    """vet_adapter.h, instantiated with stand-ins that carry the member names of VET's NeuralScene, ReducedImageInfo
    (Eigen-style crop_rotation(r, c), enum camera model), RenderParams and NeuralRenderInfo, hands the shim the same
    call as the tensor binding: images and masks are equal bit for bit, a rotated and scaled crop included."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=4000, K=6, seed=61, num_views=2)
    views = [list(v) for v in _views(scene)]
    c, s_ = np.cos(0.3), np.sin(0.3)
    views[1][5:10] = [0.9, 0.9, 1.5, -0.75, 0.0]   # crop_transform fx, fy, cx, cy, s
    views[1][10:14] = [c, -s_, s_, c]              # crop_rotation, row-major
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    args = (cu(scene.texture), cu(scene.background), cu(scene.position),
            torch.zeros((scene.poses_se3.shape[0], 6), dtype=torch.float64, device="cuda"), cu(scene.intrinsics),
            cu(scene.confidence.reshape(1, -1)), cu(scene.poses_se3))
    want = torch_ops.blend_point_cloud(*args, None, views, scene.num_layers, train=False, use_environment_map=0,
                                       dropout=0, render_mode=render_mode, debug_max_list_length=6,
                                       output_background_mask=1)
    got = torch_ops.adapter_selftest(*args, views, scene.num_layers, render_mode=render_mode, max_list_length=6,
                                     output_background_mask=True)
    assert len(got) == len(want) == 2 * scene.num_layers
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert float(got[0][1].abs().max()) > 0  # the rotated crop shows points
