"""Randomised parity sweep: many small scenes with randomly drawn shapes and switches, all three render modes, the HIP
path against the oracle. Every case is seeded and prints its configuration before it runs."""
import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params
from vet_amd.synthetic import ViewSpec

pytestmark = pytest.mark.gpu


def _draw(seed):
    rng = np.random.default_rng(1000 + seed)
    w, h = int(rng.integers(17, 140)), int(rng.integers(17, 100))
    L = int(rng.integers(1, 6))
    while (w >> (L - 1)) < 1 or (h >> (L - 1)) < 1:
        L -= 1
    C = int(rng.integers(1, 5))
    N = int(rng.choice([1, 7, 300, 2500, 12000]))
    K = int(rng.choice([-1, 0, 1, 3, 8, 16, 40]))
    views = int(rng.integers(1, 4))
    scene = synthetic.tiny_scene(num_points=N, w=w, h=h, num_layers=L, K=K, seed=2000 + seed, channels=C, num_views=views)
    # cameras: a small random rotation per view, a crop with skew and a rotated crop now and then
    for b in range(views):
        q = rng.normal(size=4) * [0.05, 0.05, 0.05, 1.0]
        scene.poses_se3[b, :4] = q / np.linalg.norm(q)
    if rng.random() < 0.5:
        ang = rng.uniform(-0.3, 0.3)
        scene.views = [ViewSpec(w, h, image_index=b, crop_transform=(rng.uniform(0.8, 1.2), rng.uniform(0.8, 1.2),
                                                                     rng.uniform(-3, 3), rng.uniform(-3, 3), 0.01),
                                crop_rotation=(np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang))) for b in range(views)]
    if rng.random() < 0.4:
        scene.index = rng.integers(0, max(1, N // 3), size=N).astype(np.int32)
    if rng.random() < 0.3:
        scene.dropout = (rng.random((views, N)) < 0.2).astype(np.float32)
    if rng.random() < 0.4:  # depth levels, so that FUZZY_BLEND buckets and depth ties occur
        scene.position[:, 2] = (np.round(scene.position[:, 2] / 0.25) * 0.25
                                + rng.choice([0.0, 0.004], size=N)).astype(np.float32)
    over = {
        "use_environment_map": int(rng.random() < 0.3),
        "drop_out_points_by_radius": int(rng.random() < 0.3),
        "output_background_mask": int(rng.random() < 0.3),
        "output_background_mask_value": 0.25,
        "need_point_gradient": int(rng.random() < 0.8),
        "quirk_background_confidence_leak": int(rng.random() < 0.5),
        "point_gradient_normalization": int(rng.integers(0, 3)),
        "camera_gradient_normalization": int(rng.random() < 0.5),
        "render_mode": int(rng.choice([1, 2, 3])),
        "depth_accept_blend": float(rng.choice([0.01, 0.1, 0.6])),
    }
    if rng.random() < 0.25:
        over.update(confidence_activation=1, confidence_scale=float(rng.uniform(1, 12)), texture_abs=int(rng.random() < 0.5))
        scene.confidence = (rng.normal(size=N) * 0.3).astype(np.float32)
    if rng.random() < 0.15:
        over.update(viewer_only=1, stability_cutoff_value=0.4)
    want_cameras = bool(rng.random() < 0.4) and over["need_point_gradient"] == 1
    return scene, over, want_cameras


@pytest.mark.parametrize("seed", list(range(48)))
def test_random_case(seed, rasterizer, oracle):
    scene, over, want_cameras = _draw(seed)
    print(f"[case] sweep seed={seed} N={scene.num_points} {scene.views[0].w}x{scene.views[0].h} L={scene.num_layers} "
          f"C={scene.num_channels} K={scene.max_list_length} views={len(scene.views)} index={scene.index is not None} "
          f"dropout={scene.dropout is not None} cameras={want_cameras} {over}", flush=True)
    params = make_params(scene, **over)
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    K = params.debug_max_list_length
    bilinear = over["render_mode"] == abi.RENDER_BILINEAR_BLEND
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64), err_msg="per-pixel counts")
        total = int(off[-1])
        if bilinear:
            kept = res.kept(b)
            np.testing.assert_array_equal(kept, ref.kept[b].astype(np.int64), err_msg="blended counts")
            counts = np.diff(off)
            keep = (np.arange(total) - np.repeat(off[:-1], counts)) < np.repeat(kept, counts)
        else:
            keep = kept_mask(off, K)
        np.testing.assert_array_equal(res.fragments(b)[keep], ref.fragments[b, :total][keep], err_msg="lists")
        np.testing.assert_array_equal(res.transmittance(b)[keep], ref.transmittance[b, :total][keep], err_msg="T")
        np.testing.assert_array_equal(res.weight(b), ref.weight[b], err_msg="weight")
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l], err_msg=f"layer {l}")
        if over["output_background_mask"]:
            np.testing.assert_array_equal(res.out_mask[l].cpu().numpy(), ref.out_mask[l], err_msg=f"mask {l}")
    grad_out = scene.grad_out()
    want_points = over["need_point_gradient"] == 1
    want = oracle.backward(ref, grad_out, want_points=want_points, want_cameras=want_cameras)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_points=want_points,
                              want_cameras=want_cameras)
    torch.cuda.synchronize()
    keys = ["texture", "confidence", "background"] + (["points"] if want_points else []) \
        + (["pose", "intrinsics"] if want_cameras else [])
    if want_points:
        np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in keys:
        g, w_ = got[key].cpu().numpy(), want[key]
        assert np.all(np.isfinite(g)), key
        err = max_rel_err(g, w_) if np.abs(w_).max() > 0 else float(np.abs(g).max())
        assert err <= 1e-4, (key, err)


def _draw_clustered(seed):
    """Scenes whose points crowd into a few spots of the image: bins far beyond the room they own (records go through
    the overflow log), lists of hundreds to thousands of fragments (every sorting method), with a sparse rest."""
    rng = np.random.default_rng(5000 + seed)
    w, h = int(rng.integers(40, 200)), int(rng.integers(30, 120))
    L = int(rng.integers(1, 5))
    N = int(rng.choice([20_000, 60_000, 150_000]))
    K = int(rng.choice([-1, 0, 16, 100]))
    views = int(rng.integers(1, 3))
    scene = synthetic.tiny_scene(num_points=N, w=w, h=h, num_layers=L, K=K, seed=6000 + seed, channels=4, num_views=views)
    spots = int(rng.integers(1, 6))
    crowd = rng.random(N) < rng.uniform(0.5, 0.95)
    centre = rng.uniform(-0.6, 0.6, size=(spots, 2))
    which = rng.integers(0, spots, size=N)
    spread = rng.choice([0.01, 0.05, 0.15, 0.3])
    scene.position[crowd, 0] = (centre[which[crowd], 0] + rng.normal(size=int(crowd.sum())) * spread).astype(np.float32)
    scene.position[crowd, 1] = (centre[which[crowd], 1] * 0.6 + rng.normal(size=int(crowd.sum())) * spread).astype(np.float32)
    if rng.random() < 0.5:  # depth ties
        scene.position[:, 2] = (np.round(scene.position[:, 2] / 0.05) * 0.05).astype(np.float32)
    scene.position = np.ascontiguousarray(scene.position[rng.permutation(N)])
    over = {
        "render_mode": int(rng.choice([1, 2, 3])),
        "depth_accept_blend": 0.05,
        "need_point_gradient": 1,
        "drop_out_points_by_radius": int(rng.random() < 0.2),
        "use_environment_map": int(rng.random() < 0.3),
    }
    return scene, over


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_clustered_case(seed, rasterizer, oracle):
    scene, over = _draw_clustered(seed)
    print(f"[case] clustered sweep seed={seed} N={scene.num_points} {scene.views[0].w}x{scene.views[0].h} "
          f"L={scene.num_layers} K={scene.max_list_length} views={len(scene.views)} {over}", flush=True)
    params = make_params(scene, **over)
    ref = oracle.forward(scene, params, num_threads=8)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    K = params.debug_max_list_length
    bilinear = over["render_mode"] == abi.RENDER_BILINEAR_BLEND
    longest = 0
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64), err_msg="per-pixel counts")
        total = int(off[-1])
        counts = np.diff(off)
        longest = max(longest, int(counts.max()))
        if bilinear:
            kept = res.kept(b)
            np.testing.assert_array_equal(kept, ref.kept[b].astype(np.int64), err_msg="blended counts")
            keep = (np.arange(total) - np.repeat(off[:-1], counts)) < np.repeat(kept, counts)
        else:
            keep = kept_mask(off, K)
        np.testing.assert_array_equal(res.fragments(b)[keep], ref.fragments[b, :total][keep], err_msg="lists")
        np.testing.assert_array_equal(res.transmittance(b)[keep], ref.transmittance[b, :total][keep], err_msg="T")
        np.testing.assert_array_equal(res.weight(b), ref.weight[b], err_msg="weight")
    print(f"  longest list {longest}", flush=True)
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l], err_msg=f"layer {l}")
    tol = 1e-4  # also for uncut lists of tens of thousands of fragments
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, num_threads=8)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in ("texture", "confidence", "points"):
        g, w_ = got[key].cpu().numpy(), want[key]
        assert np.all(np.isfinite(g)), key
        err = max_rel_err(g, w_) if np.abs(w_).max() > 0 else float(np.abs(g).max())
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= tol, (key, err)
