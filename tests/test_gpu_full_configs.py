"""BASELINE's configurations at their full sizes on the GPU: parity against the oracle (it finishes each in seconds
on the host cores) plus size-independent properties of the domain: the scan totals the accepted (point, layer) pairs,
kept lists are strictly ascending, the blend is a partition of unity, the backward pass is linear in the upstream
gradient and its descriptor/background gradients sum to the pixel count for a constant upstream gradient."""
import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu


def _forward_parity(scene, rasterizer, oracle, threads=16, **overrides):
    params = make_params(scene, **overrides)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    ref = oracle.forward(scene, params, num_threads=threads)
    K = params.debug_max_list_length
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64))
        keep = kept_mask(off, K)
        got = res.fragments(b)
        np.testing.assert_array_equal(got[keep], ref.fragments[b, :int(off[-1])][keep])
        # kept part of every list is strictly ascending in (depth bits, id)
        rank_zero = np.zeros(len(got), dtype=bool)
        rank_zero[off[:-1][np.diff(off) > 0]] = True
        inner = keep & ~rank_zero
        assert np.all(got[inner] > got[np.flatnonzero(inner) - 1])
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    return params, dev, res, ref


def _backward_parity(scene, res, ref, rasterizer, oracle, threads=16):
    grad_out = scene.grad_out()
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    want = oracle.backward(ref, grad_out, num_threads=threads)
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in ("texture", "confidence", "points"):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= 1e-4, key
    # The background gradient is one sum over every pixel of every view (10^7 terms of either sign). Added up in
    # float32 in arrival order, as the reference's atomics and the oracle do, it carries an error of a few 1e-4 of its
    # own, so the GPU value is checked against the same sum in float64: sum_pixels T_final * G.
    bg64 = np.zeros(scene.num_channels)
    for b in range(len(scene.views)):
        for l, (w, h) in enumerate(scene.layer_sizes()):
            T = ref.weight[b, ref.layer_base(l):ref.layer_base(l) + w * h].astype(np.float64).reshape(h, w)
            bg64 += (grad_out[l][b].astype(np.float64) * T[None]).sum(axis=(1, 2))
    err = max_rel_err(got["background"].cpu().numpy(), bg64)
    err_oracle = max_rel_err(want["background"], bg64)
    print(f"  background: max rel err {err:.3e} vs float64 sum (oracle's float32 sum: {err_oracle:.3e})", flush=True)
    assert err <= 1e-4
    assert err_oracle <= 2e-3
    return got


def test_config2_forward_full_size(rasterizer, oracle):
    print("[case] config 2, 2M points, 1080p, forward", flush=True)
    _forward_parity(synthetic.config2(), rasterizer, oracle)


def test_config3_forward_backward_full_size(rasterizer, oracle):
    print("[case] config 3, 2M points, 1080p, forward+backward", flush=True)
    scene = synthetic.config3()
    _, dev, res, ref = _forward_parity(scene, rasterizer, oracle, need_point_gradient=1)
    g1 = _backward_parity(scene, res, ref, rasterizer, oracle)
    # linearity in the upstream gradient: scaling by 2 is exact in binary floating point and every term of the
    # gradients is linear in G, so backward(2 G) must equal 2 backward(G) bit for bit
    go = [torch.from_numpy(g).cuda() * 2.0 for g in scene.grad_out()]
    g2 = rasterizer.backward(res, go)
    torch.cuda.synchronize()
    for key in ("texture", "confidence", "background", "points"):
        np.testing.assert_array_equal(g2[key].cpu().numpy(), 2.0 * g1[key].cpu().numpy(), err_msg=key)


def test_config3_generated_point_order(rasterizer, oracle):
    print("[case] config 3 in the generator's raw point order", flush=True)
    scene = synthetic.config3(point_order="generated")
    _, dev, res, ref = _forward_parity(scene, rasterizer, oracle, need_point_gradient=1)
    _backward_parity(scene, res, ref, rasterizer, oracle)


@pytest.mark.parametrize("drop_by_radius", [0, 1])
def test_config3_without_the_cut_as_vet_ships_it(drop_by_radius, rasterizer, oracle):
    """debug_max_list_length = -1 (configs/config.ini:123): no top-K cut, so the coarse layers blend lists of hundreds to
    thousands of fragments, sorted in full; with and without the radius drop-out VET trains with."""
    print(f"[case] config 3 without a cut, drop_out_points_by_radius={drop_by_radius}, forward+backward", flush=True)
    scene = synthetic.config3(K=-1)
    _, dev, res, ref = _forward_parity(scene, rasterizer, oracle, need_point_gradient=1,
                                       drop_out_points_by_radius=drop_by_radius)
    counts = np.diff(res.offsets(0))
    print(f"  longest list {counts.max()}, lists beyond 64 / 256 / 1024 keys: {(counts > 64).sum()} / "
          f"{(counts > 256).sum()} / {(counts > 1024).sum()}", flush=True)
    _backward_parity(scene, res, ref, rasterizer, oracle)


def test_config4_batch_of_views_full_size(rasterizer, oracle):
    print("[case] config 4, 5.5M points incl. 3 environment spheres, 4 views", flush=True)
    scene = synthetic.config4()
    _, dev, res, ref = _forward_parity(scene, rasterizer, oracle, need_point_gradient=1)
    _backward_parity(scene, res, ref, rasterizer, oracle)


def test_config5_depth_complexity_full_size(rasterizer, oracle):
    print("[case] config 5, 10M points in 1 m^3, K=16", flush=True)
    scene = synthetic.config5()
    params, dev, res, ref = _forward_parity(scene, rasterizer, oracle, need_point_gradient=1)
    off = res.offsets(0)
    counts = np.diff(off)
    P3 = res.layer_bases()[3]
    assert counts[P3:].mean() > 100, "the coarsest layer must average more than 100 fragments per pixel"
    _backward_parity(scene, res, ref, rasterizer, oracle)


def test_partition_of_unity_and_gradient_sum_full_size(rasterizer):
    """Descriptor == 1 and background == 1 render to 1 everywhere; with upstream gradient 1 the descriptor and
    background gradients add up to the number of pixels (no oracle involved)."""
    scene = synthetic.config3()
    scene.texture[:] = 1.0
    scene.background[:] = 1.0
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, make_params(scene))
    ones = [torch.ones_like(o) for o in res.out]
    g = rasterizer.backward(res, ones, want_points=False)
    torch.cuda.synchronize()
    for o in res.out:
        assert float((o - 1).abs().max()) <= 3e-6
    pixels = sum(w * h for w, h in scene.layer_sizes())
    for ci in range(scene.num_channels):
        total = float(g["texture"][ci].double().sum() + g["background"][ci].double())
        assert total == pytest.approx(pixels, rel=1e-5)
