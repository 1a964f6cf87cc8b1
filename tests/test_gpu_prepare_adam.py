"""GPU parity of the fused steps either side of the rasterizer: confidence sigmoid and |texture| folded into the
descriptor interleave with their chain rule in the per-point backward kernel, and the one-kernel Adam step. The
canonical sigmoid is built from +, *, rint and one division, so it agrees with the oracle bit for bit."""
import numpy as np
import pytest
import torch

from tests.helpers import max_rel_err
from tests.test_oracle_prepare_adam import FUSED, _raw_scene
from vet_amd import abi
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("render_mode", [abi.RENDER_FULL_BLEND, abi.RENDER_BILINEAR_BLEND])
@pytest.mark.parametrize("with_index", [False, True])
@pytest.mark.parametrize("num_views", [1, 2])  # (a call with one view interleaves the rows of visible points only)
def test_fused_preparation_matches_oracle(render_mode, with_index, num_views, rasterizer, oracle):
    scene = _raw_scene(51, num_points=6000, K=8, num_views=num_views)
    if with_index:
        scene.index = np.random.default_rng(3).integers(0, 1200, size=scene.num_points).astype(np.int32)
    params = make_params(scene, need_point_gradient=1, render_mode=render_mode, quirk_background_confidence_leak=1,
                         **FUSED)
    ref = oracle.forward(scene, params)
    res = rasterizer.forward(DeviceScene(scene), params)
    torch.cuda.synchronize()
    for b in range(num_views):
        np.testing.assert_array_equal(res.offsets(b), ref.offsets[b].astype(np.int64))
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    go = scene.grad_out()
    want = oracle.backward(ref, go)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in go])
    torch.cuda.synchronize()
    for key in ("texture", "confidence", "background", "points"):
        assert max_rel_err(got[key].cpu().numpy(), want[key]) <= 1e-4, key
    assert (got["texture"].cpu().numpy() < 0).any() and (want["background"] != 0).all()


def test_viewer_cutoff_uses_the_activated_confidence(rasterizer, oracle):
    scene = _raw_scene(52, num_points=4000, K=8)
    params = make_params(scene, viewer_only=1, stability_cutoff_value=0.5, **FUSED)
    ref = oracle.forward(scene, params)
    res = rasterizer.forward(DeviceScene(scene), params, save_for_backward=False)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(res.offsets(0), ref.offsets[0].astype(np.int64))
    visible = int(ref.offsets[0, -1])
    assert 0.2 * scene.num_points * scene.num_layers < visible < 0.8 * scene.num_points * scene.num_layers
    np.testing.assert_array_equal(res.out[0].cpu().numpy(), ref.out[0])


@pytest.mark.parametrize("weight_decay", [0.0, 0.01])
def test_adam_step_is_bit_exact_against_the_oracle(weight_decay, rasterizer, oracle):
    rng = np.random.default_rng(9)
    n = 1_000_003
    p = rng.standard_normal(n).astype(np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    dp, dm, dv = (torch.from_numpy(a.copy()).cuda() for a in (p, m, v))
    for step in range(1, 5):
        g = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 2)).astype(np.float32)
        dg = torch.from_numpy(g.copy()).cuda()
        zero = step % 2 == 0
        oracle.adam_step(p, g, m, v, step, 0.003, 0.9, 0.999, 1e-8, weight_decay, zero_grad=zero)
        rasterizer.adam_step(dp, dg, dm, dv, step, 0.003, 0.9, 0.999, 1e-8, weight_decay, zero_grad=zero)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(dp.cpu().numpy(), p)
        np.testing.assert_array_equal(dm.cpu().numpy(), m)
        np.testing.assert_array_equal(dv.cpu().numpy(), v)
        np.testing.assert_array_equal(dg.cpu().numpy(), g)


def test_adam_step_refuses_bad_arguments(rasterizer):
    a = abi.AdamArgs()
    a.n, a.step = 10, 0
    assert rasterizer.lib.vetrast_adam_step(rasterizer.ctx, a, None) == abi.ERR_INVALID_ARG
    a.step = 1
    assert rasterizer.lib.vetrast_adam_step(rasterizer.ctx, a, None) == abi.ERR_INVALID_ARG  # null tensors
    a.n = 0
    assert rasterizer.lib.vetrast_adam_step(rasterizer.ctx, a, None) == abi.OK
