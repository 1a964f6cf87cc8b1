"""Descriptor records kept by the caller (vetrast_pack_descriptors, vetrast_forward_args.packed_descriptors).

A forward call normally interleaves texture and confidence into 32-byte records on the side, every time. A caller that
renders a scene more than once between changes of its texture writes them once and hands them in. Nothing about the
result may depend on which of the two happened: outputs, lists and gradients are compared bit for bit between the two
ways of calling, the records against their definition (the per-channel reads they replace:
src/lib/rendering/RenderForward.cu:1338-1342; the activation steps: src/lib/models/NeuralTexture.h:38-55), and the
libtorch binding's bookkeeping (which decides by itself when kept records are safe to use) against changes made to
the tensors between calls.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.helpers import kept_mask
from tests.test_gpu_torch_ext import _plain_call
from tests.test_oracle_prepare_adam import FUSED, _raw_scene
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x.astype(np.float64)))


@pytest.mark.parametrize("fused", [False, True], ids=["plain", "activated"])
def test_records_are_the_interleaved_rows(fused, rasterizer):
    scene = _raw_scene(71, num_points=5000, K=8) if fused else synthetic.tiny_scene(num_points=5000, K=8, seed=71)
    params = make_params(scene, **(FUSED if fused else {}))
    packed = rasterizer.pack_descriptors(DeviceScene(scene), params).cpu().numpy()
    Cn = scene.num_channels
    assert packed.shape == (scene.num_points, 8)
    tex = np.abs(scene.texture) if fused else scene.texture
    np.testing.assert_array_equal(packed[:, :Cn], tex.T)
    np.testing.assert_array_equal(packed[:, Cn:4], 0)
    np.testing.assert_array_equal(packed[:, 5:], 0)
    if fused:
        want = _sigmoid(np.float32(params.confidence_scale) * scene.confidence.ravel())
        np.testing.assert_allclose(packed[:, 4], want, rtol=1e-6)
    else:
        np.testing.assert_array_equal(packed[:, 4], scene.confidence.ravel())


@pytest.mark.parametrize("render_mode", [abi.RENDER_FULL_BLEND, abi.RENDER_FUZZY_BLEND, abi.RENDER_BILINEAR_BLEND])
@pytest.mark.parametrize("variant", ["one_view", "two_views_index", "activated"])
def test_kept_records_change_nothing(render_mode, variant, rasterizer):
    """The same call with and without caller-kept records: every output, list and gradient bit for bit."""
    if variant == "activated":
        scene = _raw_scene(72, num_points=6000, K=8, num_views=2)
        extra = dict(FUSED, quirk_background_confidence_leak=1 if render_mode == abi.RENDER_FULL_BLEND else 0)
    else:
        scene = synthetic.tiny_scene(num_points=6000, K=8, seed=73, num_views=1 if variant == "one_view" else 2)
        extra = {}
        if variant == "two_views_index":
            scene.index = np.random.default_rng(4).integers(0, 1500, size=scene.num_points).astype(np.int32)
    params = make_params(scene, need_point_gradient=1, render_mode=render_mode, **extra)
    dev = DeviceScene(scene)
    grads = [torch.from_numpy(g).cuda() for g in scene.grad_out()]
    plain = rasterizer.forward(dev, params)
    plain_grads = rasterizer.backward(plain, grads)
    packed = rasterizer.pack_descriptors(dev, params)
    kept = rasterizer.forward(dev, params, packed=packed)
    # the workspace's own record array is not written by such a call: poison it to show that nothing reads it either
    lay = kept.layout
    kept.workspace[lay.packed_base:lay.packed_base + 32 * scene.num_points].fill_(0xFF)
    kept_grads = rasterizer.backward(kept, grads)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(kept) == 0
    for b in range(len(scene.views)):
        np.testing.assert_array_equal(kept.offsets(b), plain.offsets(b))
        # the places of a list behind the cut hold the rest of its fragments in arrival order, which no two runs share
        m = kept_mask(plain.offsets(b), params.debug_max_list_length)
        np.testing.assert_array_equal(kept.fragments(b)[m], plain.fragments(b)[m])
        if render_mode != abi.RENDER_BILINEAR_BLEND:  # (there the blend can stop before the cut)
            np.testing.assert_array_equal(kept.transmittance(b)[m], plain.transmittance(b)[m])
        np.testing.assert_array_equal(kept.weight(b), plain.weight(b))
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(kept.out[l].cpu().numpy(), plain.out[l].cpu().numpy())
    for key in ("texture", "confidence", "background", "points", "point_count"):
        got, want = kept_grads[key].cpu().numpy(), plain_grads[key].cpu().numpy()
        if variant == "two_views_index" and key in ("texture", "confidence"):
            # rows that several points share through the index are added up with float atomics, in arrival order
            np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-6, err_msg=key)
        else:
            np.testing.assert_array_equal(got, want, err_msg=key)
    assert float(plain_grads["texture"].abs().sum()) > 0


def test_argument_checks(rasterizer):
    scene = synthetic.tiny_scene(num_points=300, seed=74)
    dev = DeviceScene(scene)
    params = make_params(scene)
    lib = rasterizer.lib
    assert lib.vetrast_packed_descriptor_bytes(300) == 300 * 32 and lib.vetrast_packed_descriptor_bytes(-1) == 0
    buf = torch.zeros(300 * 8 + 8, dtype=torch.float32, device="cuda")
    a = abi.PackArgs()
    a.num_points = 300
    a.texture, a.confidence = dev.ptr("texture"), dev.ptr("confidence")
    C.memmove(C.byref(a.params), C.byref(params), C.sizeof(abi.Params))
    a.packed = buf.data_ptr() + 4  # not 32-byte aligned
    assert lib.vetrast_pack_descriptors(rasterizer.ctx, C.byref(a), None) == abi.ERR_INVALID_ARG
    a.packed = None
    assert lib.vetrast_pack_descriptors(rasterizer.ctx, C.byref(a), None) == abi.ERR_INVALID_ARG
    a.packed = buf.data_ptr()
    a.params.num_texture_channels = 5
    assert lib.vetrast_pack_descriptors(rasterizer.ctx, C.byref(a), None) == abi.ERR_INVALID_ARG
    a.params.num_texture_channels = scene.num_channels
    a.num_points = 0
    assert lib.vetrast_pack_descriptors(rasterizer.ctx, C.byref(a), None) == abi.OK
    # a forward call refuses records that are not 32-byte aligned
    res = rasterizer.forward(dev, params)
    args = abi.ForwardArgs()
    C.memmove(C.byref(args), C.byref(res.args), C.sizeof(abi.ForwardArgs))
    args.packed_descriptors = buf.data_ptr() + 16
    assert lib.vetrast_forward(rasterizer.ctx, C.byref(args), None) == abi.ERR_INVALID_ARG
    torch.cuda.synchronize()


def test_the_binding_keeps_records_only_while_the_tensors_stand_still(oracle):
    """Through the libtorch binding: the second call in a row on unchanged tensors packs once, later calls read those
    records; any in-place change of texture or confidence (new version counter) is seen by the next call, which renders
    the new values: a stale set of records cannot be used."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=4000, K=8, seed=75)
    params = make_params(scene)
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    texture, confidence = cu(scene.texture), cu(scene.confidence.reshape(1, -1))
    want = oracle.forward(scene, params).out
    torch_ops.set_keep_packed_descriptors(True)
    calls = torch_ops.kept_descriptor_calls()
    for k in range(4):
        outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence)
        for l in range(scene.num_layers):
            np.testing.assert_array_equal(outs[l].cpu().numpy(), want[l])
        assert torch_ops.kept_descriptor_calls() - calls == max(0, k)  # not the first call, every one after it
    # in-place changes, one tensor at a time
    calls = torch_ops.kept_descriptor_calls()
    texture.mul_(0.5)
    scene.texture = (scene.texture * np.float32(0.5)).astype(np.float32)
    want = oracle.forward(scene, params).out
    outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence)
    assert torch_ops.kept_descriptor_calls() == calls
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(outs[l].cpu().numpy(), want[l])
    outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence)
    assert torch_ops.kept_descriptor_calls() == calls + 1
    confidence.mul_(0.25)
    scene.confidence = (scene.confidence * np.float32(0.25)).astype(np.float32)
    want = oracle.forward(scene, params).out
    for k in range(3):
        outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence)
        for l in range(scene.num_layers):
            np.testing.assert_array_equal(outs[l].cpu().numpy(), want[l])
    assert torch_ops.kept_descriptor_calls() == calls + 3
    # other tensors of the same size and values elsewhere in memory: not mistaken for the ones the records came from
    texture2 = texture.clone().add_(0.125)
    scene.texture = (scene.texture + np.float32(0.125)).astype(np.float32)
    want = oracle.forward(scene, params).out
    outs = _plain_call(scene, torch_ops, texture=texture2, confidence=confidence)
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(outs[l].cpu().numpy(), want[l])
    # switched off: never
    torch_ops.set_keep_packed_descriptors(False)
    calls = torch_ops.kept_descriptor_calls()
    for k in range(3):
        _plain_call(scene, torch_ops, texture=texture2, confidence=confidence)
    assert torch_ops.kept_descriptor_calls() == calls
    torch_ops.set_keep_packed_descriptors(True)


def test_the_binding_keeps_records_for_calls_without_a_backward_pass_only(oracle):
    """Forward calls that are saved for a backward pass interleave inside the call whatever the tensors did since the
    last call (gradient accumulation over unchanged leaves gives the same gradients every time); calls under no_grad
    on the same leaves read kept records from the second one on, with the same images."""
    from vet_amd import torch_ops

    scene = synthetic.tiny_scene(num_points=3000, K=8, seed=76)
    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    texture = cu(scene.texture).requires_grad_(True)
    confidence = cu(scene.confidence.reshape(1, -1)).requires_grad_(True)
    torch_ops.set_keep_packed_descriptors(True)
    grads, images = [], []
    calls = torch_ops.kept_descriptor_calls()
    for k in range(3):
        texture.grad = confidence.grad = None
        outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence, train=True)
        sum((o * o).sum() for o in outs).backward()
        grads.append((texture.grad.clone(), confidence.grad.clone()))
        images.append([o.detach().clone() for o in outs])
    assert torch_ops.kept_descriptor_calls() == calls
    for gt, gc in grads[1:]:
        assert torch.equal(gt, grads[0][0]) and torch.equal(gc, grads[0][1])
    assert float(grads[0][0].abs().sum()) > 0
    with torch.no_grad():
        for k in range(3):
            outs = _plain_call(scene, torch_ops, texture=texture, confidence=confidence)
            for a, b in zip(outs, images[0]):
                assert torch.equal(a, b)
    assert torch_ops.kept_descriptor_calls() == calls + 2
