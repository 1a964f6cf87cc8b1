"""GPU parity of FUZZY_BLEND (render_mode 2): the HIP path through the C ABI against the CPU oracle.

Bars as for the other modes: lists, stored transmittances, weights and blended features bit-exact (same operation
order), gradients within 1e-4 relative.
"""
import numpy as np
import pytest
import torch

from tests.helpers import kept_mask, max_rel_err
from vet_amd import abi, synthetic
from vet_amd.rasterizer import DeviceScene, make_params

pytestmark = pytest.mark.gpu
MODE = dict(render_mode=abi.RENDER_FUZZY_BLEND)


def _levels(scene, step=0.25, seed=5):
    """Moves the points onto depth levels with a jitter below the default depth range, so that buckets form everywhere."""
    rng = np.random.default_rng(seed)
    level = np.round(scene.position[:, 2] / step)
    scene.position[:, 2] = (level * step + rng.uniform(0.0, 0.008, len(level))).astype(np.float32)
    return scene


def _far(scene, depth=95000.0):
    """Moves the points out along their viewing rays (the tiny scene's camera looks down z from z = -2)."""
    z = scene.position[:, 2].astype(np.float64) + 2.0
    scale = (z + depth) / z
    scene.position[:, 0] = (scene.position[:, 0] * scale).astype(np.float32)
    scene.position[:, 1] = (scene.position[:, 1] * scale).astype(np.float32)
    scene.position[:, 2] = (z + depth - 2.0).astype(np.float32)
    return scene


def _scenes():
    yield "tiny_K4", synthetic.tiny_scene(), {}
    yield "tiny_levels_K8", _levels(synthetic.tiny_scene(num_points=6000, K=8, seed=81)), {}
    yield "tiny_levels_nocut_3ch", _levels(synthetic.tiny_scene(num_points=5000, K=-1, channels=3, seed=82)), {}
    yield "tiny_long_lists_levels", _levels(synthetic.tiny_scene(num_points=40000, K=0, seed=83)), {}
    yield "tiny_long_lists_K16", _levels(synthetic.tiny_scene(num_points=40000, K=16, seed=84)), {}
    # a cut of 17 to 32 lays lists of up to 32 fragments out densely, in slots of 32 lanes that span two rows of the
    # wave (more slots than a wave's table holds at once: it goes through them in batches); beyond that cut lists of
    # more than 16 fragments are taken a wave per list (those of up to 64 in one pass, longer ones in two)
    yield "tiny_long_lists_K24", _levels(synthetic.tiny_scene(num_points=40000, K=24, seed=99)), {}
    yield "tiny_long_lists_K40", _levels(synthetic.tiny_scene(num_points=40000, K=40, seed=97)), {}
    yield "tiny_long_lists_K64_3ch", _levels(synthetic.tiny_scene(num_points=40000, K=64, channels=3, seed=100)), {}
    yield "tiny_long_lists_K100", _levels(synthetic.tiny_scene(num_points=40000, K=100, seed=98)), {}
    # the lengths either side of a change of method: 17 (first slot of 32 lanes), 33 (first list for the wave-per-list
    # kernel under a cut beyond 32), 65 (first list of two steps: one element in the second)
    yield "tiny_long_lists_K17", _levels(synthetic.tiny_scene(num_points=40000, K=17, seed=105)), {}
    yield "tiny_long_lists_K33", _levels(synthetic.tiny_scene(num_points=40000, K=33, seed=106)), {}
    yield "tiny_long_lists_K65", _levels(synthetic.tiny_scene(num_points=40000, K=65, seed=107)), {}
    yield "tiny_2views_envmap", _levels(synthetic.tiny_scene(num_points=3000, K=8, num_views=2, seed=85)), \
        {"use_environment_map": 1}
    yield "wide_depth_range", synthetic.tiny_scene(num_points=5000, K=12, seed=86), {"depth_accept_blend": 0.3}
    yield "odd_size_5_layers", _levels(synthetic.tiny_scene(num_points=9000, w=83, h=61, num_layers=5, K=6, seed=87)), {}
    # a depth range that covers the nearest fragments from zero (they join the bucket that is open from the start,
    # RenderBackward.cu:706-714), one that covers all fragments, and one that also covers the background element at
    # depth 1e5 (the largest range the library takes is 1e4, so the points are moved out to 95 000); each with short
    # lists and with lists too long for the kernel that lays fragments out densely
    yield "range_reaches_zero_K8", synthetic.tiny_scene(num_points=3000, K=8, seed=90), {"depth_accept_blend": 2.0}
    # (8 000 points: buckets of up to some two hundred elements. With 30 000 the oracle's own float32 sums over buckets
    # of 800 elements, added front to back as the reference adds them, are 2e-6 off a float64 evaluation of the same
    # formulas, which is beyond the bar below for the smallest gradients; the library's pairwise sums are not.)
    yield "range_reaches_zero_nocut", synthetic.tiny_scene(num_points=8000, K=-1, seed=91), {"depth_accept_blend": 2.0}
    yield "one_bucket_K8", synthetic.tiny_scene(num_points=3000, K=8, seed=92), {"depth_accept_blend": 9.0e3}
    yield "one_bucket_nocut", synthetic.tiny_scene(num_points=30000, K=-1, seed=93), {"depth_accept_blend": 9.0e3}
    yield "background_in_last_bucket_K8", _far(synthetic.tiny_scene(num_points=3000, K=8, seed=95)), \
        {"depth_accept_blend": 9.0e3}
    yield "background_in_last_bucket_nocut", _far(synthetic.tiny_scene(num_points=30000, K=-1, seed=96)), \
        {"depth_accept_blend": 9.0e3}
    yield "range_reaches_zero_K28", synthetic.tiny_scene(num_points=8000, K=28, seed=101), {"depth_accept_blend": 2.0}
    yield "range_reaches_zero_K48", synthetic.tiny_scene(num_points=8000, K=48, seed=104), {"depth_accept_blend": 2.0}
    yield "one_bucket_K64", synthetic.tiny_scene(num_points=30000, K=64, seed=102), {"depth_accept_blend": 9.0e3}
    yield "one_bucket_K65", synthetic.tiny_scene(num_points=30000, K=65, seed=108), {"depth_accept_blend": 9.0e3}
    yield "background_in_last_bucket_K32", _far(synthetic.tiny_scene(num_points=30000, K=32, seed=103)), \
        {"depth_accept_blend": 9.0e3}
    yield "single_fragments_K1", _levels(synthetic.tiny_scene(num_points=6000, K=1, seed=94)), {}
    yield "config1", synthetic.config1(), {"depth_accept_blend": 0.05}
    yield "config2_200k", synthetic.config2(num_points=200_000), {"depth_accept_blend": 0.05}


SCENES = list(_scenes())


def _check_forward(scene, overrides, rasterizer, oracle):
    params = make_params(scene, **{**MODE, **overrides})
    ref = oracle.forward(scene, params)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    torch.cuda.synchronize()
    assert rasterizer.check_device_flags(res) == 0
    K = params.debug_max_list_length
    for b in range(len(scene.views)):
        off = res.offsets(b)
        np.testing.assert_array_equal(off, ref.offsets[b].astype(np.int64))
        total = int(off[-1])
        keep = kept_mask(off, K)
        np.testing.assert_array_equal(res.fragments(b)[keep], ref.fragments[b, :total][keep])
        np.testing.assert_array_equal(res.transmittance(b)[keep], ref.transmittance[b, :total][keep])
        np.testing.assert_array_equal(res.weight(b), ref.weight[b])
    for l in range(scene.num_layers):
        np.testing.assert_array_equal(res.out[l].cpu().numpy(), ref.out[l])
    return params, ref, dev, res


@pytest.mark.parametrize("name,scene,overrides", SCENES, ids=[s[0] for s in SCENES])
def test_forward_matches_oracle(name, scene, overrides, rasterizer, oracle):
    print(f"[case] fuzzy forward {name} N={scene.num_points}", flush=True)
    _check_forward(scene, overrides, rasterizer, oracle)


@pytest.mark.parametrize("name,scene,overrides", SCENES, ids=[s[0] for s in SCENES])
def test_backward_matches_oracle(name, scene, overrides, rasterizer, oracle):
    print(f"[case] fuzzy backward {name} N={scene.num_points}", flush=True)
    overrides = dict(overrides, need_point_gradient=1)
    params, ref, dev, res = _check_forward(scene, overrides, rasterizer, oracle)
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in ("texture", "confidence", "background", "points"):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= 1e-4, key


def test_fuzzy_differs_from_full_blend_on_levels(rasterizer):
    """The mode is not FULL_BLEND under another name: where several fragments share the nearest level the image
    changes; with a vanishing depth range it is FULL_BLEND bit for bit."""
    scene = _levels(synthetic.tiny_scene(num_points=6000, K=8, seed=88))
    dev = DeviceScene(scene)
    full = [o.clone() for o in rasterizer.forward(dev, make_params(scene)).out]
    fuzzy = [o.clone() for o in rasterizer.forward(dev, make_params(scene, **MODE)).out]
    same = [o.clone() for o in rasterizer.forward(dev, make_params(scene, depth_accept_blend=1e-12, **MODE)).out]
    torch.cuda.synchronize()
    assert max(float((a - b).abs().max()) for a, b in zip(full, fuzzy)) > 1e-3
    for a, b in zip(full, same):
        assert torch.equal(a, b)


def test_leak_switch_has_no_effect_and_index_indirection(rasterizer, oracle):
    """The background never adds to confidence row 0 in this mode (guarded in the reference), whatever the switch
    says; several points sharing a descriptor row add up."""
    scene = _levels(synthetic.tiny_scene(num_points=4000, K=8, seed=89))
    rng = np.random.default_rng(1)
    scene.index = rng.integers(0, 500, size=scene.num_points).astype(np.int32)
    params, ref, dev, res = _check_forward(scene, {"quirk_background_confidence_leak": 1}, rasterizer, oracle)
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, want_points=False)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_points=False)
    torch.cuda.synchronize()
    for key in ("texture", "confidence", "background"):
        assert max_rel_err(got[key].cpu().numpy(), want[key]) <= 1e-4, key
    params0 = make_params(scene, **MODE)
    ref0 = oracle.forward(scene, params0)
    want0 = oracle.backward(ref0, grad_out, want_points=False)
    np.testing.assert_array_equal(want0["confidence"], want["confidence"])


def test_config3_full_size(rasterizer, oracle):
    print("[case] fuzzy config 3, 2M points, 1080p, forward+backward", flush=True)
    scene = synthetic.config3()
    over = {"need_point_gradient": 1, "depth_accept_blend": 0.05}
    params, ref, dev, res = _check_forward(scene, over, rasterizer, oracle)
    grad_out = scene.grad_out()
    want = oracle.backward(ref, grad_out, num_threads=16)
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out])
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got["point_count"].cpu().numpy(), want["point_count"])
    for key in ("texture", "confidence", "points"):
        err = max_rel_err(got[key].cpu().numpy(), want[key])
        print(f"  {key}: max rel err {err:.3e}", flush=True)
        assert err <= 1e-4, key
    # the background gradient is one float32 sum over 2.75 M pixels on either side: compare loosely, as for FULL_BLEND
    assert max_rel_err(got["background"].cpu().numpy(), want["background"]) <= 2e-3


def test_depth_range_is_checked(rasterizer):
    scene = synthetic.tiny_scene(num_points=500)
    dev = DeviceScene(scene)
    for bad in (0.0, -1.0, 1e5, float("nan")):
        with pytest.raises(abi.VetrastError) as e:
            rasterizer.forward(dev, make_params(scene, depth_accept_blend=bad, **MODE))
        assert e.value.status == abi.ERR_INVALID_ARG
    rasterizer.forward(dev, make_params(scene, depth_accept_blend=0.0))  # ignored by the other modes


def _float64_model(scene, res, grad_out, depth_accept):
    """BlendBackwardsFuzzy's value gradients (src/lib/rendering/RenderBackward.cu:570-727) evaluated in float64 from the
    lists the forward pass left: bucket boundaries by the float32 comparison the kernels make, everything else (bucket
    means, transmittance chain, bucket terms, the sum of the later buckets' terms) in double precision. One view, no
    texture index, no environment map. Returns (d texture [C,N], d confidence [N], d background [C])."""
    N, C = scene.num_points, scene.num_channels
    off, keys = res.offsets(0), res.fragments(0)
    depth32 = (keys >> np.uint64(32)).astype(np.uint32).view(np.float32)
    pid = (keys & np.uint64(0xFFFFFFFF)).astype(np.int64)
    conf, tex = scene.confidence.astype(np.float64), scene.texture.astype(np.float64)
    bg = scene.background.astype(np.float64)
    g_tex, g_conf, g_bg = np.zeros((C, N)), np.zeros(N), np.zeros(C)
    accept = np.float32(depth_accept)
    bases = res.layer_bases()
    for l, (w, h) in enumerate(scene.layer_sizes()):
        G = grad_out[l][0].astype(np.float64).reshape(C, -1)
        for local in range(w * h):
            q = bases[l] + local
            lo, hi = int(off[q]), int(off[q + 1])
            g = G[:, local]
            d, ids = depth32[lo:hi], pid[lo:hi]
            heads, last_min = [], np.float32(0.0)
            for i in range(hi - lo):
                if not (np.float32(d[i] - last_min) < accept):
                    last_min = d[i]
                    heads.append(i)
                elif i == 0:
                    heads.append(0)
            joins = hi > lo and bool(np.float32(np.float32(100000.0) - last_min) < accept)  # background into the last bucket
            A, terms, buckets = 1.0, [], []
            for b, s_ in enumerate(heads):
                e_ = heads[b + 1] if b + 1 < len(heads) else hi - lo
                last = b + 1 == len(heads)
                m = e_ - s_ + (1 if last and joins else 0)
                bc = (conf[ids[s_:e_]].sum() + (1.0 if last and joins else 0.0)) / m
                tb = (tex[:, ids[s_:e_]].sum(axis=1) + (bg if last and joins else 0.0)) / m
                dot = float((tb * g).sum())
                buckets.append((s_, e_, m, bc, dot, A, last and joins))
                terms.append(dot * A * bc)
                A *= 1.0 - bc
            total = sum(terms) + (0.0 if joins else float((g * bg).sum()) * A)
            if not joins:
                g_bg += A * g
            prefix = 0.0
            for (s_, e_, m, bc, dot, Ab, with_bg), x in zip(buckets, terms):
                prefix += x
                np.add.at(g_conf, ids[s_:e_], dot * Ab / m - (total - prefix) / ((1.0 - bc) + 1e-9))
                np.add.at(g_tex, (slice(None), ids[s_:e_]), (Ab * bc / m) * g[:, None])
                if with_bg:
                    g_bg += (Ab * bc / m) * g
    return g_tex, g_conf, g_bg


def test_long_buckets_against_a_float64_evaluation(rasterizer, oracle):
    """Lists of hundreds to thousands of fragments in two or three buckets per pixel. The oracle adds a bucket's
    confidences and descriptors up front to back in float32, as the reference does; over 800 elements that sum alone is
    a few 1e-6 off. The library combines pairwise. Both are compared with the same formulas in float64: the library
    must agree within half the bar the oracle comparisons use (observed 2e-5, the oracle 2e-4)."""
    scene = synthetic.tiny_scene(num_points=30000, K=-1, seed=91)
    params = make_params(scene, depth_accept_blend=2.0, need_point_gradient=0, **MODE)
    dev = DeviceScene(scene)
    res = rasterizer.forward(dev, params, save_for_backward=True)
    grad_out = scene.grad_out()
    got = rasterizer.backward(res, [torch.from_numpy(g).cuda() for g in grad_out], want_points=False)
    torch.cuda.synchronize()
    assert int(np.diff(res.offsets(0)).max()) > 1000, "the scene is meant to have very long lists"
    m_tex, m_conf, m_bg = _float64_model(scene, res, grad_out, 2.0)
    want = oracle.backward(oracle.forward(scene, params), grad_out, want_points=False)
    for key, model in (("texture", m_tex), ("confidence", m_conf), ("background", m_bg)):
        lib_err = max_rel_err(got[key].cpu().numpy().astype(np.float64), model)
        oracle_err = max_rel_err(want[key].astype(np.float64), model)
        print(f"  {key}: library vs float64 {lib_err:.2e}, oracle vs float64 {oracle_err:.2e}", flush=True)
        assert lib_err <= 5e-5, key
        assert oracle_err <= 1e-3, key
