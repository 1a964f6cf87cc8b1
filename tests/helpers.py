"""Comparison helpers shared by the parity tests."""
import numpy as np


def kept_mask(offsets, K):
    """Boolean mask over the fragment buffer: entry belongs to the first min(count, K) of its pixel list."""
    offsets = np.asarray(offsets, dtype=np.int64)
    counts = np.diff(offsets)
    total = int(offsets[-1])
    rank = np.arange(total, dtype=np.int64) - np.repeat(offsets[:-1], counts)
    if K is None or K <= 0:
        return np.ones(total, dtype=bool)
    return rank < K


def rel_err(a, b, floor_frac=1e-3):
    """Element-wise |a-b| / max(|b|, floor) with floor = floor_frac * max|b| (guards elements that cancel to ~0)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    scale = float(np.max(np.abs(b))) if b.size else 0.0
    floor = max(scale * floor_frac, 1e-30)
    return np.abs(a - b) / np.maximum(np.abs(b), floor)


def max_rel_err(a, b, floor_frac=1e-3):
    e = rel_err(a, b, floor_frac)
    return float(e.max()) if e.size else 0.0


# ---------------------------------------------------------------------------------------------------------------------
# A case small enough to work out on paper: the position heuristic of BlendBackwards2
# (src/lib/rendering/RenderBackward.cu:1346-1377) and of the second half of BlendBackwardsFuzzy (:729-1080).
# ---------------------------------------------------------------------------------------------------------------------
def hand_case():
    """Seven by seven pixels, one layer, camera at the origin looking down +z with fx = 2, fy = 4, cx = 1, cy = -1, so a
    point (X,Y,Z) lands on pixel (2X/Z + 1, 4Y/Z - 1). Only the centre pixel (3,3) is more than two pixels from the
    border, so only its two fragments A and B receive a position gradient. Every number is a multiple of a power of two.

        point  position            pixel   confidence  descriptor
        A      (1, 1, 1)           (3,3)   0.5         (1, 0, 0, 0.5)
        B      (2, 2, 2)           (3,3)   0.5         (0, 1, 0.5, 0)
        C      (1.5, 1, 1)         (4,3)   0.5         (0.5, 0.5, 0, 1)
        C2     C * 1.0078125       (4,3)   0.25        (0, 1, 1, 0.5)      same depth bucket as C in FUZZY_BLEND
        D      (1, 0.75, 1)        (3,2)   0.25        (1, 1, 1, 1)
        E      (0.5, 1, 1)         (2,3)   0.75        (0, 0, 1, 0.5)
        background                                     (0, 1, 0.5, 0.25)

    Returns (scene, grad_out, expected) with expected[mode] = dict(image={pixel: row}, points={0: gA, 1: gB}),
    mode in ("full", "fuzzy"); the literals below were worked out by hand, the steps are in the comments."""
    from vet_amd import synthetic

    s = 1.0078125
    position = np.array([[1, 1, 1, 1], [2, 2, 2, 1], [1.5, 1, 1, 1], [1.5 * s, 1 * s, s, 1], [1, 0.75, 1, 1],
                         [0.5, 1, 1, 1]], dtype=np.float32)
    texture = np.array([[1, 0, 0, 0.5], [0, 1, 0.5, 0], [0.5, 0.5, 0, 1], [0, 1, 1, 0.5], [1, 1, 1, 1],
                        [0, 0, 1, 0.5]], dtype=np.float32).T.copy()
    confidence = np.array([0.5, 0.5, 0.5, 0.25, 0.25, 0.75], dtype=np.float32)
    background = np.array([0, 1, 0.5, 0.25], dtype=np.float32)
    scene = synthetic.Scene("hand", position, texture, confidence, background, synthetic._identity_pose((0, 0, 0)),
                            synthetic._intrinsics(2.0, 4.0, 1.0, -1.0), [synthetic.ViewSpec(7, 7)], num_layers=1,
                            max_list_length=4, seed=0)
    G = np.zeros((1, 4, 7, 7), dtype=np.float32)
    G[0, :, 3, 2] = [1, 2, -1, 0]       # px0 = (2,3)
    G[0, :, 3, 4] = [2, 0, 1, -1]       # px1 = (4,3)
    G[0, :, 2, 3] = [-1, 1, 0, 2]       # py0 = (3,2)
    G[0, :, 4, 3] = [0.5, -1, 2, 4]     # py1 = (3,4)
    G[0, :, 3, 3] = [1, 1, 1, 1]        # the centre: feeds the value gradients only

    # Forward image, front to back, colour += T * conf * t, T *= 1 - conf, background with what is left:
    #   (3,3) = .5 A + .25 B + .25 bg                      = (.5, .5, .25, .3125)
    #   (2,3) = .75 E + .25 bg                              = (0, .25, .875, .4375)
    #   (3,2) = .25 D + .75 bg                              = (.25, 1, .625, .4375)
    #   (3,4) = bg
    #   (4,3) FULL : .5 C + .5*.25 C2 + .375 bg             = (.25, .75, .3125, .65625)
    #   (4,3) FUZZY: one bucket, mean confidence .375, mean descriptor (.25, .75, .5, .75):
    #                .375 mean + .625 bg                    = (.09375, .90625, .5, .4375)
    common = {(3, 3): [.5, .5, .25, .3125], (2, 3): [0, .25, .875, .4375], (3, 2): [.25, 1, .625, .4375],
              (3, 4): [0, 1, .5, .25], (0, 0): [0, 1, .5, .25]}
    # Heuristic for a fragment with descriptor t at (3,3), four channels:
    #   dx = ( -(t - I(2,3)).G(2,3) + (t - I(4,3)).G(4,3) ) / 2 / 4,   dy likewise with (3,2) and (3,4).
    # A, t = (1,0,0,.5):
    #   (t-I(2,3)).G = (1,-.25,-.875,.0625).(1,2,-1,0)      = 1.375
    #   (t-I(3,2)).G = (.75,-1,-.625,.0625).(-1,1,0,2)      = -1.625
    #   (t-I(3,4)).G = (1,-1,-.5,.25).(.5,-1,2,4)           = 1.5            dy = (1.625 + 1.5)/8 = .390625
    #   FULL : (t-I(4,3)).G = (.75,-.75,-.3125,-.15625).(2,0,1,-1) = 1.34375  dx = (-1.375 + 1.34375)/8 = -.00390625
    #   FUZZY: (t-I(4,3)).G = (.90625,-.90625,-.5,.0625).(2,0,1,-1) = 1.25    dx = (-1.375 + 1.25)/8 = -.015625
    # B, t = (0,1,.5,0):
    #   (t-I(2,3)).G = (0,.75,-.375,-.4375).(1,2,-1,0)      = 1.875
    #   (t-I(3,2)).G = (-.25,0,-.125,-.4375).(-1,1,0,2)     = -.625
    #   (t-I(3,4)).G = (0,0,0,-.25).(.5,-1,2,4)             = -1             dy = (.625 - 1)/8 = -.046875
    #   FULL : (t-I(4,3)).G = (-.25,.25,.1875,-.65625).(2,0,1,-1) = .34375    dx = (-1.875 + .34375)/8 = -.19140625
    #   FUZZY: (t-I(4,3)).G = (-.09375,.09375,0,-.4375).(2,0,1,-1) = .25      dx = (-1.875 + .25)/8 = -.203125
    # Chain through the projection u = 2X/Z + 1, v = 4Y/Z - 1:  g = (2 dx / Z, 4 dy / Z, -(2X dx + 4Y dy) / Z^2).
    #   A (1,1,1): (2dx, 4dy, -2dx - 4dy)        B (2,2,2): (dx, 2dy, -dx - 2dy)
    expected = {
        "full": dict(image={**common, (4, 3): [.25, .75, .3125, .65625]},
                     points={0: [-.0078125, 1.5625, -1.5546875], 1: [-.19140625, -.09375, .28515625]}),
        "fuzzy": dict(image={**common, (4, 3): [.09375, .90625, .5, .4375]},
                      points={0: [-.03125, 1.5625, -1.53125], 1: [-.203125, -.09375, .296875]}),
    }
    return scene, [G], expected


def check_hand_case(out0, points, point_count, want):
    """out0 [1,4,7,7] the forward image, points [N,4] and point_count [N] from the backward pass."""
    for (x, y), row in want["image"].items():
        np.testing.assert_allclose(out0[0, :, y, x], row, rtol=0, atol=1e-6, err_msg=f"pixel {(x, y)}")
    np.testing.assert_array_equal(point_count, [1, 1, 0, 0, 0, 0])
    for i, g in want["points"].items():
        np.testing.assert_allclose(points[i, :3], g, rtol=0, atol=2e-6, err_msg=f"point {i}")
    assert not points[2:].any() and not points[:, 3].any()


# ---------------------------------------------------------------------------------------------------------------------
# BILINEAR_BLEND backward in O(n) per pixel list
# ---------------------------------------------------------------------------------------------------------------------
def bilinear_backward_model(oracle, fwd, grad_out, use_env=False):
    """Float64 statement of BlendBackwardsBilinear (src/lib/rendering/RenderBackward.cu:2936-3175) that replaces the
    kernel's loop over all earlier fragments (:2987-3012) by a suffix sum. With a_i = weight_i * confidence_i,
    T_i = prod_{j<i} (1 - a_j) and d_i = <descriptor_i, G> the kernel leaves in gradient_sum_backwards

        s_i = T_i d_i  -  ( sum_{k>i} T_k a_k d_k ) / (1 - a_i + 1e-9),

    the sum running over the later blended fragments and the background (a = 1) where the list did not stop early.
    The lists, the number of blended fragments and the transmittance behind them are taken from the forward result
    `fwd` of the oracle; the projection is the oracle's float32 one (so that floor() agrees), its Jacobian a central
    difference of the float64 textbook projection. Returns the gradient dict of oracle.backward (no cameras)."""
    from tests.test_oracle_pinning import project64

    scene = fwd.scene
    Cn, N = scene.num_channels, scene.num_points
    tex = scene.texture.astype(np.float64)
    conf = scene.confidence.astype(np.float64)
    bg = scene.background.astype(np.float64)
    index = np.arange(N) if scene.index is None else scene.index.astype(np.int64)
    K = fwd.params.debug_max_list_length
    res = dict(texture=np.zeros((Cn, tex.shape[1])), confidence=np.zeros(tex.shape[1]), background=np.zeros(Cn),
               points=np.zeros((N, 4)), point_count=np.zeros(N))
    jacobian, image_pos = {}, {}
    for b, v in enumerate(scene.views):
        prepared = oracle.prepare_view(scene.poses_se3[v.image_index], scene.intrinsics[v.camera_index])
        crop = np.array(v.crop_transform, np.float32).astype(np.float64)
        rot = np.array(v.crop_rotation, np.float32).astype(np.float64)
        K5 = scene.intrinsics[v.camera_index][:5].astype(np.float64)

        def point(i):
            if (b, i) not in image_pos:
                ok, pr = oracle.project_point(prepared, fwd.views[b], scene.position[i])
                assert ok
                image_pos[(b, i)] = (np.float32(pr[0]), np.float32(pr[1]))
                p = scene.position[i].astype(np.float64)
                J = np.zeros((2, 3))
                for k in range(3):
                    e = np.zeros(4)
                    e[k] = 1e-6
                    hi, _ = project64(p + e, scene.poses_se3[v.image_index], K5, crop, rot, v.w, v.h)
                    lo, _ = project64(p - e, scene.poses_se3[v.image_index], K5, crop, rot, v.w, v.h)
                    J[:, k] = (hi - lo) / 2e-6
                jacobian[(b, i)] = J
            return image_pos[(b, i)], jacobian[(b, i)]

        for l, (w, h) in enumerate(fwd.sizes):
            G = grad_out[l][b].astype(np.float64)
            for y in range(h):
                for x in range(w):
                    q = fwd.layer_base(l) + y * w + x
                    n = int(fwd.kept[b, q])
                    with_background = (not use_env) and float(fwd.weight[b, q]) >= 0.001
                    keys = fwd.pixel_list(b, l, x, y)[:n]
                    ids = (keys & np.uint64(0xFFFFFFFF)).astype(np.int64) >> 2
                    corner = (keys & np.uint64(3)).astype(np.int64)
                    g = G[:, y, x]
                    wgt = np.zeros(n)
                    dw = np.zeros((n, 2))
                    for t in range(n):
                        (u32, v32), _ = point(int(ids[t]))
                        for _ in range(l):
                            u32, v32 = np.float32(u32 * np.float32(0.5)), np.float32(v32 * np.float32(0.5))
                        sx, sy = float(u32 - np.floor(u32)), float(v32 - np.floor(v32))
                        wgt[t] = [(1 - sx) * (1 - sy), sx * (1 - sy), (1 - sx) * sy, sx * sy][corner[t]]
                        dw[t] = [(sy - 1, sx - 1), (1 - sy, -sx), (-sy, 1 - sx), (sy, sx)][corner[t]]
                    rows = index[ids]
                    a = wgt * conf[rows]
                    T = np.concatenate([[1.0], np.cumprod(1.0 - a)])      # T[n] is what is left behind the list
                    d = tex[:, rows].T @ g                                 # [n]
                    term = T[:n] * a * d
                    tail = T[n] * float(bg @ g) if with_background else 0.0
                    later = np.concatenate([np.cumsum(term[::-1])[::-1][1:], [0.0]]) + tail
                    s = T[:n] * d - later / (1.0 - a + 1e-9)
                    np.add.at(res["texture"].T, rows, (T[:n] * a)[:, None] * g[None, :])
                    if with_background:
                        res["background"] += T[n] * g
                    if min(x, y, w - 1 - x, h - 1 - y) <= 2:
                        continue
                    np.add.at(res["confidence"], rows, wgt * s)
                    for t in range(n):
                        _, J = point(int(ids[t]))
                        res["points"][ids[t], :3] += (0.5 ** l) * (J.T @ dw[t]) * conf[rows[t]] * s[t]
                        res["point_count"][ids[t]] += 1
    return res
