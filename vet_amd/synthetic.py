"""Seeded synthetic scenes for the rasterizer's five benchmark / parity configurations.

All random numbers come from one in-repo counter-based generator (SplitMix64 finaliser over key + counter), evaluated
on the host with numpy, so that the CPU check and the GPU path see identical bits. Uniforms use the top 24 bits, so
they are exact in float32; normals are Box-Muller in float64, rounded once to float32.
"""
import math
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_MASK = (1 << 64) - 1


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def _fnv1a(tag: str) -> int:
    h = 0xCBF29CE484222325
    for ch in tag.encode():
        h = ((h ^ ch) * 0x100000001B3) & _MASK
    return h


class Stream:
    """Independent random stream per (seed, tag)."""

    def __init__(self, seed: int, tag: str):
        with np.errstate(over="ignore"):
            k = np.array([(seed * 0x9E3779B97F4A7C15 + _fnv1a(tag)) & _MASK], dtype=np.uint64)
            self.key = _mix(k)[0]
        self.counter = 0

    def u64(self, n: int) -> np.ndarray:
        idx = np.arange(self.counter + 1, self.counter + n + 1, dtype=np.uint64)
        self.counter += n
        with np.errstate(over="ignore"):
            return _mix(self.key + idx * _GOLDEN)

    def uniform(self, n: int) -> np.ndarray:
        """float64 in [0, 1) with 24 significant bits."""
        return (self.u64(n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)

    def normal(self, n: int) -> np.ndarray:
        u1 = ((self.u64(n) >> np.uint64(40)).astype(np.float64) + 1.0) / float(1 << 24)
        u2 = (self.u64(n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
        return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * math.pi * u2)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


@dataclass
class ViewSpec:
    w: int
    h: int
    image_index: int = 0
    camera_index: int = 0
    camera_model_type: int = 0
    crop_transform: tuple = (1.0, 1.0, 0.0, 0.0, 0.0)
    crop_rotation: tuple = (1.0, 0.0, 0.0, 1.0)


@dataclass
class Scene:
    """Host-side inputs of one render call (numpy, C-contiguous) in the layouts the C ABI expects."""
    name: str
    position: np.ndarray      # [N,4] f32
    texture: np.ndarray       # [C,N] f32
    confidence: np.ndarray    # [N] f32
    background: np.ndarray    # [C] f32
    poses_se3: np.ndarray     # [F,8] f64
    intrinsics: np.ndarray    # [Ncam,13] f32
    views: List[ViewSpec]
    num_layers: int
    max_list_length: int
    seed: int
    index: Optional[np.ndarray] = None    # [N] i32
    dropout: Optional[np.ndarray] = None  # [B,N] f32
    params: dict = field(default_factory=dict)

    @property
    def num_points(self):
        return int(self.position.shape[0])

    @property
    def num_channels(self):
        return int(self.texture.shape[0])

    def layer_sizes(self):
        w, h = self.views[0].w, self.views[0].h
        out = []
        for _ in range(self.num_layers):
            out.append((w, h))
            w //= 2
            h //= 2
        return out

    def grad_out(self, seed_offset=0):
        """Upstream gradient N(0,1) per output element, one array [B,C,h_l,w_l] per layer."""
        res = []
        B, Cn = len(self.views), self.num_channels
        for l, (w, h) in enumerate(self.layer_sizes()):
            st = Stream(self.seed + seed_offset, f"grad_out_{l}")
            res.append(st.normal(B * Cn * h * w).astype(np.float32).reshape(B, Cn, h, w))
        return res


def _identity_pose(t):
    return np.array([[0.0, 0.0, 0.0, 1.0, t[0], t[1], t[2], 0.0]], dtype=np.float64)


def _intrinsics(fx, fy, cx, cy, s=0.0):
    k = np.zeros((1, 13), dtype=np.float32)
    k[0, :5] = [fx, fy, cx, cy, s]
    return k


def config1(num_points=20000, seed=0) -> Scene:
    """Tiny case: uniform cube, 256x256, one layer, K=8, forward only."""
    N = num_points
    pos = np.empty((N, 4), dtype=np.float32)
    pos[:, :3] = (Stream(seed, "position").uniform(3 * N).reshape(N, 3) - 0.5).astype(np.float32)
    pos[:, 3] = 0.01
    tex = Stream(seed, "texture").uniform(4 * N).reshape(4, N).astype(np.float32)
    conf = sigmoid(Stream(seed, "confidence").normal(N)).astype(np.float32)
    return Scene("config1_cube20k", pos, tex, conf, np.zeros(4, np.float32), _identity_pose((0, 0, 2.0)),
                 _intrinsics(256, 256, 128, 128), [ViewSpec(256, 256)], num_layers=1, max_list_length=8, seed=seed)


def _orthonormal_frame(n):
    n = n / np.linalg.norm(n, axis=1, keepdims=True)
    helper = np.where(np.abs(n[:, :1]) < 0.9, np.array([[1.0, 0.0, 0.0]]), np.array([[0.0, 1.0, 0.0]]))
    u = np.cross(n, helper)
    u /= np.linalg.norm(u, axis=1, keepdims=True)
    v = np.cross(n, u)
    return n, u, v


def surface_points(seed, num_primitives, points_per_primitive, box=5.0, jitter=0.01, tag=""):
    """Points on random plane patches and spheres inside [-box, box]^3 with N(0, jitter) noise, float64 [n,3]."""
    Pn, M = num_primitives, points_per_primitive
    st = Stream(seed, "primitives" + tag)
    is_sphere = st.uniform(Pn) < 0.5
    centre = (st.uniform(3 * Pn).reshape(Pn, 3) * 2.0 - 1.0) * box
    normal = st.normal(3 * Pn).reshape(Pn, 3)
    size = 0.5 + 1.5 * st.uniform(Pn)
    n, u, v = _orthonormal_frame(normal)
    sp = Stream(seed, "surface" + tag)
    a = sp.uniform(Pn * M).reshape(Pn, M) * 2.0 - 1.0
    b = sp.uniform(Pn * M).reshape(Pn, M) * 2.0 - 1.0
    d = sp.normal(3 * Pn * M).reshape(Pn, M, 3)
    d /= np.maximum(np.linalg.norm(d, axis=2, keepdims=True), 1e-12)
    plane = centre[:, None, :] + size[:, None, None] * (a[..., None] * u[:, None, :] + b[..., None] * v[:, None, :])
    sphere = centre[:, None, :] + (0.5 * size)[:, None, None] * d
    pts = np.where(is_sphere[:, None, None], sphere, plane).reshape(Pn * M, 3)
    pts += jitter * Stream(seed, "jitter" + tag).normal(3 * Pn * M).reshape(Pn * M, 3)
    return pts


def _spread_bits21(v):
    """Spreads the low 21 bits of v so that two zero bits follow every bit (3-D Morton interleave)."""
    v = v.astype(np.uint64) & np.uint64(0x1FFFFF)
    v = (v | (v << np.uint64(32))) & np.uint64(0x1F00000000FFFF)
    v = (v | (v << np.uint64(16))) & np.uint64(0x1F0000FF0000FF)
    v = (v | (v << np.uint64(8))) & np.uint64(0x100F00F00F00F00F)
    v = (v | (v << np.uint64(4))) & np.uint64(0x10C30C30C30C30C3)
    v = (v | (v << np.uint64(2))) & np.uint64(0x1249249249249249)
    return v


def vet_preprocess_order(xyz, seed, block=256, radius=None):
    """The point order VET's scene preprocessing produces before the rasterizer ever sees a cloud:
    ReorderMorton64() followed by RandomBlockShuffle(256) (src/lib/data/SceneData.cpp:105-106 of the reference) and, with
    `radius` (the drop-out radius of every point), SortBlocksByRadius(256) (:108,1005-1018).
    Returns the permutation: 63-bit Morton order of the positions in their bounding box, then whole blocks of `block`
    consecutive points shuffled with the seeded generator, then every complete block sorted by radius."""
    xyz = np.asarray(xyz, dtype=np.float64)
    lo, hi = xyz.min(axis=0), xyz.max(axis=0)
    cell = np.floor((xyz - lo) / np.maximum(hi - lo, 1e-30) * ((1 << 21) - 1)).astype(np.uint64)
    code = _spread_bits21(cell[:, 0]) | (_spread_bits21(cell[:, 1]) << np.uint64(1)) | (_spread_bits21(cell[:, 2]) << np.uint64(2))
    order = np.argsort(code, kind="stable")
    n = order.shape[0]
    nb = (n + block - 1) // block
    keys = Stream(seed, "block_shuffle").u64(nb)
    block_perm = np.argsort(keys, kind="stable")
    idx = (block_perm[:, None] * block + np.arange(block)[None, :]).reshape(-1)
    idx = idx[idx < n]
    order = order[idx]
    if radius is not None:
        full = n // block * block
        r = np.asarray(radius)[order[:full]].reshape(-1, block)
        inner = np.argsort(r, axis=1, kind="stable") + (np.arange(n // block) * block)[:, None]
        order = np.concatenate([order[:full][inner.reshape(-1)], order[full:]])
    return order


def ordered_cloud(xyz, radius, seed, point_order):
    """Positions and radii in one of the orders a rasterizer meets:
    "vet_preprocess": what VET's loader hands over (Morton order, 256-point blocks shuffled, blocks sorted by radius);
    "generated": the generator's order (primitive by primitive, random inside);
    "grown": a cloud that grew during training: four fifths preprocessed, one fifth (a random subset) appended behind
    them in arbitrary order, as NeuralScene::AddNewPoints leaves it (src/lib/data/NeuralScene.cpp:1013; the reference
    does not sort again)."""
    if point_order == "generated":
        return xyz, radius
    if point_order == "vet_preprocess":
        o = vet_preprocess_order(xyz, seed, radius=radius)
        return xyz[o], radius[o]
    assert point_order == "grown", point_order
    n = xyz.shape[0]
    pick = np.argsort(Stream(seed, "grown").u64(n), kind="stable")
    old, new = pick[: n - n // 5], pick[n - n // 5:]
    o = old[vet_preprocess_order(xyz[old], seed, radius=radius[old])]
    o = np.concatenate([o, new])
    return xyz[o], radius[o]


def point_radii(seed, n, spread):
    """Drop-out radius per point: 1 cm, or with `spread` > 0 log-normal around it (VET computes it from the distance to
    the nearest neighbours, src/lib/data/SceneData.cpp:983-1001)."""
    if spread <= 0:
        return np.full(n, 0.01, dtype=np.float32)
    return (0.01 * np.exp(spread * Stream(seed, "radius").normal(n))).astype(np.float32)


def _descriptors(seed, N, channels=4, sigma=0.5):
    tex = (sigma * Stream(seed, "texture").normal(channels * N)).reshape(channels, N).astype(np.float32)
    conf = sigmoid(Stream(seed, "confidence").normal(N)).astype(np.float32)
    bg = Stream(seed, "background").uniform(channels).astype(np.float32)
    return tex, conf, bg


def config2(num_points=2_000_000, seed=1, w=1920, h=1080, num_layers=4, K=16, point_order="vet_preprocess",
            radius_spread=0.0) -> Scene:
    """SfM-like scene: points on 200 planes/spheres in a 10 m box, 1080p, fx=1000, 4 layers, K=16.

    point_order: see ordered_cloud. radius_spread: 0 gives every point the drop-out radius 1 cm; > 0 spreads the radii
    log-normally (for runs with drop_out_points_by_radius)."""
    prims = 200
    per = max(1, num_points // prims)
    N = prims * per
    pos = np.empty((N, 4), dtype=np.float32)
    xyz, radius = ordered_cloud(surface_points(seed, prims, per), point_radii(seed, N, radius_spread), seed, point_order)
    pos[:, :3] = xyz.astype(np.float32)
    pos[:, 3] = radius
    tex, conf, bg = _descriptors(seed, N)
    scale = w / 1920.0
    return Scene("config2_sfm", pos, tex, conf, bg, _identity_pose((0, 0, 4.5)),
                 _intrinsics(1000 * scale, 1000 * scale, w / 2, h / 2), [ViewSpec(w, h)], num_layers=num_layers,
                 max_list_length=K, seed=seed)


def config3(num_points=2_000_000, seed=1, **kw) -> Scene:
    """Config 2's scene with the backward pass: gradients to descriptors, confidence and xyz."""
    s = config2(num_points=num_points, seed=seed, **kw)
    s.name = "config3_sfm_fwd_bwd"
    s.params["need_point_gradient"] = 1
    return s


def _random_poses(seed, B, extent=4.0):
    st = Stream(seed, "poses")
    q = st.normal(4 * B).reshape(B, 4)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    c = (st.uniform(3 * B).reshape(B, 3) * 2.0 - 1.0) * extent
    poses = np.zeros((B, 8), dtype=np.float64)
    for b in range(B):
        x, y, z, w_ = q[b]
        R = np.array([
            [1 - 2 * (y * y + z * z), 2 * (x * y - w_ * z), 2 * (x * z + w_ * y)],
            [2 * (x * y + w_ * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w_ * x)],
            [2 * (x * z - w_ * y), 2 * (y * z + w_ * x), 1 - 2 * (x * x + y * y)],
        ])
        poses[b, :4] = q[b]
        poses[b, 4:7] = -R @ c[b]
    return poses


def config4(surface_points_n=4_000_000, sphere_points=500_000, seed=3, w=1920, h=1080, num_views=4, num_layers=4,
            K=16, point_order="vet_preprocess") -> Scene:
    """Surface points plus three nested environment spheres (r = 50/100/200 m), a batch of random views."""
    prims = 400
    per = max(1, surface_points_n // prims)
    surf = surface_points(seed, prims, per)
    shells = []
    for k, r in enumerate((50.0, 100.0, 200.0)):
        d = Stream(seed, f"sphere{k}").normal(3 * sphere_points).reshape(sphere_points, 3)
        d /= np.maximum(np.linalg.norm(d, axis=1, keepdims=True), 1e-12)
        shells.append(r * d)
    xyz = np.concatenate([surf] + shells, axis=0)
    N = xyz.shape[0]
    xyz, radius = ordered_cloud(xyz, point_radii(seed, N, 0.0), seed, point_order)
    pos = np.empty((N, 4), dtype=np.float32)
    pos[:, :3] = xyz.astype(np.float32)
    pos[:, 3] = radius
    tex, conf, bg = _descriptors(seed, N)
    scale = w / 1920.0
    views = [ViewSpec(w, h, image_index=b) for b in range(num_views)]
    s = Scene("config4_envspheres_batch", pos, tex, conf, bg, _random_poses(seed, num_views),
              _intrinsics(1000 * scale, 1000 * scale, w / 2, h / 2), views, num_layers=num_layers, max_list_length=K,
              seed=seed)
    s.params["need_point_gradient"] = 1
    return s


def config5(num_points=10_000_000, seed=4, w=1920, h=1080, num_layers=4, K=16, point_order="vet_preprocess") -> Scene:
    """Depth-complexity stress: a 1 m^3 cube of points filling the frustum."""
    N = num_points
    pos = np.empty((N, 4), dtype=np.float32)
    xyz = Stream(seed, "position").uniform(3 * N).reshape(N, 3) - 0.5
    xyz[:, 2] += 1.2
    xyz, radius = ordered_cloud(xyz, point_radii(seed, N, 0.0), seed, point_order)
    pos[:, :3] = xyz.astype(np.float32)
    pos[:, 3] = radius
    tex, conf, bg = _descriptors(seed, N)
    scale = w / 1920.0
    s = Scene("config5_depth_stress", pos, tex, conf, bg, _identity_pose((0, 0, 0)),
              _intrinsics(1000 * scale, 1000 * scale, w / 2, h / 2), [ViewSpec(w, h)], num_layers=num_layers,
              max_list_length=K, seed=seed)
    s.params["need_point_gradient"] = 1
    return s


def tiny_scene(num_points=300, w=24, h=16, num_layers=3, K=4, seed=7, channels=4, num_views=1) -> Scene:
    """A few hundred points on a small image: every pixel list is long enough to exercise sort and cut."""
    N = num_points
    st = Stream(seed, "tiny")
    pos = np.empty((N, 4), dtype=np.float32)
    pos[:, 0] = (st.uniform(N) * 2.4 - 1.2).astype(np.float32)
    pos[:, 1] = (st.uniform(N) * 1.6 - 0.8).astype(np.float32)
    pos[:, 2] = (st.uniform(N) * 2.0 - 0.5).astype(np.float32)
    pos[:, 3] = (0.05 + 1.0 * st.uniform(N)).astype(np.float32)  # splat radii of 0.2 .. 8 pixels at layer 0
    tex = (0.5 * st.normal(channels * N)).reshape(channels, N).astype(np.float32)
    conf = sigmoid(st.normal(N)).astype(np.float32)
    bg = st.uniform(channels).astype(np.float32)
    poses = _random_poses(seed, num_views, extent=0.2)
    poses[:, :4] = [0, 0, 0, 1]
    poses[:, 4:7] = np.array([[0.02 * b, -0.01 * b, 2.0 + 0.1 * b] for b in range(num_views)])
    views = [ViewSpec(w, h, image_index=b) for b in range(num_views)]
    return Scene("tiny", pos, tex, conf, bg, poses, _intrinsics(0.45 * w, 0.45 * w, w / 2.0, h / 2.0, 0.0), views,
                 num_layers=num_layers, max_list_length=K, seed=seed)


def cell_grid(xyz, cell_size):
    """Uniform grid of cells over the bounding box of the points, built the way VET does for point adding
    (UpdateCellStructureForPointOptim, src/lib/rendering/NeuralPointCloudCuda.cpp:95-147): the box grows by 0.01 on
    every side, ceil(extent / cell_size) slices per axis, cells numbered x fastest, then y, then z.
    Returns (bb_min [n,3] f32, bb_length [n,3] f32)."""
    lo = xyz.min(axis=0).astype(np.float32) - np.float32(0.01)
    hi = xyz.max(axis=0).astype(np.float32) + np.float32(0.01)
    size = np.float32(cell_size)
    slices = np.ceil((hi - lo) / size).astype(np.int64)
    zz, yy, xx = np.meshgrid(np.arange(slices[2]), np.arange(slices[1]), np.arange(slices[0]), indexing="ij")
    steps = np.stack([xx.ravel(), yy.ravel(), zz.ravel()], axis=1).astype(np.float32)
    bb_min = (lo[None, :] + steps * size).astype(np.float32)
    bb_length = np.full_like(bb_min, size)
    return np.ascontiguousarray(bb_min), np.ascontiguousarray(bb_length)


def error_image(seed, channels, h, w):
    """A per-pixel error image [channels,h,w] of either sign (the lifting takes absolute values): smooth blobs plus
    noise, like |target - output| of a half-trained scene with the sign kept."""
    st = Stream(seed, "error_image")
    y, x = np.mgrid[0:h, 0:w].astype(np.float32)
    img = np.empty((channels, h, w), dtype=np.float32)
    for c in range(channels):
        fx, fy, ph = st.uniform(3)
        blob = np.sin(x * np.float32(0.01 + 0.03 * fx) + np.float32(6.0 * ph)) * np.cos(y * np.float32(0.01 + 0.03 * fy))
        img[c] = (0.2 * blob + 0.05 * st.normal(h * w).reshape(h, w)).astype(np.float32)
    return np.ascontiguousarray(img)
