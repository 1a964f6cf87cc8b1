"""The point order VET's preprocessing produces (Morton order, then shuffled 256-point blocks) as the shim computes it:
against an independent bit-by-bit interleave, against the numpy generator of the benchmark scenes, and its block
structure. Runs on the CPU (the function is host code)."""
import numpy as np
import torch

from vet_amd import synthetic, torch_ops


def _morton_by_hand(xyz):
    """63-bit Morton code with plain Python integers: bit k of axis a goes to bit 3k + a."""
    lo, hi = xyz.min(axis=0), xyz.max(axis=0)
    cells = np.floor((xyz - lo) / np.maximum(hi - lo, 1e-30) * ((1 << 21) - 1)).astype(np.int64)
    codes = []
    for c in cells:
        code = 0
        for a in range(3):
            for k in range(21):
                code |= ((int(c[a]) >> k) & 1) << (3 * k + a)
        codes.append(code)
    return codes


def test_single_block_is_the_morton_order():
    rng = np.random.default_rng(0)
    xyz = rng.uniform(-3, 5, size=(2000, 3))
    order = torch_ops.morton_block_shuffle_order(torch.from_numpy(xyz), block=4096, seed=7).numpy()
    assert sorted(order.tolist()) == list(range(2000))
    codes = _morton_by_hand(xyz)
    sorted_codes = [codes[i] for i in order]
    assert all(a <= b for a, b in zip(sorted_codes, sorted_codes[1:]))
    # the generator of the benchmark scenes computes the same order (one block: nothing to shuffle)
    np.testing.assert_array_equal(order, synthetic.vet_preprocess_order(xyz, seed=3, block=4096))
    # float32 [N,4] input (the rasterizer's position tensor) works as well
    pos4 = torch.zeros((2000, 4), dtype=torch.float32)
    pos4[:, :3] = torch.from_numpy(xyz).float()
    order4 = torch_ops.morton_block_shuffle_order(pos4, block=4096).numpy()
    codes4 = _morton_by_hand(pos4[:, :3].double().numpy())
    assert all(codes4[a] <= codes4[b] for a, b in zip(order4, order4[1:]))


def test_blocks_are_shuffled_whole():
    rng = np.random.default_rng(1)
    xyz = rng.normal(size=(10_000, 3))
    morton = torch_ops.morton_block_shuffle_order(torch.from_numpy(xyz), block=1 << 20).numpy()
    a = torch_ops.morton_block_shuffle_order(torch.from_numpy(xyz), block=256, seed=1).numpy()
    b = torch_ops.morton_block_shuffle_order(torch.from_numpy(xyz), block=256, seed=2).numpy()
    assert sorted(a.tolist()) == list(range(10_000)) and sorted(b.tolist()) == list(range(10_000))
    assert not np.array_equal(a, b) and not np.array_equal(a, morton)
    np.testing.assert_array_equal(a, torch_ops.morton_block_shuffle_order(torch.from_numpy(xyz), block=256, seed=1).numpy())
    # every run of the result that came from one block is a stretch of the Morton order
    where = np.empty(10_000, np.int64)
    where[morton] = np.arange(10_000)
    pos = where[a]
    blocks = pos // 256
    starts = np.flatnonzero(np.diff(blocks) != 0) + 1
    for seg in np.split(pos, starts):
        assert np.all(np.diff(seg) == 1) and seg[0] % 256 == 0
    assert len(starts) + 1 == (10_000 + 255) // 256
    assert torch_ops.morton_block_shuffle_order(torch.zeros((0, 3))).numel() == 0


def test_blocks_sorted_by_radius():
    """SceneData::SortBlocksByRadius(256) (src/lib/data/SceneData.cpp:1005-1018): every complete block sorted by radius,
    the incomplete tail left alone, nothing moves between blocks."""
    rng = np.random.default_rng(5)
    radius = rng.uniform(0.001, 0.1, size=1000).astype(np.float32)
    order = torch_ops.sort_blocks_by_radius_order(torch.from_numpy(radius), block=256).numpy()
    assert sorted(order.tolist()) == list(range(1000))
    for b in range(3):  # 1000 // 256 complete blocks
        seg = order[256 * b:256 * (b + 1)]
        assert seg.min() >= 256 * b and seg.max() < 256 * (b + 1)
        assert np.all(np.diff(radius[seg]) >= 0)
        np.testing.assert_array_equal(seg, 256 * b + np.argsort(radius[256 * b:256 * (b + 1)], kind="stable"))
    np.testing.assert_array_equal(order[768:], np.arange(768, 1000))


def test_scene_preprocess_order_is_the_three_steps_in_a_row():
    rng = np.random.default_rng(6)
    pos = np.zeros((5000, 4), np.float32)
    pos[:, :3] = rng.normal(size=(5000, 3))
    pos[:, 3] = rng.uniform(0.001, 0.05, size=5000)
    t = torch.from_numpy(pos)
    first = torch_ops.morton_block_shuffle_order(t, block=256, seed=9).numpy()
    second = torch_ops.sort_blocks_by_radius_order(torch.from_numpy(pos[first, 3]), block=256).numpy()
    got = torch_ops.scene_preprocess_order(t, block=256, seed=9).numpy()
    np.testing.assert_array_equal(got, first[second])
    # every block of the result is one block of the shuffled Morton order, radius ascending
    for b in range(5000 // 256):
        assert set(got[256 * b:256 * (b + 1)].tolist()) == set(first[256 * b:256 * (b + 1)].tolist())
        assert np.all(np.diff(pos[got[256 * b:256 * (b + 1)], 3]) >= 0)
    # the generator of the benchmark scenes sorts its blocks the same way (its block shuffle draws from another
    # generator, so only the structure can be compared)
    own = synthetic.vet_preprocess_order(pos[:, :3], seed=9, block=256, radius=pos[:, 3])
    plain = synthetic.vet_preprocess_order(pos[:, :3], seed=9, block=256)
    for b in range(5000 // 256):
        assert set(own[256 * b:256 * (b + 1)].tolist()) == set(plain[256 * b:256 * (b + 1)].tolist())
        assert np.all(np.diff(pos[own[256 * b:256 * (b + 1)], 3]) >= 0)
    np.testing.assert_array_equal(own[5000 // 256 * 256:], plain[5000 // 256 * 256:])


def test_grown_cloud_order():
    """A cloud that grew during training (NeuralScene::AddNewPoints appends, src/lib/data/NeuralScene.cpp:1013): the
    preprocessed part keeps its order, the appended fifth is in arbitrary order."""
    s = synthetic.config2(num_points=20_000, point_order="grown")
    ordered = synthetic.config2(num_points=20_000, point_order="vet_preprocess")
    assert s.num_points == ordered.num_points == 20_000
    # the same set of points
    a = np.sort(s.position.view([("", np.float32)] * 4).ravel())
    b = np.sort(ordered.position.view([("", np.float32)] * 4).ravel())
    assert np.array_equal(a, b)
    assert not np.array_equal(s.position, ordered.position)


def test_processing_order_on_device_is_a_permutation_with_compact_blocks():
    """The order the shim builds for the binning pass (tensor operations, here on the CPU device): every point once,
    and a 256-point block is a run of the Morton curve, i.e. small in space (random blocks span the scene)."""
    import torch

    from vet_amd import torch_ops

    scene = synthetic.config2(num_points=60_000, point_order="generated")
    xyz = scene.position[:, :3]
    order = torch_ops.processing_order_on_device(torch.from_numpy(scene.position), 256, 3)
    assert order.dtype == torch.int32 and tuple(order.shape) == (scene.num_points,)
    o = order.numpy().astype(np.int64)
    np.testing.assert_array_equal(np.sort(o), np.arange(scene.num_points))

    def mean_block_diagonal(perm):
        n = len(perm) // 256 * 256
        b = xyz[perm[:n]].reshape(-1, 256, 3)
        return float(np.linalg.norm(b.max(axis=1) - b.min(axis=1), axis=1).mean())

    assert mean_block_diagonal(o) * 3 < mean_block_diagonal(np.random.default_rng(0).permutation(scene.num_points))
    # deterministic for a seed, another seed shuffles the blocks differently
    again = torch_ops.processing_order_on_device(torch.from_numpy(scene.position), 256, 3)
    other = torch_ops.processing_order_on_device(torch.from_numpy(scene.position), 256, 4)
    assert torch.equal(order, again) and not torch.equal(order, other)
    assert torch_ops.processing_order_on_device(torch.zeros((0, 4))).numel() == 0
