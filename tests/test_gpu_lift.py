"""GPU parity of the error lifting (vetrast_lift_error) against the oracle: per-cell pixel counts bit-exact, per-cell
sums within 1e-6 relative (both sides add the float terms of a cell in double and round once; only the order of the
double additions differs)."""
import numpy as np
import pytest
import torch

from vet_amd import abi, synthetic
from vet_amd.synthetic import ViewSpec

pytestmark = pytest.mark.gpu

VALUE_TOL = 1e-6


def _run_both(rasterizer, oracle, mn, ln, view, poses, intr, img, border=abi.LIFT_BORDER_PIXELS, start=None,
              threads=16):
    n = len(mn)
    v0 = np.zeros(n, np.float32) if start is None else start[0]
    c0 = np.zeros(n, np.int32) if start is None else start[1]
    want_v, want_c = v0.copy(), c0.copy()
    oracle.lift_error(mn, ln, want_v, want_c, view, poses, intr, img, border_pixels=border, num_threads=threads)
    dev = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (mn, ln, v0, c0, poses, intr, img)]
    ws = rasterizer.lift_error(dev[0], dev[1], dev[2], dev[3], view, dev[4], dev[5], dev[6], border_pixels=border)
    torch.cuda.synchronize()
    assert rasterizer.lift_flags(ws) == 0
    queued = int(ws[abi.LIFT_QUEUE_LENGTH_OFFSET:abi.LIFT_QUEUE_LENGTH_OFFSET + 4].view(torch.int32).item())
    return dev[2].cpu().numpy(), dev[3].cpu().numpy(), want_v, want_c, queued


def _assert_parity(got_v, got_c, want_v, want_c):
    np.testing.assert_array_equal(got_c, want_c)
    scale = np.maximum(np.abs(want_v), 1e-3)
    err = float(np.max(np.abs(got_v.astype(np.float64) - want_v) / scale)) if len(want_v) else 0.0
    print(f"  cells hit {int((want_c > 0).sum())}, pixels added {int(want_c.sum())}, value max rel err {err:.2e}", flush=True)
    assert err <= VALUE_TOL


def _rotated_view_case(seed, W=160, H=120):
    rng = np.random.default_rng(seed)
    q = rng.normal(size=4) * [0.15, 0.15, 0.15, 1.0]
    q /= np.linalg.norm(q)
    poses = np.zeros((2, 8), np.float64)
    poses[:, 3] = 1
    poses[1, :4] = q
    poses[1, 4:7] = [0.1, -0.2, 3.0]
    intr = np.zeros((2, 13), np.float32)
    intr[0, :4] = [1, 1, 0, 0]
    intr[1, :5] = [130.0, 125.0, 80.5, 61.0, 0.7]
    ang = 0.2 * seed
    view = ViewSpec(W, H, image_index=1, camera_index=1, crop_transform=(0.9, 1.1, 4.0, -3.0, 0.02),
                    crop_rotation=(np.cos(ang), -np.sin(ang), np.sin(ang), np.cos(ang)))
    pts = rng.uniform(-1.5, 1.5, size=(50, 3))
    mn, ln = synthetic.cell_grid(pts, 0.3)
    ln = (ln * rng.uniform(0.5, 1.5, size=ln.shape)).astype(np.float32)
    return mn, ln, view, poses, intr, synthetic.error_image(seed, 3, H, W)


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("border", [0, 8, 32])
def test_small_image_rotated_crop(seed, border, rasterizer, oracle):
    print(f"[case] lift small seed={seed} border={border}", flush=True)
    mn, ln, view, poses, intr, img = _rotated_view_case(seed)
    got_v, got_c, want_v, want_c, _ = _run_both(rasterizer, oracle, mn, ln, view, poses, intr, img, border=border)
    assert want_c.sum() > 1000
    _assert_parity(got_v, got_c, want_v, want_c)


def test_accumulates_into_existing_values(rasterizer, oracle):
    print("[case] lift accumulate", flush=True)
    mn, ln, view, poses, intr, img = _rotated_view_case(3)
    rng = np.random.default_rng(0)
    start = (rng.uniform(0, 50, len(mn)).astype(np.float32), rng.integers(0, 9, len(mn)).astype(np.int32))
    got_v, got_c, want_v, want_c, _ = _run_both(rasterizer, oracle, mn, ln, view, poses, intr, img, border=8,
                                                start=(start[0].copy(), start[1].copy()))
    _assert_parity(got_v, got_c, want_v, want_c)
    untouched = want_c == start[1]
    assert untouched.any()
    np.testing.assert_array_equal(got_v[untouched], start[0][untouched])


def test_single_channel_and_one_cell(rasterizer, oracle):
    print("[case] lift one cell, one channel", flush=True)
    poses = np.zeros((1, 8), np.float64)
    poses[0, 3] = 1
    intr = np.zeros((1, 13), np.float32)
    intr[0, :4] = [100, 100, 64, 48]
    img = synthetic.error_image(4, 1, 96, 128)
    mn = np.array([[-0.5, -0.25, 2.0]], np.float32)
    ln = np.array([[1.0, 0.75, 1.0]], np.float32)
    got_v, got_c, want_v, want_c, _ = _run_both(rasterizer, oracle, mn, ln, ViewSpec(128, 96), poses, intr, img, border=0)
    assert got_c[0] == 50 * 36  # hand-computed rectangle of the front face
    _assert_parity(got_v, got_c, want_v, want_c)


def test_config3_grid_full_size(rasterizer, oracle):
    """The 2 M point scene's grid at 0.25 m (146 k cells) under its 1080p camera, which stands inside the grid: cells
    next to the camera cover up to half the image and go through the shared path."""
    print("[case] lift config 3 grid, 1080p", flush=True)
    scene = synthetic.config3(num_points=200_000)
    mn, ln = synthetic.cell_grid(scene.position[:, :3], 0.25)
    img = synthetic.error_image(5, 3, 1080, 1920)
    got_v, got_c, want_v, want_c, queued = _run_both(rasterizer, oracle, mn, ln, scene.views[0], scene.poses_se3,
                                                     scene.intrinsics, img)
    print(f"  cells {len(mn)}, queued for the shared path {queued}", flush=True)
    assert queued > 100 and want_c.max() > 500_000
    _assert_parity(got_v, got_c, want_v, want_c)
    # every pixel of a cell adds a non-negative term: a cell with pixels has a positive value
    assert np.all((got_v > 0) == (got_c > 0))


def test_constant_image_gives_channels_times_count(rasterizer):
    """No oracle: with |error| = 0.5 in each of 3 channels a cell's value is 1.5 * its count exactly."""
    scene = synthetic.config3(num_points=200_000)
    mn, ln = synthetic.cell_grid(scene.position[:, :3], 0.5)
    img = torch.full((3, 1080, 1920), -0.5, device="cuda")
    val = torch.zeros(len(mn), device="cuda")
    cnt = torch.zeros(len(mn), dtype=torch.int32, device="cuda")
    rasterizer.lift_error(torch.from_numpy(mn).cuda(), torch.from_numpy(ln).cuda(), val, cnt, scene.views[0],
                          torch.from_numpy(scene.poses_se3).cuda(), torch.from_numpy(scene.intrinsics).cuda(), img)
    torch.cuda.synchronize()
    assert int(cnt.sum()) > 1_000_000
    np.testing.assert_allclose(val.cpu().numpy(), 1.5 * cnt.cpu().numpy().astype(np.float64), rtol=1e-6)
    assert int(cnt.max()) <= (1920 - 64) * (1080 - 64)


def test_argument_checks(rasterizer):
    scene = synthetic.tiny_scene()
    mn, ln = synthetic.cell_grid(scene.position[:, :3], 0.5)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    val = torch.zeros(len(mn), device="cuda")
    cnt = torch.zeros(len(mn), dtype=torch.int32, device="cuda")
    img = torch.zeros((3, 16, 24), device="cuda")
    args = (dev(mn), dev(ln), val, cnt, scene.views[0], dev(scene.poses_se3), dev(scene.intrinsics), img)
    with pytest.raises(abi.VetrastError) as e:
        rasterizer.lift_error(*args, workspace=torch.empty(256, dtype=torch.uint8, device="cuda"))
    assert e.value.status == abi.ERR_WORKSPACE_SMALL
    with pytest.raises(abi.VetrastError) as e:
        rasterizer.lift_error(*args, border_pixels=-1)
    assert e.value.status == abi.ERR_INVALID_ARG
    bad_view = ViewSpec(24, 16, image_index=5)
    with pytest.raises(abi.VetrastError):
        rasterizer.lift_error(args[0], args[1], val, cnt, bad_view, args[5], args[6], img)
    # a border wider than the image: nothing is added, nothing is read
    rasterizer.lift_error(*args, border_pixels=32)
    torch.cuda.synchronize()
    assert int(cnt.sum()) == 0


def test_lift_replays_from_a_hip_graph(rasterizer, oracle):
    """vetrast_lift_error only launches kernels (no memsets, allocations or host reads): captured in a graph and
    replayed, each replay adds the same counts and sums again; eager work (an optimiser step) runs between replays."""
    import ctypes as C

    mn, ln, view, poses, intr, img = _rotated_view_case(7)
    n = len(mn)
    want_v, want_c = np.zeros(n, np.float32), np.zeros(n, np.int32)
    oracle.lift_error(mn, ln, want_v, want_c, view, poses, intr, img, border_pixels=8)
    dev = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (mn, ln, poses, intr, img)]
    val = torch.zeros(n, device="cuda")
    cnt = torch.zeros(n, dtype=torch.int32, device="cuda")
    ws = rasterizer.lift_error(dev[0], dev[1], val, cnt, view, dev[2], dev[3], dev[4], border_pixels=8)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(cnt.cpu().numpy(), want_c)
    p = torch.linspace(-1, 1, 5000, device="cuda")
    g = torch.cos(torch.arange(5000, device="cuda", dtype=torch.float32))
    m, v = torch.zeros_like(p), torch.zeros_like(p)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rasterizer.lift_error(dev[0], dev[1], val, cnt, view, dev[2], dev[3], dev[4], border_pixels=8, workspace=ws)
    for replay in range(3):
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(cnt.cpu().numpy(), (replay + 2) * want_c)
        np.testing.assert_allclose(val.cpu().numpy(), (replay + 2) * want_v.astype(np.float64), rtol=2e-6)
        rasterizer.adam_step(p, g, m, v, replay + 1, 1e-2)  # eager work between the replays
        torch.cuda.synchronize()
    assert torch.isfinite(p).all()
