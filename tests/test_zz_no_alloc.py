"""vetrast_lift_error_static, the entry point that allocates nothing (its scratch is an array inside the library),
against vetrast_lift_error with a caller-owned workspace: per-cell pixel counts bit-equal, per-cell sums within 1e-6
relative (a cell's float terms are summed in double and rounded once on both paths; for cells on the shared path only
the order of the double additions differs between two runs). Two calls in a row share the one scratch array, the second
on a smaller grid, so stale queue entries, sums and prefix sums of the first call would show."""
import gc

import numpy as np
import pytest
import torch

from vet_amd import abi, synthetic

pytestmark = pytest.mark.gpu

VALUE_TOL = 1e-6


def _case(num_points, cell_size, seed, width=1920, height=1080):
    scene = synthetic.config3(num_points=num_points)
    mn, ln = synthetic.cell_grid(scene.position[:, :3], cell_size)
    img = synthetic.error_image(seed, 3, height, width)
    return scene, mn, ln, img


def _both(rasterizer, scene, mn, ln, img):
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    d_mn, d_ln, d_pose, d_intr, d_img = dev(mn), dev(ln), dev(scene.poses_se3), dev(scene.intrinsics), dev(img)
    n = len(mn)
    rng = np.random.default_rng(n)
    v0 = rng.uniform(0, 5, n).astype(np.float32)  # both paths accumulate into existing values
    c0 = rng.integers(0, 4, n).astype(np.int32)
    want_v, want_c = dev(v0), dev(c0)
    ws = rasterizer.lift_error(d_mn, d_ln, want_v, want_c, scene.views[0], d_pose, d_intr, d_img)
    got_v, got_c = dev(v0), dev(c0)
    # Nothing is allocated: neither through torch's caching allocator nor straight from the device (free bytes as
    # hipMemGetInfo reports them, which a hipMalloc inside the library would lower).
    # (Tensors of earlier tests that the garbage collector frees meanwhile lower the bytes in use, so the check is on
    # the allocator's count of allocations, which only ever goes up.)
    gc.collect()
    torch.cuda.synchronize()
    allocations = lambda: torch.cuda.memory_stats()["allocation.all.allocated"]
    before, free_before = allocations(), torch.cuda.mem_get_info()[0]
    ret = rasterizer.lift_error(d_mn, d_ln, got_v, got_c, scene.views[0], d_pose, d_intr, d_img, static_scratch=True)
    torch.cuda.synchronize()
    assert ret is None and allocations() == before, "a tensor was allocated during the call"
    assert torch.cuda.mem_get_info()[0] >= free_before, "the device lost free memory during the call"
    queued = int(ws[abi.LIFT_QUEUE_LENGTH_OFFSET:abi.LIFT_QUEUE_LENGTH_OFFSET + 4].view(torch.int32).item())
    return got_v.cpu().numpy(), got_c.cpu().numpy(), want_v.cpu().numpy(), want_c.cpu().numpy(), c0, queued


def _assert_same(got_v, got_c, want_v, want_c):
    np.testing.assert_array_equal(got_c, want_c)
    scale = np.maximum(np.abs(want_v.astype(np.float64)), 1e-3)
    err = float(np.max(np.abs(got_v.astype(np.float64) - want_v) / scale))
    print(f"  value max rel err {err:.2e}", flush=True)
    assert err <= VALUE_TOL


def test_static_scratch_matches_workspace_twice_in_a_row(rasterizer):
    # first call: the 0.25 m grid of the 2 M point scene (146 k cells, several thousand on the shared path)
    print("[case] lift_error_static, 0.25 m grid", flush=True)
    scene, mn, ln, img = _case(200_000, 0.25, 5)
    got_v, got_c, want_v, want_c, c0, queued = _both(rasterizer, scene, mn, ln, img)
    print(f"  cells {len(mn)}, queued {queued}, pixels added {int((want_c - c0).sum())}", flush=True)
    assert len(mn) <= abi.LIFT_STATIC_MAX_CELLS and queued > 100 and (want_c - c0).sum() > 10_000_000
    _assert_same(got_v, got_c, want_v, want_c)
    # second call, right behind it on the same stream: a smaller grid (0.5 m, 19 k cells, fewer queued cells) and
    # another image, through the same scratch array
    print("[case] lift_error_static, 0.5 m grid right after", flush=True)
    scene2, mn2, ln2, img2 = _case(200_000, 0.5, 6)
    got_v, got_c, want_v, want_c, c0, queued2 = _both(rasterizer, scene2, mn2, ln2, img2)
    print(f"  cells {len(mn2)}, queued {queued2}, pixels added {int((want_c - c0).sum())}", flush=True)
    assert len(mn2) < len(mn) and 0 < queued2 < queued
    _assert_same(got_v, got_c, want_v, want_c)


def test_static_scratch_refuses_grids_beyond_its_maximum(rasterizer):
    n = abi.LIFT_STATIC_MAX_CELLS + 1
    scene = synthetic.tiny_scene()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    mn = torch.zeros((n, 3), device="cuda")
    ln = torch.ones((n, 3), device="cuda")
    val = torch.zeros(n, device="cuda")
    cnt = torch.zeros(n, dtype=torch.int32, device="cuda")
    img = torch.zeros((3, 64, 64), device="cuda")
    with pytest.raises(abi.VetrastError) as e:
        rasterizer.lift_error(mn, ln, val, cnt, scene.views[0], dev(scene.poses_se3), dev(scene.intrinsics), img,
                              static_scratch=True)
    assert e.value.status == abi.ERR_TOO_LARGE
    torch.cuda.synchronize()
    assert int(cnt.sum()) == 0
