"""GPU parity on both sides of the limit at which the forward call changes how it scans the bin counts.

A view with up to 15 359 bins has their counts scanned, and the records that overflowed their bin's room filed, by one
launch that holds the whole scan in LDS; a view with more bins takes the hierarchical scan and a move kernel of its own.
The image sizes below put the bin count at 15 358, 15 359 (the last on the first path), 15 360 (the first on the second)
and 15 361; a part of the cloud is pulled together so that bins overflow and both ways of filing records run.
Counterpart of the scan between the counting and the collection pass, src/lib/rendering/PointRenderer.cu:799-813.
"""
import numpy as np
import pytest

from tests.test_gpu_wide_records import _compare
from vet_amd import synthetic
from vet_amd.rasterizer import make_params

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bins, layers, w, h", [(15358, 4, 1801, 1202), (15359, 3, 2566, 999), (15360, 3, 2035, 1265),
                                                (15361, 2, 2689, 1153)])
def test_bin_counts_around_the_single_launch_scan(bins, layers, w, h, rasterizer, oracle):
    print(f"[case] scan limit: {bins} bins, {w}x{h}, {layers} layers, clustered", flush=True)
    scene = synthetic.config2(num_points=200_000, seed=40 + layers, w=w, h=h, num_layers=layers, K=16)
    sel = np.arange(scene.num_points) % 2 == 0
    scene.position[sel, :2] *= np.float32(0.05)  # half of the cloud in a few bins: rooms overflow
    assert int(rasterizer.layout(scene).num_bins) == bins, "the bin table changed: pick new image sizes for this test"
    params = make_params(scene, need_point_gradient=1)
    res, ref = _compare(scene, params, rasterizer, oracle, bilinear=False)
    # the overflow path did run: some bin holds more records than any room has
    assert int(np.diff(res.offsets(0)).max()) > 0 and int(res.offsets(0)[-1]) > 4096
