"""Writes tests/golden/config1_oracle.npz, tests/golden/config1_bilinear_oracle.npz and tests/golden/config1_fuzzy_oracle.npz
(the same scene in render_mode 3 and in render_mode 2, gradient samples included): the CPU oracle's result for BASELINE config 1 (20 000 points uniform in the
unit cube, 256x256, one layer, K=8, seed 0). The reference has no fixtures of its own and cannot run here, so this
vector records the oracle (after it has been pinned by tests/test_oracle_pinning.py) and serves as a regression pin for
the oracle and as a second, oracle-free check of the GPU path.

    python tests/golden/make_config1_fixture.py
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle_py  # noqa: E402
from vet_amd import synthetic  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    scene = synthetic.config1()
    f = oracle_py.forward(scene)
    counts = np.diff(f.offsets[0].astype(np.int64))
    assert counts.max() < 256
    total = int(f.offsets[0, -1])
    out = f.out[0][0]
    path = os.path.join(ROOT, "tests", "golden", "config1_oracle.npz")
    np.savez_compressed(
        path,
        counts=counts.astype(np.uint8),                      # per-pixel fragment counts, row-major 256x256
        fragments=f.fragments[0, :total],                    # every list fully sorted by (depth bits, point id)
        out_rows=out[:, 96:160:4, :].copy(),                 # 16 image rows of the blended features, all channels
        out_sha256=np.array(sha(out)),
        weight_sha256=np.array(sha(f.weight[0])),
        input_sha256=np.array([sha(scene.position), sha(scene.texture), sha(scene.confidence)]),
    )
    print("wrote", path, os.path.getsize(path), "bytes; fragments", total, "max list", counts.max())

    # the same scene in BILINEAR_BLEND; gradients for the upstream gradient scene.grad_out()
    from vet_amd import abi

    f = oracle_py.forward(scene, render_mode=abi.RENDER_BILINEAR_BLEND, need_point_gradient=1)
    g = oracle_py.backward(f, scene.grad_out())
    counts = np.diff(f.offsets[0].astype(np.int64))
    assert counts.max() < 256 and f.kept.max() < 256
    out = f.out[0][0]
    path = os.path.join(ROOT, "tests", "golden", "config1_bilinear_oracle.npz")
    np.savez_compressed(
        path,
        counts=counts.astype(np.uint8),
        kept=f.kept[0].astype(np.uint8),                     # fragments of every list that took part in the blend
        out_rows=out[:, 96:160:4, :].copy(),
        out_sha256=np.array(sha(out)),
        fragments_sha256=np.array(sha(f.fragments[0, :int(f.offsets[0, -1])])),
        weight_sha256=np.array(sha(f.weight[0])),
        grad_texture_rows=g["texture"][:, ::97].copy(),      # every 97th point: gradients are compared with a tolerance
        grad_confidence_rows=g["confidence"][::97].copy(),
        grad_points_rows=g["points"][::97].copy(),
        grad_background=g["background"].copy(),
        point_count_sha256=np.array(sha(g["point_count"])),
    )
    print("wrote", path, os.path.getsize(path), "bytes; fragments", int(f.offsets[0, -1]))

    # the same scene in FUZZY_BLEND with a depth range wide enough for buckets of several fragments
    f = oracle_py.forward(scene, render_mode=abi.RENDER_FUZZY_BLEND, depth_accept_blend=0.5, need_point_gradient=1)
    g = oracle_py.backward(f, scene.grad_out())
    out = f.out[0][0]
    path = os.path.join(ROOT, "tests", "golden", "config1_fuzzy_oracle.npz")
    np.savez_compressed(
        path,
        out_rows=out[:, 96:160:4, :].copy(),
        out_sha256=np.array(sha(out)),
        fragments_sha256=np.array(sha(f.fragments[0, :int(f.offsets[0, -1])])),
        weight_sha256=np.array(sha(f.weight[0])),
        grad_texture_rows=g["texture"][:, ::97].copy(),
        grad_confidence_rows=g["confidence"][::97].copy(),
        grad_points_rows=g["points"][::97].copy(),
        grad_background=g["background"].copy(),
        point_count_sha256=np.array(sha(g["point_count"])),
    )
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
