"""BASELINE config 1 against the committed golden vector (tests/golden/config1_oracle.npz, written by
tests/golden/make_config1_fixture.py): the oracle must still reproduce it, and the GPU path must match it without the
oracle in the loop."""
import hashlib
import os

import numpy as np
import pytest

from tests.helpers import kept_mask
from vet_amd import synthetic

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1_oracle.npz")


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.fixture(scope="module")
def golden():
    return np.load(FIXTURE, allow_pickle=False)


@pytest.fixture(scope="module")
def scene(golden):
    s = synthetic.config1()
    got = [sha(s.position), sha(s.texture), sha(s.confidence)]
    assert got == list(golden["input_sha256"]), "the seeded generator no longer produces the fixture's inputs"
    return s


def test_oracle_reproduces_the_golden_vector(oracle, scene, golden):
    f = oracle.forward(scene)
    counts = np.diff(f.offsets[0].astype(np.int64))
    np.testing.assert_array_equal(counts, golden["counts"].astype(np.int64))
    np.testing.assert_array_equal(f.fragments[0, :len(golden["fragments"])], golden["fragments"])
    np.testing.assert_array_equal(f.out[0][0][:, 96:160:4, :], golden["out_rows"])
    assert sha(f.out[0][0]) == str(golden["out_sha256"])
    assert sha(f.weight[0]) == str(golden["weight_sha256"])


@pytest.mark.gpu
def test_gpu_reproduces_the_golden_vector(rasterizer, scene, golden):
    import torch

    from vet_amd.rasterizer import DeviceScene

    res = rasterizer.forward(DeviceScene(scene), save_for_backward=False)
    torch.cuda.synchronize()
    off = res.offsets(0)
    np.testing.assert_array_equal(np.diff(off), golden["counts"].astype(np.int64))
    keep = kept_mask(off, scene.max_list_length)
    np.testing.assert_array_equal(res.fragments(0)[keep], golden["fragments"][keep])
    out = res.out[0].cpu().numpy()[0]
    np.testing.assert_array_equal(out[:, 96:160:4, :], golden["out_rows"])
    assert sha(out) == str(golden["out_sha256"])
    assert sha(res.weight(0)) == str(golden["weight_sha256"])
