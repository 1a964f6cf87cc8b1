"""Host-side checks of bench.py and __graft_entry__.py that need no GPU: the byte model is the one the design states,
a run on several GPUs is refused with a message, a run without a GPU fails loudly (there is no CPU path in the
product), and the entry file exposes build() and smoke()."""
import importlib.util
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _load(name):
    spec = importlib.util.spec_from_file_location(name, os.path.join(ROOT, name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_byte_model_adds_up_to_the_stated_totals():
    """B_fwd = 32N + 36P + 24F + 28F', B_bwd = 32P + 116F' + 40N for four channels; config 3's measured counts give
    the 866.6 MB per frame the bench line reports."""
    bench = _load("bench")
    N, P, F, Fk = 2_000_000, 2_754_000, 3_808_194, 3_082_581
    fwd, bwd = bench.algorithmic_bytes(N, P, F, Fk, 4)
    assert sum(fwd.values()) == 32 * N + 36 * P + 24 * F + 28 * Fk
    assert sum(bwd.values()) == 32 * P + 116 * Fk + 40 * N
    assert abs((sum(fwd.values()) + sum(bwd.values())) / 1e6 - 866.56) < 0.01
    # every term is attributed to a kernel scope the library reports
    from vet_amd import abi
    assert set(fwd) | set(bwd) <= set(abi.SCOPE_NAMES)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
    env = dict(os.environ, WORLD_SIZE="4")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode != 0 and "ONE GPU" in r.stderr


def test_without_a_gpu_the_bench_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "needs a GPU" in r.stderr and r.stdout.strip() == ""


def test_entry_file_has_build_and_smoke():
    entry = _load("__graft_entry__")
    assert callable(entry.build) and callable(entry.smoke)
