"""VET's scene checkpoints are libtorch module archives (torch::save of the modules that own the tensors,
src/lib/data/NeuralScene.cpp:407-431). The shim reads and writes the entries the rasterizer needs by name; PyTorch's own
TorchScript reader and writer of the same archive format serve as the independent check (what libtorch's torch::save
writes for a module is what torch.jit.load opens, and the other way round). Host code: runs without a GPU."""
import numpy as np
import torch

from vet_amd import synthetic, torch_ops


def _scene_tensors():
    s = synthetic.tiny_scene(num_points=500, num_views=3, seed=91)
    rng = np.random.default_rng(0)
    return {
        "t_position": torch.from_numpy(s.position),
        "t_index": torch.arange(500, dtype=torch.int32).reshape(-1, 1),
        "texture": torch.from_numpy(rng.normal(size=(4, 500)).astype(np.float32)),
        "background_color": torch.from_numpy(rng.normal(size=4).astype(np.float32)),
        "confidence_value_of_point": torch.from_numpy(rng.normal(size=(1, 500)).astype(np.float32)),
        "tangent_poses": torch.zeros((3, 6), dtype=torch.float64),
        "poses_se3": torch.from_numpy(s.poses_se3),
        "intrinsics": torch.from_numpy(s.intrinsics),
    }


def test_round_trip_through_the_shim(tmp_path):
    want = _scene_tensors()
    prefix = str(tmp_path / "scene_test_")
    torch_ops.save_scene_checkpoint(prefix, **want)
    got = torch_ops.load_scene_checkpoint(prefix)
    # t_original_color is always written (the reference's module registers it): zeros when none was given
    assert sorted(got) == sorted(list(want) + ["t_original_color"])
    assert got["t_original_color"].shape == (500, 4) and not got["t_original_color"].any()
    for k, v in want.items():
        assert got[k].dtype == v.dtype and torch.equal(got[k], v), k
    # only the files whose tensors were given are written; missing files leave their tensors out
    prefix2 = str(tmp_path / "scene_partial_")
    torch_ops.save_scene_checkpoint(prefix2, intrinsics=want["intrinsics"])
    assert sorted(torch_ops.load_scene_checkpoint(prefix2)) == ["intrinsics"]


def test_files_written_by_the_shim_open_as_module_archives(tmp_path):
    want = _scene_tensors()
    prefix = str(tmp_path / "scene_a_")
    torch_ops.save_scene_checkpoint(prefix, **want)
    points = torch.jit.load(prefix + "points.pth")
    assert torch.equal(dict(points.named_parameters())["t_position"], want["t_position"])
    assert torch.equal(dict(points.named_buffers())["t_index"], want["t_index"])
    texture = dict(torch.jit.load(prefix + "texture.pth").named_parameters())
    assert sorted(texture) == ["background_color", "confidence_value_of_point", "texture"]
    assert torch.equal(texture["texture"], want["texture"])
    poses = torch.jit.load(prefix + "poses.pth")
    assert torch.equal(dict(poses.named_buffers())["poses_se3"], want["poses_se3"])
    assert torch.equal(dict(poses.named_parameters())["tangent_poses"], want["tangent_poses"])


class _Points(torch.nn.Module):
    """Registers its tensors under the names NeuralPointCloudCudaImpl uses (NeuralPointCloudCuda.cpp:71-73)."""

    def __init__(self, position, index):
        super().__init__()
        self.t_position = torch.nn.Parameter(position)
        self.register_buffer("t_index", index)
        self.register_buffer("t_original_color", torch.zeros(4, 3))  # an entry the rasterizer does not read

    def forward(self):
        return self.t_position


class _Texture(torch.nn.Module):
    def __init__(self, t):
        super().__init__()
        self.texture = torch.nn.Parameter(t["texture"])
        self.background_color = torch.nn.Parameter(t["background_color"])
        self.confidence_value_of_point = torch.nn.Parameter(t["confidence_value_of_point"])

    def forward(self):
        return self.texture


def test_module_archives_written_by_pytorch_load_through_the_shim(tmp_path):
    want = _scene_tensors()
    prefix = str(tmp_path / "scene_b_")
    torch.jit.script(_Points(want["t_position"], want["t_index"])).save(prefix + "points.pth")
    torch.jit.script(_Texture(want)).save(prefix + "texture.pth")
    got = torch_ops.load_scene_checkpoint(prefix)
    assert sorted(got) == ["background_color", "confidence_value_of_point", "t_index", "t_original_color", "t_position",
                           "texture"]
    for k in got:
        if k != "t_original_color":
            assert torch.equal(got[k], want[k]), k


class _StrictPoints(torch.nn.Module):
    """What torch::load of the reference's NeuralPointCloudCudaImpl demands of points.pth: Module::load reads every name
    the module registered and throws on a missing one (src/lib/data/NeuralScene.cpp:349). load_state_dict(strict=True)
    is the same rule on the Python side."""

    def __init__(self, n, with_normal, with_cells, cells=0):
        super().__init__()
        self.t_position = torch.nn.Parameter(torch.zeros(n, 4))                      # NeuralPointCloudCuda.cpp:71
        self.register_buffer("t_index", torch.zeros(n, 1, dtype=torch.int32))         # :72
        self.register_buffer("t_original_color", torch.zeros(n, 4))                   # :73
        if with_normal:
            self.register_buffer("t_normal", torch.zeros(n, 1, dtype=torch.int32))    # :53
        if with_cells:                                                                # :84-87
            self.register_buffer("t_cell_bb_min", torch.zeros(cells, 3))
            self.register_buffer("t_cell_bb_length", torch.zeros(cells, 3))
            self.register_buffer("t_cell_value", torch.zeros(cells, 1))
            self.register_buffer("t_cell_access_count", torch.zeros(cells, 1, dtype=torch.int32))


def _strict_read(path, module):
    archive = torch.jit.load(path)
    state = {k: v for k, v in list(archive.named_parameters()) + list(archive.named_buffers())}
    module.load_state_dict(state, strict=True)  # raises on a missing or an unexpected name
    return state


def test_points_file_holds_every_tensor_the_reference_module_registers(tmp_path):
    want = _scene_tensors()
    # 1. the rasterizer's tensors only, no index: identity index and zero colours are written
    prefix = str(tmp_path / "scene_c_")
    torch_ops.save_scene_checkpoint(prefix, t_position=want["t_position"])
    state = _strict_read(prefix + "points.pth", _StrictPoints(500, False, False))
    assert torch.equal(state["t_index"], torch.arange(500, dtype=torch.int32).reshape(-1, 1))
    assert state["t_original_color"].shape == (500, 4) and state["t_original_color"].dtype == torch.float32
    # 2. a cloud with colours, normals and the cell grid: carried through load and save unchanged
    rng = np.random.default_rng(3)
    extra = {
        "t_original_color": torch.from_numpy(rng.uniform(size=(500, 4)).astype(np.float32)),
        "t_normal": torch.from_numpy(rng.integers(0, 1 << 30, size=(500, 1)).astype(np.int32)),
        "t_cell_bb_min": torch.from_numpy(rng.normal(size=(7, 3)).astype(np.float32)),
        "t_cell_bb_length": torch.from_numpy(rng.uniform(size=(7, 3)).astype(np.float32)),
        "t_cell_value": torch.from_numpy(rng.uniform(size=(7, 1)).astype(np.float32)),
        "t_cell_access_count": torch.from_numpy(rng.integers(0, 9, size=(7, 1)).astype(np.int32)),
    }
    prefix = str(tmp_path / "scene_d_")
    torch_ops.save_scene_checkpoint(prefix, t_position=want["t_position"], t_index=want["t_index"], **extra)
    state = _strict_read(prefix + "points.pth", _StrictPoints(500, True, True, cells=7))
    loaded = torch_ops.load_scene_checkpoint(prefix)
    for k, v in extra.items():
        assert torch.equal(state[k], v) and torch.equal(loaded[k], v), k
    # ... and once more through the shim: load, save, strict read
    prefix2 = str(tmp_path / "scene_e_")
    torch_ops.save_scene_checkpoint(prefix2, **loaded)
    state2 = _strict_read(prefix2 + "points.pth", _StrictPoints(500, True, True, cells=7))
    for k in state:
        assert torch.equal(state2[k], state[k]), k
    # a module without normals refuses the file that has them, as Module::load would
    import pytest

    with pytest.raises(RuntimeError):
        _strict_read(prefix2 + "points.pth", _StrictPoints(500, False, True, cells=7))
