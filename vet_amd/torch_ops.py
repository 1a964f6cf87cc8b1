"""Loader of the libtorch shim (vet_amd/lib/vetrast_torch.so) for Python callers and tests."""
import importlib.util
import os

import torch  # noqa: F401  (libtorch must be loaded before the extension)

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "vetrast_torch.so")
_mod = None


def load():
    global _mod
    if _mod is None:
        if not os.path.exists(_PATH):
            raise OSError(f"{_PATH} is missing: build it with `python -m vet_amd.build`")
        spec = importlib.util.spec_from_file_location("vetrast_torch", _PATH)
        _mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_mod)
    return _mod


def blend_point_cloud(texture, background_color, points, pose_tangents, intrinsics, confidence, poses_se3, t_index,
                      views, num_layers, train=False, environment=None, **params):
    """BlendPointCloud of the reference (src/lib/rendering/PointRenderer.h:53) on tensors; differentiable.

    views: list of (w, h, image_index, camera_index, camera_model, crop fx,fy,cx,cy,s, rot r00,r01,r10,r11).
    Returns L tensors [B,C,h_l,w_l], then L masks if output_background_mask (through the render module, i.e. with
    super_sampling, cat_masks_to_color, add_depth_to_network or an environment: the images with their extra channels,
    then the masks).
    environment: a callable standing in for the environment map of PointRenderModuleImpl::forward
    (src/lib/rendering/RenderModule.cpp:129-202): it gets layers[l][b] = the [1,1,h_l,w_l] per-pixel transmittance left
    behind the points and returns L tensors [B,C_env,h_l,w_l]; they are added to the images (masked with
    no_envmap_at_points, the default) or appended as channels (cat_env_to_color). Needs output_background_mask.
    """
    if t_index is None:
        t_index = torch.empty(0, dtype=torch.int32, device=points.device)
    return load().blend_point_cloud(texture, background_color, points, pose_tangents, intrinsics, confidence, poses_se3,
                                    t_index, [list(map(float, v)) for v in views], int(num_layers), bool(train),
                                    {k: float(v) for k, v in params.items()}, environment)


def adapter_selftest(texture, background_color, points, pose_tangents, intrinsics, confidence, poses_se3, views,
                     num_layers, render_mode=1, max_list_length=-1, output_background_mask=False):
    """Renders through vet_amd/torch_ext/vet_adapter.h (the templates that turn the reference's NeuralScene,
    ReducedImageInfo, RenderParams and NeuralRenderInfo into the shim's types), instantiated with stand-ins that have the
    reference's member names. Same result as blend_point_cloud(..., use_environment_map=0, dropout=0)."""
    return load().adapter_selftest(texture, background_color, points, pose_tangents, intrinsics, confidence, poses_se3,
                                   [list(map(float, v)) for v in views], int(num_layers), int(render_mode),
                                   int(max_list_length), bool(output_background_mask))


def MyAdam(groups, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0):
    """The reference's texture optimiser (torch::optim::MyAdam, src/lib/models/my_adam.cpp) with one fused kernel per
    tensor and step. groups: list of (list of float32 CUDA parameter tensors, learning rate)."""
    return load().MyAdam([(list(ts), float(lr)) for ts, lr in groups], beta1, beta2, eps, weight_decay)


def fill_scene_grid_with_loss(batch, cell_bb_min, cell_bb_length, cell_value, cell_access_count, views, poses_se3,
                              intrinsics, loss_img):
    """PointRendererCache::FillSceneGridWithLoss of the reference (src/lib/rendering/RenderForward.cu:763-791): adds
    the error image [C,h,w] of view `batch` to cell_value / cell_access_count in place. views as in blend_point_cloud."""
    load().fill_scene_grid_with_loss(int(batch), cell_bb_min, cell_bb_length, cell_value, cell_access_count,
                                     [list(map(float, v)) for v in views], poses_se3, intrinsics, loss_img)


def morton_block_shuffle_order(positions, block=256, seed=0):
    """The point order of the reference's scene preprocessing (ReorderMorton64 + RandomBlockShuffle(256),
    src/lib/data/SceneData.cpp:105-106) as a permutation [N] int64 of a [N,3] or [N,4] CPU tensor of positions."""
    return load().morton_block_shuffle_order(positions, int(block), int(seed))


def sort_blocks_by_radius_order(radius, block=256):
    """SceneData::SortBlocksByRadius(256) (src/lib/data/SceneData.cpp:108,1005-1018) as a permutation [N] int64: inside
    every complete block the points sorted by drop-out radius, ascending. radius: [N] CPU tensor."""
    return load().sort_blocks_by_radius_order(radius, int(block))


def scene_preprocess_order(positions_radius, block=256, seed=0):
    """All three steps of src/lib/data/SceneData.cpp:105-108 (Morton order, block shuffle, blocks sorted by radius) for a
    [N,4] CPU tensor (x, y, z, drop-out radius), as a permutation [N] int64."""
    return load().scene_preprocess_order(positions_radius, int(block), int(seed))


def processing_order_on_device(positions, block=256, seed=0):
    """Morton order with shuffled blocks computed on the device of `positions`: int32 [N], for point_order."""
    return load().processing_order_on_device(positions, block, seed)


def set_point_order_refresh(every):
    """Forward calls between rebuilds of the processing order the shim's cache keeps; 0 switches it off."""
    load().set_point_order_refresh(int(every))


def point_order():
    """The processing order the shim's cache currently holds, or None."""
    t = load().point_order()
    return t if t is not None and t.numel() > 0 else None


def point_order_in_use():
    """Whether forward calls are handed the processing order (False: the array's own order is as good)."""
    return bool(load().point_order_in_use())


def fragment_history():
    """Fragments per layer that one view of a recent call left, as the shim's cache has read them back ([] = none yet)."""
    return list(load().fragment_history())


def kept_descriptor_calls():
    """Forward calls of the shim's cache so far that read descriptor records kept from an earlier call."""
    return int(load().kept_descriptor_calls())


def set_keep_packed_descriptors(keep):
    """Whether the shim's cache keeps descriptor records across calls while texture and confidence stay unchanged."""
    load().set_keep_packed_descriptors(bool(keep))


def train_workspace_info():
    """(data_ptr, bytes) of the workspace the binding's cache keeps between training steps; (0, 0) before the first."""
    d = load().train_workspace_info()
    return int(d["data_ptr"]), int(d["bytes"])


def save_scene_checkpoint(prefix, **tensors):
    """Writes VET's scene checkpoint files (<prefix>points.pth, texture.pth, poses.pth, intrinsics.pth; the reference's
    NeuralScene::SaveCheckpoint, src/lib/data/NeuralScene.cpp:407-431) for the given tensors: t_position, t_index,
    texture, background_color, confidence_value_of_point (the raw tensors), tangent_poses, poses_se3, intrinsics."""
    load().save_scene_checkpoint(str(prefix), dict(tensors))


def load_scene_checkpoint(prefix):
    """Reads the same files back (NeuralScene::LoadCheckpoint, src/lib/data/NeuralScene.cpp:343-405) as a dict of CPU
    tensors; files that do not exist leave their tensors out."""
    return dict(load().load_scene_checkpoint(str(prefix)))
