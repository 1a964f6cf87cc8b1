// Adapter between VET's own types and this shim's, for the maintainer's RenderModule.cpp: the few lines that turn a
// NeuralScene, a ReducedImageInfo, a RenderParams and a NeuralRenderInfo of the reference into the shim's bundle, view,
// parameter struct and render info.
//
// Everything here is a template over VET's type, and only the members named in the bodies are touched, so the header
// compiles without VET's headers (saiga, Sophus and Eigen are not needed) and is instantiated in VET with
//   NeuralScene          src/lib/data/NeuralScene.h:22-113
//   ReducedImageInfo     src/lib/data/SceneData.h:39-50
//   RenderParams         src/lib/data/Settings.h:19-93
//   NeuralRenderInfo     src/lib/rendering/PointRenderer.h:23-34
// as they are. The shim's self test (adapter_selftest in point_render.cpp) instantiates it with stand-ins that have the
// same member names and spellings (module holders with operator->, an Eigen-style operator()(row, col), an enum class
// for the camera model) and renders through it.
//
// In RenderModule.cpp (src/lib/models/Pipeline / rendering/RenderModule.cpp:150-232) the call
//     auto combined_images_masks = BlendPointCloud(&nri);                  // nri: the reference's NeuralRenderInfo
// becomes
//     vet_amd::SceneTensors bundle;
//     auto combined_images_masks = vet_amd::BlendPointCloudOf(&nri, shim_cache.get(), &bundle);
// with one `std::shared_ptr<vet_amd::PointRendererCache> shim_cache` kept beside the module's own cache.
#pragma once
#include "point_render.h"

namespace vet_amd
{
// The tensors BlendPointCloud reads through info->scene (src/lib/rendering/RenderInfo.cpp:25-29,
// src/lib/rendering/PointRenderer.cu:129-135,1198-1204).
template <class SceneT>
SceneTensors SceneTensorsOf(SceneT& scene)
{
    SceneTensors st;
    st.texture                   = scene.texture->texture;                    // [C,N] f32
    st.background_color          = scene.texture->background_color;           // [C]
    st.confidence_value_of_point = scene.texture->confidence_value_of_point;  // [1,N]
    st.t_position                = scene.point_cloud_cuda->t_position;        // [N,4]
    st.t_index                   = scene.point_cloud_cuda->t_index;           // [N,1] i32, may be undefined
    st.t_original_color          = scene.point_cloud_cuda->t_original_color;
    st.t_normal                  = scene.point_cloud_cuda->t_normal;
    st.tangent_poses             = scene.poses->tangent_poses;                // [F,6] f64
    st.poses_se3                 = scene.poses->poses_se3;                    // [F,8] f64
    st.intrinsics                = scene.intrinsics->intrinsics;              // [Ncam,13]
    st.dynamic_refinement_t      = scene.dynamic_refinement_t;                // [1] dummy unless dynamic refinement is on
    return st;
}

// ReducedImageInfo -> vetrast_view. crop_transform is saiga's IntrinsicsPinhole (members fx, fy, cx, cy, s);
// crop_rotation an Eigen 2x2 (column-major in memory, read here element by element).
template <class ImageT>
ReducedImageInfo ViewOf(const ImageT& img)
{
    ReducedImageInfo v;
    v.w                 = img.w;
    v.h                 = img.h;
    v.image_index       = img.image_index;
    v.camera_index      = img.camera_index;
    v.camera_model_type = static_cast<int>(img.camera_model_type);  // CameraModel::PINHOLE_DISTORTION = 0, OCAM = 1
    v.crop_transform[0] = img.crop_transform.fx;
    v.crop_transform[1] = img.crop_transform.fy;
    v.crop_transform[2] = img.crop_transform.cx;
    v.crop_transform[3] = img.crop_transform.cy;
    v.crop_transform[4] = img.crop_transform.s;
    v.crop_rotation[0]  = img.crop_rotation(0, 0);
    v.crop_rotation[1]  = img.crop_rotation(0, 1);
    v.crop_rotation[2]  = img.crop_rotation(1, 0);
    v.crop_rotation[3]  = img.crop_rotation(1, 1);
    return v;
}

// The RenderParams members the blending path reads, by name. Members of the shim's struct that the reference does not
// have (the switches for its accidents, the fused preparation steps, the bin-size hints) keep their defaults, which
// reproduce the reference.
template <class ParamsT>
RenderParams RenderParamsOf(const ParamsT& p)
{
    RenderParams r;
    r.check_normal                 = p.check_normal;
    r.dropout                      = p.dropout;
    r.drop_out_radius_threshold    = p.drop_out_radius_threshold;
    r.drop_out_points_by_radius    = p.drop_out_points_by_radius;
    r.K_gradient_factor            = p.K_gradient_factor;
    r.distortion_gradient_factor   = p.distortion_gradient_factor;
    r.num_texture_channels         = p.num_texture_channels;
    r.output_background_mask       = p.output_background_mask;
    r.output_background_mask_value = p.output_background_mask_value;
    r.add_depth_to_network         = p.add_depth_to_network;
    r.dist_cutoff                  = p.dist_cutoff;
    r.stability_cutoff_value       = p.stability_cutoff_value;
    r.need_point_gradient          = p.need_point_gradient;
    r.use_environment_map          = p.use_environment_map;
    r.render_mode                  = p.render_mode;
    r.depth_accept_blend           = p.depth_accept_blend;
    r.viewer_only                  = p.viewer_only;
    r.debug_max_list_length        = p.debug_max_list_length;
    return r;
}

// The reference's NeuralRenderInfo -> the shim's. `bundle` receives the scene's tensors and must outlive the call
// (the backward pass does not touch it: what it needs is saved with the graph).
template <class InfoT>
c10::intrusive_ptr<NeuralRenderInfo> RenderInfoOf(const InfoT& info, PointRendererCache* cache, SceneTensors* bundle)
{
    *bundle        = SceneTensorsOf(*info.scene);
    auto nri       = c10::make_intrusive<NeuralRenderInfo>();
    nri->scene     = bundle;
    nri->params    = RenderParamsOf(info.params);
    nri->num_layers    = info.num_layers;
    nri->train         = info.train;
    nri->current_epoch = info.current_epoch;
    nri->timer_system  = nullptr;  // per-kernel times come from vetrast_scope_times
    nri->cache         = cache;
    nri->images.reserve(info.images.size());
    for (const auto& img : info.images) nri->images.push_back(ViewOf(img));
    return nri;
}

// BlendPointCloud(NeuralRenderInfo*) of the reference (src/lib/rendering/RenderInfo.cpp:18-47) on the reference's own
// info object: L images, then L depth images with add_depth_to_network, then L masks with output_background_mask
// (the order of src/lib/rendering/PointRenderer.cu:1061-1066).
template <class InfoT>
std::vector<torch::Tensor> BlendPointCloudOf(InfoT* info, PointRendererCache* cache, SceneTensors* bundle)
{
    auto nri = RenderInfoOf(*info, cache, bundle);
    return BlendPointCloud(nri.get());
}
}  // namespace vet_amd
