// libtorch host side of the MI355X blending point rasterizer: autograd Function with the reference's argument order,
// calling the C ABI of include/vetrast.h. See point_render.h for the reference lines each piece mirrors.
#include "point_render.h"
#include "vet_adapter.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>
#include <random>

#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

namespace vet_amd
{
namespace
{
void check_status(int st, const char* where)
{
    TORCH_CHECK(st == VETRAST_OK, "vetrast ", where, " failed: ", st, " (", vetrast_status_string(st), ")");
}

void* current_stream()
{
    return (void*)c10::hip::getCurrentHIPStream().stream();
}

vetrast_params to_abi_params(const RenderParams& p, int num_layers)
{
    vetrast_params q;
    std::memset(&q, 0, sizeof(q));
    q.render_mode                      = p.render_mode;
    q.depth_accept_blend               = p.depth_accept_blend;
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l) q.expected_fragments[l] = p.expected_fragments[l] > 0.f ? p.expected_fragments[l] : 0.f;
    q.num_texture_channels             = p.num_texture_channels;
    q.num_layers                       = num_layers;
    q.debug_max_list_length            = p.debug_max_list_length;
    q.use_environment_map              = p.use_environment_map ? 1 : 0;
    q.need_point_gradient              = p.need_point_gradient ? 1 : 0;
    q.viewer_only                      = p.viewer_only ? 1 : 0;
    q.stability_cutoff_value           = p.stability_cutoff_value;
    q.drop_out_points_by_radius        = p.drop_out_points_by_radius ? 1 : 0;
    q.drop_out_radius_threshold        = p.drop_out_radius_threshold;
    q.output_background_mask           = p.output_background_mask ? 1 : 0;
    q.output_background_mask_value     = p.output_background_mask_value;
    q.check_normal                     = p.check_normal ? 1 : 0;
    q.quirk_background_confidence_leak = p.quirk_background_confidence_leak ? 1 : 0;
    q.point_gradient_normalization     = p.point_gradient_normalization;
    q.K_gradient_factor                = p.K_gradient_factor;
    q.allow_distortion                 = p.allow_distortion ? 1 : 0;
    q.distortion_gradient_factor       = p.distortion_gradient_factor;
    q.camera_gradient_normalization    = p.camera_gradient_normalization ? 1 : 0;
    q.confidence_activation            = p.fused_confidence_scale > 0.f ? 1 : 0;
    q.confidence_scale                 = p.fused_confidence_scale;
    q.texture_abs                      = p.fused_texture_abs ? 1 : 0;
    return q;
}

void check_f32_cuda(const torch::Tensor& t, const char* name)
{
    TORCH_CHECK(t.defined() && t.is_cuda() && t.scalar_type() == torch::kFloat32 && t.is_contiguous(), name,
                " must be a contiguous float32 tensor on the GPU");
}

// Fills the part of the argument struct that forward and backward share. `info->images` must outlive the call.
vetrast_forward_args make_forward_args(NeuralRenderInfo* info, const torch::Tensor& texture,
                                       const torch::Tensor& background_color, const torch::Tensor& points,
                                       const torch::Tensor& intrinsics, const torch::Tensor& confidence,
                                       const torch::Tensor& dropout, const torch::Tensor& poses_se3,
                                       const torch::Tensor& t_index)
{
    check_f32_cuda(texture, "texture");
    check_f32_cuda(background_color, "background_color");
    check_f32_cuda(points, "points");
    check_f32_cuda(intrinsics, "intrinsics");
    check_f32_cuda(confidence, "confidence");
    TORCH_CHECK(points.dim() == 2 && points.size(1) == 4, "points must be [N,4]");  // PointRenderer.cu:532
    TORCH_CHECK(texture.dim() == 2 && texture.size(1) == points.size(0), "texture must be [C,N]");
    TORCH_CHECK(confidence.numel() == points.size(0), "confidence must be [1,N]");
    TORCH_CHECK(intrinsics.dim() == 2 && intrinsics.size(1) == 13, "intrinsics must be [num_cameras,13]");
    TORCH_CHECK(poses_se3.defined() && poses_se3.is_cuda() && poses_se3.scalar_type() == torch::kFloat64 &&
                    poses_se3.is_contiguous() && poses_se3.dim() == 2 && poses_se3.size(1) == 8,
                "poses_se3 must be a contiguous [F,8] float64 tensor on the GPU");
    TORCH_CHECK(info->params.render_mode == VETRAST_RENDER_FULL_BLEND ||
                    info->params.render_mode == VETRAST_RENDER_FUZZY_BLEND ||
                    info->params.render_mode == VETRAST_RENDER_BILINEAR_BLEND,
                "only render_mode 1 (FULL_BLEND), 2 (FUZZY_BLEND) and 3 (BILINEAR_BLEND) are implemented");
    TORCH_CHECK(!info->images.empty(), "no views");

    vetrast_forward_args a;
    std::memset(&a, 0, sizeof(a));
    a.num_points  = (int32_t)points.size(0);
    a.num_views   = (int32_t)info->images.size();
    a.num_poses   = (int32_t)poses_se3.size(0);
    a.num_cameras = (int32_t)intrinsics.size(0);
    a.position    = points.data_ptr<float>();
    a.index       = nullptr;
    if (t_index.defined())
    {
        TORCH_CHECK(t_index.is_cuda() && t_index.scalar_type() == torch::kInt32 && t_index.is_contiguous() &&
                        t_index.numel() == points.size(0),
                    "t_index must be a contiguous [N,1] int32 tensor on the GPU");
        a.index = t_index.data_ptr<int32_t>();
    }
    a.texture    = texture.data_ptr<float>();
    a.confidence = confidence.data_ptr<float>();
    a.background = background_color.data_ptr<float>();
    a.dropout    = dropout.defined() ? dropout.data_ptr<float>() : nullptr;
    a.poses_se3  = poses_se3.data_ptr<double>();
    a.intrinsics = intrinsics.data_ptr<float>();
    a.views      = info->images.data();
    RenderParams prm         = info->params;
    prm.num_texture_channels = (int)texture.size(0);
    a.params                 = to_abi_params(prm, info->num_layers);
    return a;
}

}  // namespace

PointRendererCache::PointRendererCache()
{
    check_status(vetrast_create(&ctx), "create");
}

PointRendererCache::~PointRendererCache()
{
    vetrast_destroy(ctx);
}

static const char* kDistortionRefused =
    "a camera has non-zero distortion coefficients (columns 5..12 of intrinsics): the distortion model of the "
    "reference lives in saiga and is not implemented; such cameras are refused rather than rendered as "
    "undistorted pinholes (RenderParams::allow_distortion switches the published rational model on)";

void PointRendererCache::PollDeviceFlags()
{
    if (!flags_pending_ || !flags_event_ || !flags_event_->query()) return;
    flags_pending_ = false;
    if (flags_host_.data_ptr<int32_t>()[0] & 1)
    {
        checked_intrinsics_ptr_ = nullptr;  // the next call checks the tensor itself again, and blocks for it
        TORCH_CHECK(false, "an earlier forward call rendered with these intrinsics: ", kDistortionRefused);
    }
}

void PointRendererCache::CheckIntrinsics(const torch::Tensor& intrinsics)
{
    TORCH_CHECK(intrinsics.defined() && intrinsics.dim() == 2 && intrinsics.size(1) == 13,
                "intrinsics must be [num_cameras,13]");
    PollDeviceFlags();
    const void* ptr       = intrinsics.data_ptr();
    const int64_t version = (int64_t)intrinsics._version();
    const auto held = checked_intrinsics_storage_.lock();
    if (ptr == checked_intrinsics_ptr_ && intrinsics.numel() == checked_intrinsics_numel_ && held &&
        held.get() == intrinsics.storage().unsafeGetStorageImpl())
    {
        // known memory: no read here; ask for the device's own verdict on this call where the contents may have changed
        if (version != checked_intrinsics_version_ || ++calls_since_flags_ >= 64) flags_wanted_ = true;
        checked_intrinsics_version_ = version;
        return;
    }
    // blocking: one device -> host read per intrinsics tensor
    const bool distorted = intrinsics.detach().slice(1, 5, 13).ne(0).any().item<bool>();
    TORCH_CHECK(!distorted, kDistortionRefused);
    checked_intrinsics_ptr_     = ptr;
    checked_intrinsics_storage_ = intrinsics.storage().getWeakStorageImpl();
    checked_intrinsics_version_ = version;
    checked_intrinsics_numel_   = intrinsics.numel();
    flags_wanted_               = false;
    calls_since_flags_          = 0;
}

void PointRendererCache::NoteDeviceFlags(const torch::Tensor& workspace, const vetrast_workspace_layout& lay)
{
    if (!flags_wanted_ || flags_pending_) return;
    torch::NoGradGuard no_grad;
    if (!flags_host_.defined())
        flags_host_ = torch::zeros({4}, torch::TensorOptions().dtype(torch::kInt32).pinned_memory(true));
    flags_host_.copy_(workspace.narrow(0, (int64_t)lay.flags_base, 16).view(torch::kInt32), /*non_blocking=*/true);
    if (!flags_event_) flags_event_ = std::make_unique<c10::Event>(c10::DeviceType::CUDA);
    flags_event_->record(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
    flags_pending_     = true;
    flags_wanted_      = false;
    calls_since_flags_ = 0;
}

torch::Tensor PointRendererCache::KeptDescriptorsFor(const torch::Tensor& texture, const torch::Tensor& confidence,
                                                     const vetrast_params& params)
{
    if (!keep_packed_descriptors) return torch::Tensor();
    PackKey key;
    key.texture            = texture.data_ptr();
    key.confidence         = confidence.data_ptr();
    key.texture_storage    = texture.storage().unsafeGetStorageImpl();
    key.confidence_storage = confidence.storage().unsafeGetStorageImpl();
    key.texture_version    = (int64_t)texture._version();
    key.confidence_version = (int64_t)confidence._version();
    key.N                  = confidence.numel();
    key.C                  = params.num_texture_channels;
    key.activation         = params.confidence_activation;
    key.texture_abs        = params.texture_abs;
    key.scale              = params.confidence_scale;
    const bool alive       = pack_texture_storage_.lock() && pack_confidence_storage_.lock();
    if (!(alive && key == pack_key_))
    {
        // first sight of these tensors in this state: remember them, interleave inside the call
        pack_key_                = key;
        pack_texture_storage_    = texture.storage().getWeakStorageImpl();
        pack_confidence_storage_ = confidence.storage().getWeakStorageImpl();
        packed_valid_            = false;
        return torch::Tensor();
    }
    if (!packed_valid_)
    {
        if (!packed_.defined() || packed_.size(0) != key.N || packed_.device() != texture.device())
            packed_ = torch::empty({key.N, 8}, texture.options().requires_grad(false));
        vetrast_pack_args a;
        std::memset(&a, 0, sizeof(a));
        a.num_points = (int32_t)key.N;
        a.texture    = texture.data_ptr<float>();
        a.confidence = confidence.data_ptr<float>();
        a.params     = params;
        a.packed     = packed_.data_ptr<float>();
        check_status(vetrast_pack_descriptors(ctx, &a, c10::hip::getCurrentHIPStream().stream()), "pack_descriptors");
        packed_valid_ = true;
    }
    ++calls_with_kept_descriptors;
    return packed_;
}

void PointRendererCache::FillSceneGridWithLoss(int batch, const CellTensors& cells,
                                               const std::vector<ReducedImageInfo>& images, torch::Tensor poses_se3,
                                               torch::Tensor intrinsics, torch::Tensor loss_img)
{
    TORCH_CHECK(batch >= 0 && batch < (int)images.size(), "FillSceneGridWithLoss: batch index out of range");
    auto is_dev = [](const torch::Tensor& t, torch::ScalarType ty) {
        return t.defined() && t.is_cuda() && t.scalar_type() == ty && t.is_contiguous();
    };
    TORCH_CHECK(is_dev(cells.t_cell_bb_min, torch::kFloat32) && is_dev(cells.t_cell_bb_length, torch::kFloat32) &&
                    is_dev(cells.t_cell_value, torch::kFloat32) && is_dev(cells.t_cell_access_count, torch::kInt32),
                "FillSceneGridWithLoss: cell tensors must be contiguous CUDA tensors (float32, float32, float32, int32)");
    TORCH_CHECK(is_dev(poses_se3, torch::kFloat64) && is_dev(intrinsics, torch::kFloat32) && is_dev(loss_img, torch::kFloat32),
                "FillSceneGridWithLoss: poses_se3 (float64), intrinsics and loss_img (float32) must be contiguous CUDA tensors");
    TORCH_CHECK(loss_img.dim() == 3, "FillSceneGridWithLoss: loss_img is [C,h,w]");
    CheckIntrinsics(intrinsics);
    const int64_t n = cells.t_cell_value.numel();
    TORCH_CHECK(cells.t_cell_bb_min.numel() == 3 * n && cells.t_cell_bb_length.numel() == 3 * n &&
                    cells.t_cell_access_count.numel() == n,
                "FillSceneGridWithLoss: cell tensors disagree in size");
    vetrast_lift_args a;
    std::memset(&a, 0, sizeof(a));
    a.num_cells         = n;
    a.cell_bb_min       = cells.t_cell_bb_min.data_ptr<float>();
    a.cell_bb_length    = cells.t_cell_bb_length.data_ptr<float>();
    a.cell_value        = cells.t_cell_value.data_ptr<float>();
    a.cell_access_count = cells.t_cell_access_count.data_ptr<int32_t>();
    a.num_poses         = (int32_t)poses_se3.size(0);
    a.num_cameras       = (int32_t)intrinsics.size(0);
    a.poses_se3         = poses_se3.data_ptr<double>();
    a.intrinsics        = intrinsics.data_ptr<float>();
    a.view              = images[batch];
    a.loss_image        = loss_img.data_ptr<float>();
    a.channels          = (int32_t)loss_img.size(0);
    a.height            = (int32_t)loss_img.size(1);
    a.width             = (int32_t)loss_img.size(2);
    a.border_pixels     = VETRAST_LIFT_BORDER_PIXELS;
    const int64_t need  = (int64_t)vetrast_lift_workspace_bytes(n);
    if (!lift_workspace.defined() || lift_workspace.numel() < need || lift_workspace.device() != loss_img.device())
        lift_workspace = torch::empty({std::max<int64_t>(need, 256)}, torch::dtype(torch::kUInt8).device(loss_img.device()));
    a.workspace       = lift_workspace.data_ptr();
    a.workspace_bytes = (size_t)lift_workspace.numel();
    check_status(vetrast_lift_error(ctx, &a, c10::hip::getCurrentHIPStream().stream()), "lift_error");
}

std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info)
{
    TORCH_CHECK(info && info->scene && info->cache, "BlendPointCloud: scene and cache must be set");
    torch::intrusive_ptr<NeuralRenderInfo> render_data = torch::make_intrusive<NeuralRenderInfo>(*info);
    render_data->grad_mode = torch::GradMode::is_enabled();  // (inside PointRender::forward it is always off)
    SceneTensors& s                                    = *render_data->scene;
    return PointRender::apply(s.texture, s.background_color, s.t_position, s.tangent_poses, s.intrinsics,
                              s.confidence_value_of_point, s.dynamic_refinement_t, torch::IValue(render_data));
}

torch::autograd::variable_list PointRender::forward(torch::autograd::AutogradContext* ctx, torch::Tensor texture,
                                                    torch::Tensor background_color, torch::Tensor points,
                                                    torch::Tensor pose_tangents, torch::Tensor intrinsics,
                                                    torch::Tensor confidence, torch::Tensor dynamic_refinement,
                                                    torch::IValue info_value)
{
    ctx->saved_data["render_info"] = info_value;
    NeuralRenderInfo* info         = info_value.toCustomClass<NeuralRenderInfo>().get();
    TORCH_CHECK(dynamic_refinement.dim() <= 1, "per-view point displacements are not implemented");

    const int B = (int)info->images.size(), L = info->num_layers, C = (int)texture.size(0);
    const int64_t N = points.size(0);
    auto f32        = torch::TensorOptions().device(points.device()).dtype(torch::kFloat32);
    if (!info->params.allow_distortion) info->cache->CheckIntrinsics(intrinsics);

    // dropout mask per view, PointRenderer.cu:461-468 (the mask is 1 where a point is dropped)
    torch::Tensor dropout;
    if (info->train && info->params.dropout > 0) dropout = torch::empty({B, N}, f32).bernoulli_(info->params.dropout);

    if (info->params.size_bins_from_history)
        info->cache->ExpectedFragments(info->params.expected_fragments, N, L, info->images[0].w, info->images[0].h,
                                       info->params.render_mode);
    // side inputs read through info->scene; they are saved with the graph so that backward does not touch the scene
    const torch::Tensor poses_se3 = info->scene->poses_se3;
    const torch::Tensor t_index   = info->scene->t_index;
    vetrast_forward_args a =
        make_forward_args(info, texture, background_color, points, intrinsics, confidence, dropout, poses_se3, t_index);
    vetrast_workspace_layout lay;
    check_status(vetrast_workspace_layout_for_mode(a.num_points, B, L, info->images[0].w, info->images[0].h,
                                                   a.params.render_mode, &lay),
                 "layout");

    const bool need_backward =
        ctx != nullptr && info->grad_mode && (texture.requires_grad() || background_color.requires_grad() || points.requires_grad() ||
                           confidence.requires_grad() || pose_tangents.requires_grad() || intrinsics.requires_grad());
    // Kept descriptor records only serve calls without a backward pass. The interleave inside a call is also what
    // brings the rows into the last-level cache for the gathers of the backward pass: measured with kept records, the
    // forward call is 9 us faster and the backward call 12 us slower at 2 M points.
    torch::Tensor kept_pack;
    if (!need_backward) kept_pack = info->cache->KeptDescriptorsFor(texture, confidence, a.params);
    if (kept_pack.defined()) a.packed_descriptors = kept_pack.data_ptr<float>();
    auto u8 = torch::TensorOptions().device(points.device()).dtype(torch::kUInt8);
    torch::Tensor workspace;
    if (need_backward)
    {
        // Saved for backward, like the reference's buffers. The workspace of the step before is taken again once the
        // graph that saved it is gone (nothing but the cache holds it): the usual training loop allocates it once.
        auto& ws = info->cache->train_workspace;
        if (!ws.defined() || ws.use_count() > 1 || ws.numel() < (int64_t)lay.total_bytes || ws.device() != points.device())
            ws = torch::empty({(int64_t)lay.total_bytes}, u8);
        workspace = ws;
    }
    else
    {
        auto& ws = info->cache->eval_workspace;
        if (!ws.defined() || ws.numel() < (int64_t)lay.forward_only_bytes || ws.device() != points.device())
            ws = torch::empty({(int64_t)lay.forward_only_bytes}, u8);
        workspace = ws;
    }

    std::vector<torch::Tensor> out(L), mask;
    for (int l = 0; l < L; ++l)
    {
        out[l]   = torch::empty({B, C, lay.layer_h[l], lay.layer_w[l]}, f32);
        a.out[l] = out[l].data_ptr<float>();
    }
    if (info->params.output_background_mask)
    {
        mask.resize(L);
        for (int l = 0; l < L; ++l)
        {
            mask[l]       = torch::empty({B, 1, lay.layer_h[l], lay.layer_w[l]}, f32);
            a.out_mask[l] = mask[l].data_ptr<float>();
        }
    }
    if (info->cache->keep_layer_weights)
    {
        info->cache->layer_weights.resize(L);
        for (int l = 0; l < L; ++l)
        {
            info->cache->layer_weights[l] = torch::empty({B, 1, lay.layer_h[l], lay.layer_w[l]}, f32);
            a.out_weight[l]               = info->cache->layer_weights[l].data_ptr<float>();
        }
    }
    a.workspace         = workspace.data_ptr();
    a.workspace_bytes   = (size_t)workspace.numel();
    a.save_for_backward = need_backward ? 1 : 0;
    const torch::Tensor& order = info->cache->PointOrderFor(points);
    a.point_order              = order.defined() ? order.data_ptr<int32_t>() : nullptr;
    check_status(vetrast_forward(info->cache->ctx, &a, current_stream()), "forward");
    if (!info->params.allow_distortion) info->cache->NoteDeviceFlags(workspace, lay);
    if (info->params.size_bins_from_history)
        info->cache->NoteFragmentCounts(workspace, lay, N, L, info->images[0].w, info->images[0].h, a.params.render_mode);

    if (need_backward)
    {
        // saved state: workspace (scan, sorted lists, transmittance, weight), outputs, dropout. PointRenderer.cu:1027-1059
        std::vector<torch::Tensor> saved = {workspace, texture, background_color, points, intrinsics, confidence,
                                            poses_se3};
        saved.insert(saved.end(), out.begin(), out.end());
        if (dropout.defined()) saved.push_back(dropout);
        if (t_index.defined()) saved.push_back(t_index);
        ctx->save_for_backward(saved);
        ctx->saved_data["has_dropout"] = dropout.defined();
        ctx->saved_data["has_index"]   = t_index.defined();
        ctx->saved_data["points_need_grad"] = points.requires_grad();
        ctx->saved_data["pose_need_grad"]   = pose_tangents.requires_grad();
        ctx->saved_data["intr_need_grad"]   = intrinsics.requires_grad();
        ctx->saved_data["num_poses"]        = (int64_t)poses_se3.size(0);
    }
    // With add_depth_to_network the output list carries L depth tensors behind the images
    // (src/lib/rendering/PointRenderer.cu:1061-1066). The blend modes never write them: they are the zero-filled
    // buffers of the cache (:402-470), which is what is returned here.
    std::vector<torch::Tensor> depth;
    if (info->params.add_depth_to_network)
        for (int l = 0; l < L; ++l) depth.push_back(torch::zeros({B, 1, lay.layer_h[l], lay.layer_w[l]}, f32));
    // masks are not differentiable (the reference detaches them in RenderModule.cpp:74-102); nor are the zero depths
    if (ctx)
    {
        std::vector<torch::Tensor> constants = mask;
        constants.insert(constants.end(), depth.begin(), depth.end());
        ctx->mark_non_differentiable(constants);
    }
    out.insert(out.end(), depth.begin(), depth.end());
    out.insert(out.end(), mask.begin(), mask.end());
    return out;
}

torch::autograd::variable_list PointRender::backward(torch::autograd::AutogradContext* ctx,
                                                     torch::autograd::variable_list grad_output)
{
    torch::IValue info_value = ctx->saved_data["render_info"];
    NeuralRenderInfo* info   = info_value.toCustomClass<NeuralRenderInfo>().get();
    const int L              = info->num_layers;
    auto saved               = ctx->get_saved_variables();
    const bool has_dropout   = ctx->saved_data["has_dropout"].toBool();
    const bool has_index     = ctx->saved_data["has_index"].toBool();
    constexpr int kFixed     = 7;
    TORCH_CHECK((int)saved.size() == kFixed + L + (has_dropout ? 1 : 0) + (has_index ? 1 : 0),
                "unexpected number of saved tensors");  // PointRenderer.cu:1163-1164
    TORCH_CHECK((int)grad_output.size() >= L, "expected one upstream gradient per layer");  // PointRenderer.cu:1158-1159
    torch::Tensor workspace = saved[0], texture = saved[1], background_color = saved[2], points = saved[3],
                  intrinsics = saved[4], confidence = saved[5], poses_se3 = saved[6];
    torch::Tensor dropout = has_dropout ? saved[kFixed + L] : torch::Tensor();
    torch::Tensor t_index = has_index ? saved[kFixed + L + (has_dropout ? 1 : 0)] : torch::Tensor();

    vetrast_backward_args g;
    std::memset(&g, 0, sizeof(g));
    g.fwd = make_forward_args(info, texture, background_color, points, intrinsics, confidence, dropout, poses_se3, t_index);
    std::vector<torch::Tensor> grads(L);
    for (int l = 0; l < L; ++l)
    {
        g.fwd.out[l] = saved[kFixed + l].data_ptr<float>();
        TORCH_CHECK(grad_output[l].defined(), "upstream gradient of layer ", l, " is undefined");
        TORCH_CHECK(grad_output[l].scalar_type() == torch::kFloat32, "upstream gradients must be float32");  // :1117
        grads[l]      = grad_output[l].contiguous();
        g.grad_out[l] = grads[l].data_ptr<float>();
    }
    g.fwd.workspace         = workspace.data_ptr();
    g.fwd.workspace_bytes   = (size_t)workspace.numel();
    g.fwd.save_for_backward = 1;

    // zeros_like of each gradient tensor (PointRenderer.cu:267-277); the library overwrites them.
    torch::Tensor g_texture    = torch::empty_like(texture);
    torch::Tensor g_confidence = torch::empty_like(confidence);
    torch::Tensor g_background = torch::empty_like(background_color);
    torch::Tensor g_points, g_point_count;
    g.grad_texture    = g_texture.data_ptr<float>();
    g.grad_confidence = g_confidence.data_ptr<float>();
    g.grad_background = g_background.data_ptr<float>();
    if (ctx->saved_data["points_need_grad"].toBool())
    {
        g_points           = torch::empty_like(points);
        g_point_count      = torch::empty({points.size(0)}, points.options());
        g.grad_points      = g_points.data_ptr<float>();
        g.grad_point_count = g_point_count.data_ptr<float>();
    }
    torch::Tensor g_pose, g_pose_count, g_intrinsics, g_intrinsics_count;
    if (ctx->saved_data["pose_need_grad"].toBool())  // PointRenderer.cu:287-293
    {
        const int64_t F      = ctx->saved_data["num_poses"].toInt();
        g_pose               = torch::empty({F, 6}, points.options().dtype(torch::kFloat64));
        g_pose_count         = torch::empty({F}, points.options());
        g.grad_pose          = g_pose.data_ptr<double>();
        g.grad_pose_count    = g_pose_count.data_ptr<float>();
    }
    if (ctx->saved_data["intr_need_grad"].toBool())  // PointRenderer.cu:295-300
    {
        g_intrinsics            = torch::empty_like(intrinsics);
        g_intrinsics_count      = torch::empty({intrinsics.size(0)}, intrinsics.options());
        g.grad_intrinsics       = g_intrinsics.data_ptr<float>();
        g.grad_intrinsics_count = g_intrinsics_count.data_ptr<float>();
    }
    check_status(vetrast_backward(info->cache->ctx, &g, current_stream()), "backward");

    // order: texture, background, points, pose_tangent, intrinsics, confidence, dynamic (PointRenderer.cu:1319-1322),
    // plus one empty gradient for the IValue (RenderInfo.cpp:64). Undefined where the input does not require grad.
    return {g_texture, g_background, g_points, g_pose, g_intrinsics, g_confidence, torch::Tensor(), torch::Tensor()};
}

}  // namespace vet_amd

TORCH_LIBRARY(vet_amd, m)
{
    m.class_<vet_amd::NeuralRenderInfo>("NeuralRenderInfo").def(torch::init());
}

namespace vet_amd
{
std::pair<std::vector<torch::Tensor>, std::vector<torch::Tensor>> PointRenderModule::forward(NeuralRenderInfo* nri)
{
    TORCH_CHECK(nri, "PointRenderModule::forward: null NeuralRenderInfo");
    nri->cache = cache.get();
    const bool with_environment = environment_map && enable_environment_map;
    TORCH_CHECK(!with_environment || nri->params.output_background_mask,
                "the environment map needs output_background_mask");  // RenderModule.cpp:155
    cache->keep_layer_weights = with_environment;
    // IntrinsicsPinhole::scale multiplies all five entries (fx, fy, cx, cy, s)
    auto rescale = [&](float f) {
        for (auto& i : nri->images)
        {
            i.w = f > 1.f ? i.w * 2 : i.w / 2;
            i.h = f > 1.f ? i.h * 2 : i.h / 2;
            for (int k = 0; k < 5; ++k) i.crop_transform[k] *= f;
        }
    };
    if (super_sampling) rescale(2.f);
    std::vector<torch::Tensor> combined;
    try
    {
        combined = BlendPointCloud(nri);
    }
    catch (...)
    {
        if (super_sampling) rescale(0.5f);
        throw;
    }
    const int L = nri->num_layers;
    std::vector<torch::Tensor> images(combined.begin(), combined.begin() + L);
    // RenderModule.cpp:76-100: then the depths (with add_depth_to_network), then the masks
    const bool with_depth = nri->params.add_depth_to_network;
    std::vector<torch::Tensor> depths, masks;
    const int expected = L * (1 + (with_depth ? 1 : 0) + (nri->params.output_background_mask ? 1 : 0));
    TORCH_CHECK((int)combined.size() == expected, "BlendPointCloud returned ", combined.size(), " tensors, expected ", expected);
    if (with_depth) depths.assign(combined.begin() + L, combined.begin() + 2 * L);
    if (nri->params.output_background_mask)
    {
        masks.assign(combined.begin() + (with_depth ? 2 : 1) * L, combined.end());
        for (auto& m : masks) m = m.detach();
    }
    if (super_sampling)
    {
        // RenderModule.cpp:102-127 pools images, depths and masks alike
        for (auto& img : images) img = torch::avg_pool2d(img, {2, 2});
        for (auto& d : depths) d = torch::avg_pool2d(d, {2, 2});
        for (auto& m : masks) m = torch::avg_pool2d(m, {2, 2});
        rescale(0.5f);
    }
    if (with_environment)
    {
        // RenderModule.cpp:129-202 (the FUZZY_DT masking of :143-151 belongs to the depth-test mode, which is refused)
        const int64_t B = images.front().size(0);
        std::vector<std::vector<torch::Tensor>> layers(L);
        for (int i = 0; i < L; ++i)
            for (int64_t b = 0; b < B; ++b) layers[i].push_back(cache->layer_weights[i].slice(0, b, b + 1).clone());
        std::vector<torch::Tensor> env_maps = environment_map(layers, nri);
        TORCH_CHECK((int)env_maps.size() == L, "the environment map returned ", env_maps.size(), " layers, expected ", L);
        for (int i = 0; i < L; ++i)
        {
            if (cat_env_to_color)
            {
                images[i] = torch::cat({images[i], env_maps[i]}, 1);
                continue;
            }
            torch::Tensor masking = torch::ones_like(env_maps[i]);
            if (no_envmap_at_points)
            {
                std::vector<torch::Tensor> per_view;
                for (int64_t b = 0; b < B; ++b)
                    per_view.push_back(torch::where(layers[i][b] > 0.001, torch::zeros_like(layers[i][b]),
                                                    torch::ones_like(layers[i][b])));
                masking = torch::cat(per_view, 0).repeat({1, env_maps[i].size(1), 1, 1});  // num_texture_channels
            }
            images[i] = images[i] + masking * env_maps[i];
        }
    }
    if (cat_masks_to_color)
    {
        TORCH_CHECK(!masks.empty(), "cat_masks_to_color needs output_background_mask");
        for (int i = 0; i < L; ++i) images[i] = torch::cat({images[i], masks[i]}, 1);
    }
    if (with_depth)  // RenderModule.cpp:223-232
        for (int i = 0; i < L; ++i) images[i] = torch::cat({images[i], depths[i]}, 1);
    TORCH_CHECK(images.front().size(2) == nri->images.front().h && images.front().size(3) == nri->images.front().w,
                "PointRenderModule: output size does not match the view");
    return {images, masks};
}

namespace
{
bool file_exists(const std::string& path)
{
    std::ifstream f(path, std::ios::binary);
    return f.good();
}

// One entry of a module archive; false if the archive has no entry of that name.
bool read_entry(torch::serialize::InputArchive& ar, const char* name, torch::Tensor& t, bool is_buffer)
{
    return ar.try_read(name, t, is_buffer);
}
}  // namespace

SceneTensors LoadSceneCheckpoint(const std::string& prefix, torch::Device device)
{
    SceneTensors st;
    auto open = [&](const char* file, torch::serialize::InputArchive& ar) {
        const std::string path = prefix + file;
        if (!file_exists(path)) return false;
        ar.load_from(path, device);
        return true;
    };
    {
        torch::serialize::InputArchive ar;
        if (open("points.pth", ar))
        {
            TORCH_CHECK(read_entry(ar, "t_position", st.t_position, false), "points.pth has no t_position");
            read_entry(ar, "t_index", st.t_index, true);
            // what the rasterizer does not read is carried along for SaveSceneCheckpoint
            read_entry(ar, "t_original_color", st.t_original_color, true);
            read_entry(ar, "t_normal", st.t_normal, true);
            read_entry(ar, "t_cell_bb_min", st.t_cell_bb_min, true);
            read_entry(ar, "t_cell_bb_length", st.t_cell_bb_length, true);
            read_entry(ar, "t_cell_value", st.t_cell_value, true);
            read_entry(ar, "t_cell_access_count", st.t_cell_access_count, true);
            TORCH_CHECK(st.t_position.scalar_type() == torch::kFloat32 && st.t_position.dim() == 2 && st.t_position.size(1) == 4,
                        "t_position must be [N,4] float32");
            TORCH_CHECK(!st.t_index.defined() ||
                            (st.t_index.scalar_type() == torch::kInt32 && st.t_index.size(0) == st.t_position.size(0)),
                        "t_index must be [N,1] int32");  // NeuralScene.cpp:357-360
        }
    }
    {
        torch::serialize::InputArchive ar;
        if (open("texture.pth", ar))
        {
            TORCH_CHECK(read_entry(ar, "texture", st.texture, false), "texture.pth has no texture");
            TORCH_CHECK(read_entry(ar, "background_color", st.background_color, false), "texture.pth has no background_color");
            TORCH_CHECK(read_entry(ar, "confidence_value_of_point", st.confidence_value_of_point, false),
                        "texture.pth has no confidence_value_of_point");
        }
    }
    {
        torch::serialize::InputArchive ar;
        if (open("poses.pth", ar))
        {
            TORCH_CHECK(read_entry(ar, "tangent_poses", st.tangent_poses, false), "poses.pth has no tangent_poses");
            TORCH_CHECK(read_entry(ar, "poses_se3", st.poses_se3, true), "poses.pth has no poses_se3");
            TORCH_CHECK(st.poses_se3.scalar_type() == torch::kFloat64 && st.tangent_poses.scalar_type() == torch::kFloat64,
                        "poses are float64");  // NeuralScene.cpp:385-386
        }
    }
    {
        torch::serialize::InputArchive ar;
        if (open("intrinsics.pth", ar))
            TORCH_CHECK(read_entry(ar, "intrinsics", st.intrinsics, false), "intrinsics.pth has no intrinsics");
    }
    return st;
}

void SaveSceneCheckpoint(const std::string& prefix, const SceneTensors& st)
{
    auto cpu = [](const torch::Tensor& t) { return t.detach().to(torch::kCPU).contiguous(); };
    if (st.t_position.defined())
    {
        torch::serialize::OutputArchive ar;
        // Every name NeuralPointCloudCudaImpl registers has to be there: torch::load of that module
        // (src/lib/data/NeuralScene.cpp:349) reads them all and throws on a missing one. t_position, t_index and
        // t_original_color are always registered (src/lib/rendering/NeuralPointCloudCuda.cpp:71-73); an index the bundle
        // does not hold is the identity, colours it does not hold are written as zeros.
        const int64_t n = st.t_position.size(0);
        ar.write("t_position", cpu(st.t_position), false);
        ar.write("t_index", st.t_index.defined() ? cpu(st.t_index) : torch::arange(n, torch::kInt32).reshape({n, 1}), true);
        ar.write("t_original_color", st.t_original_color.defined() ? cpu(st.t_original_color) : torch::zeros({n, 4}), true);
        if (st.t_normal.defined()) ar.write("t_normal", cpu(st.t_normal), true);
        if (st.t_cell_bb_min.defined())
        {
            TORCH_CHECK(st.t_cell_bb_length.defined() && st.t_cell_value.defined() && st.t_cell_access_count.defined(),
                        "SaveSceneCheckpoint: the four cell tensors go together");
            ar.write("t_cell_bb_min", cpu(st.t_cell_bb_min), true);
            ar.write("t_cell_bb_length", cpu(st.t_cell_bb_length), true);
            ar.write("t_cell_value", cpu(st.t_cell_value), true);
            ar.write("t_cell_access_count", cpu(st.t_cell_access_count), true);
        }
        ar.save_to(prefix + "points.pth");
    }
    if (st.texture.defined())
    {
        TORCH_CHECK(st.background_color.defined() && st.confidence_value_of_point.defined(),
                    "SaveSceneCheckpoint: texture, background_color and confidence_value_of_point go together");
        torch::serialize::OutputArchive ar;
        ar.write("texture", cpu(st.texture), false);
        ar.write("background_color", cpu(st.background_color), false);
        ar.write("confidence_value_of_point", cpu(st.confidence_value_of_point), false);
        ar.save_to(prefix + "texture.pth");
    }
    if (st.poses_se3.defined())
    {
        TORCH_CHECK(st.tangent_poses.defined(), "SaveSceneCheckpoint: poses_se3 and tangent_poses go together");
        torch::serialize::OutputArchive ar;
        ar.write("tangent_poses", cpu(st.tangent_poses), false);
        ar.write("poses_se3", cpu(st.poses_se3), true);
        ar.save_to(prefix + "poses.pth");
    }
    if (st.intrinsics.defined())
    {
        torch::serialize::OutputArchive ar;
        ar.write("intrinsics", cpu(st.intrinsics), false);
        ar.save_to(prefix + "intrinsics.pth");
    }
}

namespace
{
inline uint64_t spread_bits21(uint64_t v)
{
    v &= 0x1FFFFFull;
    v = (v | (v << 32)) & 0x1F00000000FFFFull;
    v = (v | (v << 16)) & 0x1F0000FF0000FFull;
    v = (v | (v << 8)) & 0x100F00F00F00F00Full;
    v = (v | (v << 4)) & 0x10C30C30C30C30C3ull;
    v = (v | (v << 2)) & 0x1249249249249249ull;
    return v;
}
}  // namespace

torch::Tensor MortonBlockShuffleOrder(torch::Tensor positions, int64_t block, uint64_t seed)
{
    TORCH_CHECK(positions.dim() == 2 && positions.size(1) >= 3 && !positions.is_cuda() && block >= 1,
                "MortonBlockShuffleOrder: positions is a [N,3] or [N,4] CPU tensor, block >= 1");
    const torch::Tensor p = positions.slice(1, 0, 3).to(torch::kFloat64).contiguous();
    const int64_t n       = p.size(0);
    torch::Tensor out     = torch::empty({n}, torch::kInt64);
    if (n == 0) return out;
    const double* x = p.data_ptr<double>();
    double lo[3], hi[3];
    for (int k = 0; k < 3; ++k) lo[k] = hi[k] = x[k];
    for (int64_t i = 0; i < n; ++i)
        for (int k = 0; k < 3; ++k)
        {
            lo[k] = std::min(lo[k], x[3 * i + k]);
            hi[k] = std::max(hi[k], x[3 * i + k]);
        }
    std::vector<std::pair<uint64_t, int64_t>> keyed((size_t)n);
    for (int64_t i = 0; i < n; ++i)
    {
        uint64_t code = 0;
        for (int k = 0; k < 3; ++k)
        {
            const double ext = std::max(hi[k] - lo[k], 1e-30);
            const uint64_t c = (uint64_t)std::floor((x[3 * i + k] - lo[k]) / ext * (double)((1 << 21) - 1));
            code |= spread_bits21(c) << k;
        }
        keyed[(size_t)i] = {code, i};
    }
    std::stable_sort(keyed.begin(), keyed.end(),
                     [](const std::pair<uint64_t, int64_t>& a, const std::pair<uint64_t, int64_t>& b) { return a.first < b.first; });
    const int64_t blocks = (n + block - 1) / block;
    std::vector<int64_t> block_order((size_t)blocks);
    for (int64_t b = 0; b < blocks; ++b) block_order[(size_t)b] = b;
    std::mt19937_64 gen(seed);
    for (int64_t b = blocks - 1; b > 0; --b)  // Fisher-Yates
    {
        const int64_t j = (int64_t)(gen() % (uint64_t)(b + 1));
        std::swap(block_order[(size_t)b], block_order[(size_t)j]);
    }
    int64_t* o = out.data_ptr<int64_t>();
    int64_t w  = 0;
    for (int64_t b = 0; b < blocks; ++b)
        for (int64_t k = block_order[(size_t)b] * block; k < std::min(n, (block_order[(size_t)b] + 1) * block); ++k)
            o[w++] = keyed[(size_t)k].second;
    return out;
}

torch::Tensor ProcessingOrderOnDevice(const torch::Tensor& positions, int64_t block, uint64_t seed)
{
    TORCH_CHECK(positions.dim() == 2 && positions.size(1) >= 3 && block >= 1,
                "ProcessingOrderOnDevice: positions is a [N,3] or [N,4] tensor, block >= 1");
    torch::NoGradGuard no_grad;
    const int64_t n = positions.size(0);
    auto i32        = torch::TensorOptions().device(positions.device()).dtype(torch::kInt32);
    if (n == 0) return torch::empty({0}, i32);
    const torch::Tensor p   = positions.detach().slice(1, 0, 3).to(torch::kFloat32);
    const torch::Tensor lo  = std::get<0>(p.min(0)), hi = std::get<0>(p.max(0));
    const torch::Tensor ext = (hi - lo).clamp_min(1e-30);
    const torch::Tensor q   = ((p - lo) / ext * (float)((1 << 21) - 1)).floor().to(torch::kInt64);  // [N,3], 21 bits each
    auto spread = [](torch::Tensor x) {  // bit k of x to bit 3 k
        x = x.bitwise_or(x.bitwise_left_shift(32)).bitwise_and((int64_t)0x1f00000000ffffLL);
        x = x.bitwise_or(x.bitwise_left_shift(16)).bitwise_and((int64_t)0x1f0000ff0000ffLL);
        x = x.bitwise_or(x.bitwise_left_shift(8)).bitwise_and((int64_t)0x100f00f00f00f00fLL);
        x = x.bitwise_or(x.bitwise_left_shift(4)).bitwise_and((int64_t)0x10c30c30c30c30c3LL);
        x = x.bitwise_or(x.bitwise_left_shift(2)).bitwise_and((int64_t)0x1249249249249249LL);
        return x;
    };
    const torch::Tensor code = spread(q.select(1, 0))
                                   .bitwise_or(spread(q.select(1, 1)).bitwise_left_shift(1))
                                   .bitwise_or(spread(q.select(1, 2)).bitwise_left_shift(2));
    torch::Tensor order = code.argsort();
    // whole blocks change places; what is left over behind the last whole block stays last, so that every block (a
    // workgroup of the binning pass) remains one run of the curve
    const int64_t blocks = n / block;
    if (blocks > 1)
    {
        auto i64                  = torch::TensorOptions().device(positions.device()).dtype(torch::kInt64);
        auto gen                  = at::detail::createCPUGenerator(seed);
        const torch::Tensor perm  = torch::randperm(blocks, gen, torch::TensorOptions().dtype(torch::kInt64)).to(positions.device());
        const torch::Tensor at    = (perm.unsqueeze(1) * block + torch::arange(block, i64).unsqueeze(0)).reshape({-1});
        order                     = torch::cat({order.index_select(0, at), order.slice(0, blocks * block, n)});
    }
    return order.to(torch::kInt32);
}

void PointRendererCache::PollFragmentCounts()
{
    if (!counts_pending_ || !counts_event_ || !counts_event_->query()) return;
    const int32_t* v = counts_host_.data_ptr<int32_t>();
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l) counts_[l] = l < pending_key_.L ? (float)(v[l + 1] - v[l]) : 0.f;
    counts_key_     = pending_key_;
    counts_valid_   = true;
    counts_pending_ = false;
}

std::vector<float> PointRendererCache::FragmentHistory()
{
    PollFragmentCounts();
    if (!counts_valid_) return {};
    return std::vector<float>(counts_, counts_ + counts_key_.L);
}

void PointRendererCache::ExpectedFragments(float* expected, int64_t N, int L, int w, int h, int render_mode)
{
    PollFragmentCounts();
    CountsKey key;
    key.N = N, key.L = L, key.w = w, key.h = h, key.mode = render_mode;
    if (!(counts_valid_ && counts_key_ == key)) return;  // no history for such calls yet: the caller's own hints stand
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l) expected[l] = l < L ? counts_[l] + 1024.f : 0.f;
}

void PointRendererCache::NoteFragmentCounts(const torch::Tensor& workspace, const vetrast_workspace_layout& lay, int64_t N,
                                            int L, int w, int h, int render_mode)
{
    CountsKey key;
    key.N = N, key.L = L, key.w = w, key.h = h, key.mode = render_mode;
    const bool known = counts_valid_ && counts_key_ == key;
    ++calls_since_readback_;
    if (counts_pending_ || (known && calls_since_readback_ < 16)) return;
    calls_since_readback_ = 0;
    torch::NoGradGuard no_grad;
    const int64_t P = lay.layer_pixel_base[L];
    if (!counts_index_.defined() || !(pending_key_ == key) || counts_index_.device() != workspace.device())
    {
        std::vector<int64_t> at((size_t)VETRAST_MAX_LAYERS + 1, P);
        for (int l = 0; l <= L; ++l) at[(size_t)l] = lay.layer_pixel_base[l];
        counts_index_ = torch::tensor(at, torch::TensorOptions().dtype(torch::kInt64)).to(workspace.device());
    }
    if (!counts_host_.defined())
        counts_host_ = torch::empty({VETRAST_MAX_LAYERS + 1}, torch::TensorOptions().dtype(torch::kInt32).pinned_memory(true));
    // view 0's exclusive scan of the per-pixel counts: the entry at a layer's first pixel is the number of fragments
    // of the layers in front of it
    const torch::Tensor scan = workspace.narrow(0, (int64_t)lay.offsets_base, (P + 1) * 4).view(torch::kInt32);
    counts_host_.copy_(scan.index_select(0, counts_index_), /*non_blocking=*/true);
    if (!counts_event_) counts_event_ = std::make_unique<c10::Event>(c10::DeviceType::CUDA);
    counts_event_->record(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
    pending_key_    = key;
    counts_pending_ = true;
}

const torch::Tensor& PointRendererCache::PointOrderFor(const torch::Tensor& points)
{
    if (point_order_refresh <= 0)
    {
        point_order = torch::Tensor();
        return point_order;
    }
    const bool stale = !point_order.defined() || point_order.size(0) != points.size(0) ||
                       point_order.device() != points.device() || point_order_age_ >= point_order_refresh;
    if (stale)
    {
        point_order      = ProcessingOrderOnDevice(points, 256, 0);
        point_order_age_ = 0;
        // Is the array's own order as good? What the binning pass wants is that the 64 points of a wave lie close
        // together: the summed extent of the runs of 64 points, in array order and in the new order. A cloud in the
        // order of VET's preprocessing passes as it is and the call then goes without the order array (one index
        // read and one position gather per point less, and single-view calls may leave the descriptor rows of points
        // outside the view alone). One blocking read per rebuild, which costs milliseconds anyway.
        torch::NoGradGuard no_grad;
        const int64_t runs = points.size(0) / 64;
        point_order_in_use = true;
        if (runs > 0)
        {
            auto extent = [&](const torch::Tensor& xyz) {
                const torch::Tensor r = xyz.narrow(0, 0, runs * 64).view({runs, 64, 3});
                return (std::get<0>(r.max(1)) - std::get<0>(r.min(1))).sum().item<double>();
            };
            const torch::Tensor xyz = points.detach().narrow(1, 0, 3);
            const double as_is      = extent(xyz);
            const double ordered    = extent(xyz.index_select(0, point_order.to(torch::kInt64)));
            // (blocks whose points VET has sorted by radius come out at 0.5 to 0.6 and are faster as they are; a
            // cloud with a fifth of its points appended unsorted at 0.22, the generator's order at 0.33)
            point_order_in_use      = ordered < 0.4 * as_is;
        }
    }
    ++point_order_age_;
    return point_order_in_use ? point_order : no_point_order_;
}

torch::Tensor SortBlocksByRadiusOrder(torch::Tensor radius, int64_t block)
{
    TORCH_CHECK(radius.dim() == 1 && !radius.is_cuda() && block >= 1, "SortBlocksByRadiusOrder: radius is a [N] CPU tensor");
    const torch::Tensor r = radius.to(torch::kFloat32).contiguous();
    const int64_t n       = r.size(0);
    const float* rv       = r.data_ptr<float>();
    torch::Tensor out     = torch::arange(n, torch::kInt64);
    int64_t* o            = out.data_ptr<int64_t>();
    // complete blocks only: n_blocks = NumVertices() / block_size, src/lib/data/SceneData.cpp:1007
    for (int64_t b = 0; b < n / block; ++b)
        std::stable_sort(o + b * block, o + (b + 1) * block, [rv](int64_t i1, int64_t i2) { return rv[i1] < rv[i2]; });
    return out;
}

torch::Tensor ScenePreprocessOrder(torch::Tensor positions_radius, int64_t block, uint64_t seed)
{
    TORCH_CHECK(positions_radius.dim() == 2 && positions_radius.size(1) == 4 && !positions_radius.is_cuda(),
                "ScenePreprocessOrder: positions_radius is a [N,4] CPU tensor (x, y, z, drop-out radius)");
    const torch::Tensor first  = MortonBlockShuffleOrder(positions_radius, block, seed);
    const torch::Tensor radius = positions_radius.select(1, 3).index_select(0, first);
    return first.index_select(0, SortBlocksByRadiusOrder(radius, block));
}
}  // namespace vet_amd

// ---- Python binding used by the tests: builds a NeuralRenderInfo from plain arguments and calls BlendPointCloud ----
namespace
{
std::shared_ptr<vet_amd::PointRendererCache> g_cache;

std::vector<torch::Tensor> blend_point_cloud(torch::Tensor texture, torch::Tensor background_color, torch::Tensor points,
                                             torch::Tensor pose_tangents, torch::Tensor intrinsics,
                                             torch::Tensor confidence, torch::Tensor poses_se3, torch::Tensor t_index,
                                             std::vector<std::vector<double>> views, int num_layers, bool train,
                                             pybind11::dict params, pybind11::object environment)
{
    using namespace vet_amd;
    if (!g_cache) g_cache = std::make_shared<PointRendererCache>();
    SceneTensors scene;
    scene.texture                   = texture;
    scene.background_color          = background_color;
    scene.t_position                = points;
    scene.tangent_poses             = pose_tangents;
    scene.intrinsics                = intrinsics;
    scene.confidence_value_of_point = confidence;
    scene.dynamic_refinement_t      = torch::zeros({1}, points.options());
    scene.poses_se3                 = poses_se3;
    if (t_index.defined() && t_index.numel() > 0) scene.t_index = t_index;

    NeuralRenderInfo nri;
    nri.scene      = &scene;
    nri.num_layers = num_layers;
    nri.train      = train;
    nri.cache      = g_cache.get();
    for (auto& v : views)
    {
        TORCH_CHECK(v.size() == 14, "a view is (w, h, image_index, camera_index, camera_model, crop[5], rot[4])");
        ReducedImageInfo r;
        r.w                 = (int)v[0];
        r.h                 = (int)v[1];
        r.image_index       = (int)v[2];
        r.camera_index      = (int)v[3];
        r.camera_model_type = (int)v[4];
        for (int j = 0; j < 5; ++j) r.crop_transform[j] = (float)v[5 + j];
        for (int j = 0; j < 4; ++j) r.crop_rotation[j] = (float)v[10 + j];
        nri.images.push_back(r);
    }
    RenderParams& p = nri.params;
    p.dropout       = 0.f;
    bool super_sampling = false, cat_masks_to_color = false, cat_env_to_color = false, no_envmap_at_points = true;
    for (auto item : params)
    {
        const std::string k = pybind11::cast<std::string>(item.first);
        auto as_d           = [&] { return pybind11::cast<double>(item.second); };
        if (k == "dropout") p.dropout = (float)as_d();
        else if (k == "drop_out_radius_threshold") p.drop_out_radius_threshold = (float)as_d();
        else if (k == "drop_out_points_by_radius") p.drop_out_points_by_radius = as_d() != 0;
        else if (k == "output_background_mask") p.output_background_mask = as_d() != 0;
        else if (k == "output_background_mask_value") p.output_background_mask_value = (float)as_d();
        else if (k == "stability_cutoff_value") p.stability_cutoff_value = (float)as_d();
        else if (k == "need_point_gradient") p.need_point_gradient = as_d() != 0;
        else if (k == "use_environment_map") p.use_environment_map = as_d() != 0;
        else if (k == "viewer_only") p.viewer_only = as_d() != 0;
        else if (k == "debug_max_list_length") p.debug_max_list_length = (int)as_d();
        else if (k == "quirk_background_confidence_leak") p.quirk_background_confidence_leak = as_d() != 0;
        else if (k == "point_gradient_normalization") p.point_gradient_normalization = (int)as_d();
        else if (k == "render_mode") p.render_mode = (int)as_d();
        else if (k == "depth_accept_blend") p.depth_accept_blend = (float)as_d();
        else if (k == "size_bins_from_history") p.size_bins_from_history = as_d() != 0.0;
        else if (k == "expected_fragments")
        {
            auto v = item.second.cast<std::vector<double>>();
            for (size_t l = 0; l < v.size() && l < (size_t)VETRAST_MAX_LAYERS; ++l) p.expected_fragments[l] = (float)v[l];
        }
        else if (k == "K_gradient_factor") p.K_gradient_factor = (float)as_d();
        else if (k == "distortion_gradient_factor") p.distortion_gradient_factor = (float)as_d();
        else if (k == "allow_distortion") p.allow_distortion = as_d() != 0.0;
        else if (k == "camera_gradient_normalization") p.camera_gradient_normalization = as_d() != 0;
        else if (k == "fused_confidence_scale") p.fused_confidence_scale = (float)as_d();
        else if (k == "fused_texture_abs") p.fused_texture_abs = as_d() != 0;
        else if (k == "add_depth_to_network") p.add_depth_to_network = as_d() != 0;
        else if (k == "dist_cutoff") p.dist_cutoff = (float)as_d();
        else if (k == "super_sampling") super_sampling = as_d() != 0;
        else if (k == "cat_masks_to_color") cat_masks_to_color = as_d() != 0;
        else if (k == "cat_env_to_color") cat_env_to_color = as_d() != 0;
        else if (k == "no_envmap_at_points") no_envmap_at_points = as_d() != 0;
        else TORCH_CHECK(false, "unknown RenderParams field ", k);
    }
    if (super_sampling || cat_masks_to_color || p.add_depth_to_network || !environment.is_none())
    {
        // through the caller glue of the reference (PointRenderModuleImpl::forward): images, then masks
        PointRenderModule module;
        module.cache              = g_cache;
        module.super_sampling     = super_sampling;
        module.cat_masks_to_color = cat_masks_to_color;
        module.cat_env_to_color    = cat_env_to_color;
        module.no_envmap_at_points = no_envmap_at_points;
        if (!environment.is_none())
            module.environment_map = [environment](const std::vector<std::vector<torch::Tensor>>& layers, NeuralRenderInfo*) {
                return pybind11::cast<std::vector<torch::Tensor>>(environment(layers));
            };
        auto result               = module.forward(&nri);
        std::vector<torch::Tensor> out = result.first;
        out.insert(out.end(), result.second.begin(), result.second.end());
        return out;
    }
    // the scene bundle only has to live for the duration of apply(): everything backward needs is saved in the graph
    return BlendPointCloud(&nri);
}
}  // namespace

namespace vet_amd
{
MyAdam::MyAdam(std::vector<Group> groups, double beta1, double beta2, double eps, double weight_decay)
    : groups_(std::move(groups)), beta1_(beta1), beta2_(beta2), eps_(eps), weight_decay_(weight_decay),
      cache_(std::make_unique<PointRendererCache>())
{
    state_.resize(groups_.size());
    for (size_t g = 0; g < groups_.size(); ++g) state_[g].resize(groups_[g].params.size());
}

void MyAdam::step(bool zero_grad)
{
    torch::NoGradGuard no_grad;
    for (size_t g = 0; g < groups_.size(); ++g)
        for (size_t k = 0; k < groups_[g].params.size(); ++k)
        {
            torch::Tensor& p = groups_[g].params[k];
            if (!p.grad().defined()) continue;  // my_adam.cpp:38-41
            torch::Tensor grad = p.grad();
            TORCH_CHECK(p.is_cuda() && p.scalar_type() == torch::kFloat32 && p.is_contiguous() && grad.is_contiguous() &&
                            grad.scalar_type() == torch::kFloat32,
                        "MyAdam: parameters and gradients must be contiguous float32 tensors on the GPU");
            State& st = state_[g][k];
            if (!st.exp_avg.defined() || st.exp_avg.numel() != p.numel())  // state initialisation, my_adam.cpp:48-62
            {
                st.exp_avg    = torch::zeros_like(p);
                st.exp_avg_sq = torch::zeros_like(p);
                st.step       = 0;
            }
            st.step += 1;
            vetrast_adam_args a;
            std::memset(&a, 0, sizeof(a));
            a.param        = p.data_ptr<float>();
            a.grad         = grad.data_ptr<float>();
            a.exp_avg      = st.exp_avg.data_ptr<float>();
            a.exp_avg_sq   = st.exp_avg_sq.data_ptr<float>();
            a.n            = p.numel();
            a.step         = st.step;
            a.lr           = groups_[g].lr;
            a.beta1        = beta1_;
            a.beta2        = beta2_;
            a.eps          = eps_;
            a.weight_decay = weight_decay_;
            a.zero_grad    = zero_grad ? 1 : 0;
            check_status(vetrast_adam_step(cache_->ctx, &a, c10::hip::getCurrentHIPStream().stream()), "adam_step");
            // the kernel wrote through raw pointers: tell everyone who keys on the version counters
            p.unsafeGetTensorImpl()->bump_version();
            if (zero_grad) grad.unsafeGetTensorImpl()->bump_version();
        }
}

void MyAdam::zero_grad()
{
    for (auto& g : groups_)
        for (auto& p : g.params)
            if (p.grad().defined()) p.mutable_grad().zero_();
}
}  // namespace vet_amd

// ---- self test of vet_adapter.h ------------------------------------------------------------------------------------
// Stand-ins with the member names and spellings of the reference's types (module holders with operator->, an
// Eigen-style operator()(row, col), an enum class for the camera model, bool / int / float members of RenderParams under
// the reference's names and defaults), so that the adapter's templates are compiled and run without VET's headers.
namespace reference_stand_ins
{
enum class CameraModel : int { PINHOLE_DISTORTION = 0, OCAM = 1, SPHERICAL = 2 };
struct IntrinsicsPinholef { float fx = 1, fy = 1, cx = 0, cy = 0, s = 0; };
struct Mat2f
{
    float m[4] = {1, 0, 0, 1};  // column-major, as Eigen stores it
    float operator()(int r, int c) const { return m[c * 2 + r]; }
};
struct ReducedImageInfo
{
    int w = 0, h = 0;
    int image_index  = -1;
    int camera_index = -1;
    CameraModel camera_model_type = CameraModel::PINHOLE_DISTORTION;
    IntrinsicsPinholef crop_transform;
    Mat2f crop_rotation;
};
struct RenderParams  // src/lib/data/Settings.h:19-93, the members the adapter reads
{
    bool check_normal = false;
    float dropout = 0.25, depth_accept_blend = 0.01;
    float drop_out_radius_threshold = 0.6;
    bool drop_out_points_by_radius  = true;
    float distortion_gradient_factor = 0.005, K_gradient_factor = 0.5;
    int num_texture_channels = -1;
    float dist_cutoff = 20.f;
    bool output_background_mask = false;
    float output_background_mask_value = 0;
    bool add_depth_to_network = false;
    float stability_cutoff_value = 10000.f;
    bool need_point_gradient = true, use_environment_map = true;
    int render_mode = 1;
    bool viewer_only = false;
    int debug_max_list_length = -1;
};
struct TextureImpl { torch::Tensor texture, background_color, confidence_value_of_point; };
struct PointCloudImpl { torch::Tensor t_position, t_index, t_original_color, t_normal; };
struct PosesImpl { torch::Tensor tangent_poses, poses_se3; };
struct IntrinsicsImpl { torch::Tensor intrinsics; };
struct NeuralScene
{
    std::shared_ptr<PointCloudImpl> point_cloud_cuda = std::make_shared<PointCloudImpl>();
    std::shared_ptr<TextureImpl> texture             = std::make_shared<TextureImpl>();
    std::shared_ptr<PosesImpl> poses                 = std::make_shared<PosesImpl>();
    std::shared_ptr<IntrinsicsImpl> intrinsics       = std::make_shared<IntrinsicsImpl>();
    torch::Tensor dynamic_refinement_t;
};
struct NeuralRenderInfo
{
    NeuralScene* scene = nullptr;
    std::vector<ReducedImageInfo> images;
    RenderParams params;
    int num_layers = 1;
    bool train = false;
    int current_epoch = 0;
    void* timer_system = nullptr;
    void* cache = nullptr;
};
}  // namespace reference_stand_ins

// Renders through vet_adapter.h from stand-ins filled with the given tensors; `views` as for blend_point_cloud. The
// caller compares the result with blend_point_cloud's for the same input.
std::vector<torch::Tensor> adapter_selftest(torch::Tensor texture, torch::Tensor background_color, torch::Tensor points,
                                            torch::Tensor pose_tangents, torch::Tensor intrinsics, torch::Tensor confidence,
                                            torch::Tensor poses_se3, std::vector<std::vector<double>> views, int num_layers,
                                            int render_mode, int max_list_length, bool output_background_mask)
{
    namespace ref = reference_stand_ins;
    if (!g_cache) g_cache = std::make_shared<vet_amd::PointRendererCache>();
    ref::NeuralScene scene;
    scene.texture->texture                   = texture;
    scene.texture->background_color          = background_color;
    scene.texture->confidence_value_of_point = confidence;
    scene.point_cloud_cuda->t_position       = points;
    scene.poses->tangent_poses               = pose_tangents;
    scene.poses->poses_se3                   = poses_se3;
    scene.intrinsics->intrinsics             = intrinsics;
    scene.dynamic_refinement_t               = torch::zeros({1}, points.options());
    ref::NeuralRenderInfo info;
    info.scene      = &scene;
    info.num_layers = num_layers;
    info.train      = false;
    for (auto& v : views)
    {
        TORCH_CHECK(v.size() == 14, "a view is (w, h, image_index, camera_index, camera_model, crop[5], rot[4])");
        ref::ReducedImageInfo r;
        r.w = (int)v[0], r.h = (int)v[1], r.image_index = (int)v[2], r.camera_index = (int)v[3];
        r.camera_model_type = static_cast<ref::CameraModel>((int)v[4]);
        r.crop_transform.fx = (float)v[5], r.crop_transform.fy = (float)v[6], r.crop_transform.cx = (float)v[7];
        r.crop_transform.cy = (float)v[8], r.crop_transform.s = (float)v[9];
        // row-major in `views`, column-major in the stand-in, as in Eigen
        r.crop_rotation.m[0] = (float)v[10], r.crop_rotation.m[2] = (float)v[11];
        r.crop_rotation.m[1] = (float)v[12], r.crop_rotation.m[3] = (float)v[13];
        info.images.push_back(r);
    }
    info.params.dropout                = 0.f;
    info.params.num_texture_channels   = (int)texture.size(0);
    info.params.use_environment_map    = false;
    info.params.render_mode            = render_mode;
    info.params.debug_max_list_length  = max_list_length;
    info.params.output_background_mask = output_background_mask;
    vet_amd::SceneTensors bundle;
    return vet_amd::BlendPointCloudOf(&info, g_cache.get(), &bundle);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    pybind11::class_<vet_amd::MyAdam>(m, "MyAdam")
        .def(pybind11::init([](std::vector<std::pair<std::vector<torch::Tensor>, double>> groups, double beta1,
                               double beta2, double eps, double weight_decay) {
                 std::vector<vet_amd::MyAdam::Group> gs;
                 for (auto& g : groups) gs.push_back({g.first, g.second});
                 return std::make_unique<vet_amd::MyAdam>(std::move(gs), beta1, beta2, eps, weight_decay);
             }),
             pybind11::arg("groups"), pybind11::arg("beta1") = 0.9, pybind11::arg("beta2") = 0.999,
             pybind11::arg("eps") = 1e-8, pybind11::arg("weight_decay") = 0.0)
        .def("step", &vet_amd::MyAdam::step, pybind11::arg("zero_grad") = false)
        .def("zero_grad", &vet_amd::MyAdam::zero_grad);
    m.def(
        "fill_scene_grid_with_loss",
        [](int batch, torch::Tensor bb_min, torch::Tensor bb_length, torch::Tensor value, torch::Tensor access_count,
           std::vector<std::vector<double>> views, torch::Tensor poses_se3, torch::Tensor intrinsics,
           torch::Tensor loss_img) {
            if (!g_cache) g_cache = std::make_shared<vet_amd::PointRendererCache>();
            std::vector<vet_amd::ReducedImageInfo> images;
            for (auto& v : views)
            {
                TORCH_CHECK(v.size() == 14, "a view is w,h,image_index,camera_index,camera_model_type,crop[5],rot[4]");
                vet_amd::ReducedImageInfo r;
                r.w                 = (int)v[0];
                r.h                 = (int)v[1];
                r.image_index       = (int)v[2];
                r.camera_index      = (int)v[3];
                r.camera_model_type = (int)v[4];
                for (int j = 0; j < 5; ++j) r.crop_transform[j] = (float)v[5 + j];
                for (int j = 0; j < 4; ++j) r.crop_rotation[j] = (float)v[10 + j];
                images.push_back(r);
            }
            g_cache->FillSceneGridWithLoss(batch, {bb_min, bb_length, value, access_count}, images, poses_se3,
                                           intrinsics, loss_img);
        },
        "PointRendererCache::FillSceneGridWithLoss of the reference, with the cell tensors passed one by one");
    m.def(
        "save_scene_checkpoint",
        [](const std::string& prefix, pybind11::dict tensors) {
            vet_amd::SceneTensors st;
            for (auto item : tensors)
            {
                const std::string k = pybind11::cast<std::string>(item.first);
                torch::Tensor t     = pybind11::cast<torch::Tensor>(item.second);
                if (k == "texture") st.texture = t;
                else if (k == "background_color") st.background_color = t;
                else if (k == "confidence_value_of_point") st.confidence_value_of_point = t;
                else if (k == "t_position") st.t_position = t;
                else if (k == "t_index") st.t_index = t;
                else if (k == "tangent_poses") st.tangent_poses = t;
                else if (k == "poses_se3") st.poses_se3 = t;
                else if (k == "intrinsics") st.intrinsics = t;
                else if (k == "t_original_color") st.t_original_color = t;
                else if (k == "t_normal") st.t_normal = t;
                else if (k == "t_cell_bb_min") st.t_cell_bb_min = t;
                else if (k == "t_cell_bb_length") st.t_cell_bb_length = t;
                else if (k == "t_cell_value") st.t_cell_value = t;
                else if (k == "t_cell_access_count") st.t_cell_access_count = t;
                else TORCH_CHECK(false, "unknown scene tensor ", k);
            }
            vet_amd::SaveSceneCheckpoint(prefix, st);
        },
        "NeuralScene::SaveCheckpoint of the reference for the tensors the rasterizer reads");
    m.def(
        "load_scene_checkpoint",
        [](const std::string& prefix) {
            const vet_amd::SceneTensors st = vet_amd::LoadSceneCheckpoint(prefix, torch::kCPU);
            pybind11::dict d;
            auto put = [&](const char* k, const torch::Tensor& t) {
                if (t.defined()) d[k] = t;
            };
            put("texture", st.texture);
            put("background_color", st.background_color);
            put("confidence_value_of_point", st.confidence_value_of_point);
            put("t_position", st.t_position);
            put("t_index", st.t_index);
            put("tangent_poses", st.tangent_poses);
            put("poses_se3", st.poses_se3);
            put("intrinsics", st.intrinsics);
            put("t_original_color", st.t_original_color);
            put("t_normal", st.t_normal);
            put("t_cell_bb_min", st.t_cell_bb_min);
            put("t_cell_bb_length", st.t_cell_bb_length);
            put("t_cell_value", st.t_cell_value);
            put("t_cell_access_count", st.t_cell_access_count);
            return d;
        },
        "NeuralScene::LoadCheckpoint of the reference for the tensors the rasterizer reads");
    m.def("morton_block_shuffle_order", &vet_amd::MortonBlockShuffleOrder, pybind11::arg("positions"),
          pybind11::arg("block") = 256, pybind11::arg("seed") = 0,
          "ReorderMorton64 + RandomBlockShuffle(block) of the reference's scene preprocessing, as a permutation");
    m.def("sort_blocks_by_radius_order", &vet_amd::SortBlocksByRadiusOrder, pybind11::arg("radius"), pybind11::arg("block") = 256,
          "SceneData::SortBlocksByRadius(block) of the reference's scene preprocessing, as a permutation");
    m.def("scene_preprocess_order", &vet_amd::ScenePreprocessOrder, pybind11::arg("positions_radius"),
          pybind11::arg("block") = 256, pybind11::arg("seed") = 0,
          "ReorderMorton64 + RandomBlockShuffle + SortBlocksByRadius of the reference's scene preprocessing, as a permutation");
    m.def("processing_order_on_device", &vet_amd::ProcessingOrderOnDevice, pybind11::arg("positions"),
          pybind11::arg("block") = 256, pybind11::arg("seed") = 0,
          "Morton order with shuffled blocks, computed on the positions' device: int32 permutation for point_order");
    m.def(
        "set_point_order_refresh",
        [](int64_t every) {
            if (!g_cache) g_cache = std::make_shared<vet_amd::PointRendererCache>();
            g_cache->point_order_refresh = every;
            g_cache->point_order         = torch::Tensor();
        },
        "forward calls between rebuilds of the cache's processing order; 0 switches it off");
    m.def(
        "fragment_history", []() { return g_cache ? g_cache->FragmentHistory() : std::vector<float>(); },
        "fragments per layer one view of a recent call left, as read back by the cache (empty: none yet)");
    m.def(
        "point_order",
        []() { return (g_cache && g_cache->point_order.defined()) ? g_cache->point_order : torch::Tensor(); },
        "the processing order the cache currently holds (undefined tensor: none)");
    m.def(
        "point_order_in_use", []() { return g_cache && g_cache->point_order.defined() && g_cache->point_order_in_use; },
        "whether forward calls are handed the cache's processing order (false: the array's own order is as good)");
    m.def(
        "kept_descriptor_calls", []() { return g_cache ? g_cache->calls_with_kept_descriptors : (int64_t)0; },
        "forward calls of the binding's cache so far that read descriptor records kept from an earlier call");
    m.def(
        "set_keep_packed_descriptors",
        [](bool keep) {
            if (!g_cache) g_cache = std::make_shared<vet_amd::PointRendererCache>();
            g_cache->keep_packed_descriptors = keep;
        },
        "whether the binding's cache keeps descriptor records across calls while texture and confidence stay unchanged");
    m.def(
        "train_workspace_info",
        []() {
            pybind11::dict d;
            d["defined"] = g_cache && g_cache->train_workspace.defined();
            d["data_ptr"] = (g_cache && g_cache->train_workspace.defined()) ? (int64_t)(intptr_t)g_cache->train_workspace.data_ptr() : (int64_t)0;
            d["bytes"]    = (g_cache && g_cache->train_workspace.defined()) ? g_cache->train_workspace.numel() : (int64_t)0;
            return d;
        },
        "address and size of the workspace the binding's cache keeps for training steps (for the tests)");
    m.def("adapter_selftest", &adapter_selftest, pybind11::arg("texture"), pybind11::arg("background_color"),
          pybind11::arg("points"), pybind11::arg("pose_tangents"), pybind11::arg("intrinsics"), pybind11::arg("confidence"),
          pybind11::arg("poses_se3"), pybind11::arg("views"), pybind11::arg("num_layers"), pybind11::arg("render_mode") = 1,
          pybind11::arg("max_list_length") = -1, pybind11::arg("output_background_mask") = false,
          "renders through vet_adapter.h from stand-ins that have the member names of the reference's types");
    m.def("blend_point_cloud", &blend_point_cloud, pybind11::arg("texture"), pybind11::arg("background_color"),
          pybind11::arg("points"), pybind11::arg("pose_tangents"), pybind11::arg("intrinsics"), pybind11::arg("confidence"),
          pybind11::arg("poses_se3"), pybind11::arg("t_index"), pybind11::arg("views"), pybind11::arg("num_layers"),
          pybind11::arg("train"), pybind11::arg("params"), pybind11::arg("environment") = pybind11::none(),
          "BlendPointCloud(NeuralRenderInfo*) of the reference, with the scene passed as tensors; `environment`, a "
          "callable (layers[l][b] weight tensors) -> L tensors, routes the call through the render module's "
          "environment-map branch");
}
