// libtorch host side of the MI355X blending point rasterizer.
//
// Mirrors the reference's seam so that VET's pipeline can call it unchanged in spirit:
//   std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info)        src/lib/rendering/PointRenderer.h:53
//   struct PointRender : torch::autograd::Function<PointRender>              src/lib/rendering/PointRenderer.h:39-47
//   class NeuralRenderInfo : torch::CustomClassHolder                         src/lib/rendering/PointRenderer.h:23-34
// Argument order, output list and the seven returned gradients are the reference's (src/lib/rendering/RenderInfo.cpp:18-67,
// src/lib/rendering/PointRenderer.cu:1061-1068,1319-1322). All arithmetic happens behind the C ABI of include/vetrast.h.
#pragma once
#include <torch/torch.h>

#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "../../include/vetrast.h"

namespace vet_amd
{
// ReducedImageInfo (src/lib/data/SceneData.h:39-50) is the ABI's vetrast_view.
using ReducedImageInfo = vetrast_view;

// The RenderParams members the blending path reads (src/lib/data/Settings.h:19-93), same names and defaults.
struct RenderParams
{
    bool check_normal                  = false;
    float dropout                      = 0.25f;
    float drop_out_radius_threshold    = 0.6f;
    float K_gradient_factor            = 0.5f;
    float distortion_gradient_factor   = 0.005f;  // src/lib/data/Settings.h:54
    // Not in the reference: cameras with non-zero distortion coefficients are refused unless this is set; with it they
    // are rendered with the published 8-coefficient rational model (vetrast_params.allow_distortion; parity with
    // saiga's distortNormalizedPoint unpinned, dist_cutoff not applied).
    bool allow_distortion              = false;
    bool drop_out_points_by_radius     = true;
    int num_texture_channels           = -1;
    bool output_background_mask        = false;
    float output_background_mask_value = 0.f;
    bool add_depth_to_network          = false;  // the blend modes leave the depth images at zero, as the reference does
    float dist_cutoff                  = 20.f;   // accepted and ignored: it only steers saiga's distortion model, and
                                                 // cameras with non-zero distortion coefficients are refused
    float stability_cutoff_value       = 10000.f;
    bool need_point_gradient           = true;
    bool use_environment_map           = true;
    int render_mode                    = 1;  // 1 = FULL_BLEND, 2 = FUZZY_BLEND, 3 = BILINEAR_BLEND; mode 0 is not implemented
    float depth_accept_blend           = 0.01f;  // FUZZY_BLEND: depth range of a bucket
    // Not in the reference. Hints for speed only (vetrast_params.expected_fragments): how many fragments one view is
    // expected to leave in every layer, for sizing the pixel bins (0: every point lands in the layer, which is far too
    // many for a 512x512 training crop or a layer most points drop out of by radius). With size_bins_from_history the
    // cache fills the array from the fragment counts of earlier calls with the same image size, read back without
    // blocking every few calls. Results do not depend on either.
    bool size_bins_from_history        = true;
    float expected_fragments[VETRAST_MAX_LAYERS] = {0.f, 0.f, 0.f, 0.f, 0.f};
    bool viewer_only                   = false;
    int debug_max_list_length          = -1;
    // Switches for two accidents of the reference implementation; the defaults reproduce it literally.
    bool quirk_background_confidence_leak = true;   // src/lib/rendering/RenderBackward.cu:1157
    int point_gradient_normalization      = 2;      // src/lib/rendering/PointRenderer.cu:1278-1279
    bool camera_gradient_normalization    = true;   // src/lib/rendering/PointRenderer.cu:1253-1308
    // The two steps Pipeline.cpp:113-124 runs on the optimised tensors right before rendering, fused into the rasterizer
    // when switched on; `texture`, `background_color` and `confidence` passed to BlendPointCloud are then the RAW tensors
    // (texture_raw, background_color_raw, confidence_raw) and autograd returns the gradients of those.
    float fused_confidence_scale = 0.f;  // > 0: confidence = sigmoid(scale * raw), scale = 10 + narrowing * epoch
    bool fused_texture_abs       = false;  // texture = |raw|, background = |raw| (non_subzero_texture)
};

// The tensors BlendPointCloud reads through info->scene (src/lib/rendering/RenderInfo.cpp:25-29 and
// src/lib/data/NeuralScene.h:101-113): a plain bundle instead of the NeuralScene object.
struct SceneTensors
{
    torch::Tensor texture;                    // scene->texture->texture                    [C,N] f32
    torch::Tensor background_color;           // scene->texture->background_color           [C]   f32
    torch::Tensor t_position;                 // scene->point_cloud_cuda->t_position        [N,4] f32
    torch::Tensor tangent_poses;              // scene->poses->tangent_poses                [F,6] f64
    torch::Tensor intrinsics;                 // scene->intrinsics->intrinsics              [Ncam,13] f32
    torch::Tensor confidence_value_of_point;  // scene->texture->confidence_value_of_point  [1,N] f32
    torch::Tensor dynamic_refinement_t;       // scene->dynamic_refinement_t                [1] dummy
    torch::Tensor poses_se3;                  // scene->poses->poses_se3                    [F,8] f64
    torch::Tensor t_index;                    // scene->point_cloud_cuda->t_index           [N,1] i32, may be undefined
    // Entries of the reference's point cloud module that the rasterizer does not read; kept so that a checkpoint that is
    // loaded and saved again still holds every tensor NeuralPointCloudCudaImpl registers
    // (src/lib/rendering/NeuralPointCloudCuda.cpp:53,71-73,84-87).
    torch::Tensor t_original_color;           // buffer [N,4] f32, always registered by the reference
    torch::Tensor t_normal;                   // buffer [N,1] i32 (10-bit packed), only with normals
    torch::Tensor t_cell_bb_min, t_cell_bb_length, t_cell_value, t_cell_access_count;  // buffers, only with use_grid_loss
};

// The cell tensors of the point cloud (src/lib/rendering/NeuralPointCloudCuda.h:100-106).
struct CellTensors
{
    torch::Tensor t_cell_bb_min;        // [n,3] f32
    torch::Tensor t_cell_bb_length;     // [n,3] f32
    torch::Tensor t_cell_value;         // [n,1] f32
    torch::Tensor t_cell_access_count;  // [n,1] i32
};

// Owns the vetrast context and the workspace that is re-used between no-grad calls
// (counterpart of PointRendererCache, src/lib/rendering/PointRenderer.h:112-248).
class PointRendererCache
{
   public:
    PointRendererCache();
    ~PointRendererCache();
    PointRendererCache(const PointRendererCache&)            = delete;
    PointRendererCache& operator=(const PointRendererCache&) = delete;
    vetrast_ctx* ctx = nullptr;
    torch::Tensor eval_workspace;
    // The workspace of the last forward call that was saved for a backward pass. The next such call takes it again if
    // nothing but this cache still holds it (the graph of that step has been released) and it is large enough: a
    // training loop then runs in one workspace instead of allocating one per step.
    torch::Tensor train_workspace;
    // Cameras with non-zero distortion coefficients are refused unless RenderParams::allow_distortion is set. The
    // coefficients sit in device memory. The first call for an intrinsics tensor (its memory and size) reads columns
    // 5..12 of `intrinsics` [num_cameras,13] back, which blocks, and throws if they are not all zero. Later calls never
    // block: when the tensor's version counter has moved (an optimiser step), and every 64th call whatever the counter
    // says (writes through a raw pointer leave it alone), NoteDeviceFlags copies the status word that the forward call
    // raises on the device to pinned memory behind the call, and the next call that finds the copy landed throws.
    void CheckIntrinsics(const torch::Tensor& intrinsics);
    void NoteDeviceFlags(const torch::Tensor& workspace, const vetrast_workspace_layout& lay);
    // The order in which the binning pass walks the points (vetrast_forward_args.point_order): Morton order with shuffled
    // 256-point blocks, built on the device from the positions, rebuilt when the number of points changes and every
    // `point_order_refresh` forward calls (positions drift while they are optimised; the order only has to be roughly
    // right). Results do not depend on it; a cloud that has grown since it was preprocessed (NeuralScene::AddNewPoints
    // appends, src/lib/data/NeuralScene.cpp:1013) or that comes in file order renders up to twice as fast in the
    // binning pass with it, one in VET's order loses nothing. 0: never build one, walk the array as it is.
    int64_t point_order_refresh = 1000;
    torch::Tensor point_order;  // int32 [N] on the points' device, or undefined
    // false: the array's own order keeps the 64 points of a wave as close together as the built order would (checked
    // at every rebuild), and calls go without an order array
    bool point_order_in_use = true;
    const torch::Tensor& PointOrderFor(const torch::Tensor& points);
    // Descriptor records kept across calls (vetrast_forward_args.packed_descriptors), for forward calls that no
    // backward pass follows. Such a call that finds texture and confidence as the one before left them (same storage,
    // same version counters, same activation settings) packs them once with vetrast_pack_descriptors; the calls after
    // it read those records, until one of the tensors changes: a viewer or an evaluation loop renders a scene many
    // times between changes. Calls that are saved for a backward pass always interleave inside the call (that also
    // warms the cache for the backward pass's gathers, which is worth more than the interleave costs). Writers that
    // go around the version counter must bump it (vet_amd::MyAdam does). false: never keep records.
    bool keep_packed_descriptors = true;
    torch::Tensor KeptDescriptorsFor(const torch::Tensor& texture, const torch::Tensor& confidence,
                                     const vetrast_params& params);
    int64_t calls_with_kept_descriptors = 0;  // forward calls so far that read kept records
    // Fragments per layer that a view of recent calls left, for RenderParams::expected_fragments: every 16th forward
    // call copies the layer boundaries of view 0's scan to pinned host memory without blocking; the numbers are taken
    // up by a later call once the copy has landed. Kept per image size, layer count, point count and render mode.
    void ExpectedFragments(float* expected, int64_t N, int L, int w, int h, int render_mode);
    void NoteFragmentCounts(const torch::Tensor& workspace, const vetrast_workspace_layout& lay, int64_t N, int L, int w,
                            int h, int render_mode);
    // what ExpectedFragments would work from right now (empty: nothing has been read back yet)
    std::vector<float> FragmentHistory();
    // layers_cuda[l].weight of the reference's cache (src/lib/rendering/PointRenderer.h:131, written at
    // src/lib/rendering/RenderForward.cu:1355-1356): per layer [B,1,h_l,w_l], the transmittance left behind the last
    // blended fragment of every pixel. Only kept up to date by BlendPointCloud while keep_layer_weights is set.
    bool keep_layer_weights = false;
    std::vector<torch::Tensor> layer_weights;

    // Adds the error image of view `batch` to the cells its pixels fall in
    // (PointRendererCache::FillSceneGridWithLoss(int batch, NeuralPointCloudCuda point_cloud, std::vector<ReducedImageInfo>
    // images, torch::Tensor loss_img), src/lib/rendering/PointRenderer.h:175, src/lib/rendering/RenderForward.cu:763-791).
    // The point cloud object is replaced by its four cell tensors and the pose / intrinsics tables the reference reads
    // from device constants are passed along. cells.value and cells.access_count are updated in place.
    void FillSceneGridWithLoss(int batch, const CellTensors& cells, const std::vector<ReducedImageInfo>& images,
                               torch::Tensor poses_se3, torch::Tensor intrinsics, torch::Tensor loss_img);
    torch::Tensor lift_workspace;

   private:
    // the storage is held weakly: while it is, no other tensor's memory can pass for it at the same address
    const void* checked_intrinsics_ptr_ = nullptr;
    c10::weak_intrusive_ptr<c10::StorageImpl> checked_intrinsics_storage_{c10::intrusive_ptr<c10::StorageImpl>()};
    int64_t checked_intrinsics_version_ = -1, checked_intrinsics_numel_ = -1;
    bool flags_wanted_ = false, flags_pending_ = false;
    int64_t calls_since_flags_ = 0;
    torch::Tensor flags_host_;
    std::unique_ptr<c10::Event> flags_event_;
    void PollDeviceFlags();
    int64_t point_order_age_ = 0;
    torch::Tensor no_point_order_;  // stays undefined
    struct PackKey
    {
        const void *texture = nullptr, *confidence = nullptr;
        const void *texture_storage = nullptr, *confidence_storage = nullptr;
        int64_t texture_version = -1, confidence_version = -1, N = -1;
        int C = 0, activation = 0, texture_abs = 0;
        float scale = 0.f;
        bool operator==(const PackKey& o) const
        {
            return texture == o.texture && confidence == o.confidence && texture_storage == o.texture_storage &&
                   confidence_storage == o.confidence_storage && texture_version == o.texture_version &&
                   confidence_version == o.confidence_version && N == o.N && C == o.C && activation == o.activation &&
                   texture_abs == o.texture_abs && scale == o.scale;
        }
    };
    PackKey pack_key_;
    // held weakly so that the storages the key names cannot be freed and their addresses handed to other tensors
    c10::weak_intrusive_ptr<c10::StorageImpl> pack_texture_storage_{c10::intrusive_ptr<c10::StorageImpl>()};
    c10::weak_intrusive_ptr<c10::StorageImpl> pack_confidence_storage_{c10::intrusive_ptr<c10::StorageImpl>()};
    bool packed_valid_ = false;
    torch::Tensor packed_;
    struct CountsKey
    {
        int64_t N = -1;
        int L = 0, w = 0, h = 0, mode = 0;
        bool operator==(const CountsKey& o) const { return N == o.N && L == o.L && w == o.w && h == o.h && mode == o.mode; }
    };
    CountsKey counts_key_, pending_key_;
    float counts_[VETRAST_MAX_LAYERS] = {0.f, 0.f, 0.f, 0.f, 0.f};
    bool counts_valid_ = false, counts_pending_ = false;
    int64_t calls_since_readback_ = 0;
    torch::Tensor counts_host_, counts_index_;
    std::unique_ptr<c10::Event> counts_event_;
    void PollFragmentCounts();
};

class NeuralRenderInfo : public torch::CustomClassHolder
{
   public:
    SceneTensors* scene = nullptr;
    std::vector<ReducedImageInfo> images;
    RenderParams params;
    int num_layers           = 1;
    bool train               = false;
    // Set by BlendPointCloud: whether autograd was recording when the call was made. Under torch::NoGradGuard nothing
    // is saved for a backward pass, whatever the leaves require.
    bool grad_mode           = true;
    int current_epoch        = 0;
    void* timer_system       = nullptr;  // accepted for signature parity; per-kernel times come from vetrast_scope_times
    PointRendererCache* cache = nullptr;
};

struct PointRender : public torch::autograd::Function<PointRender>
{
    static torch::autograd::variable_list forward(torch::autograd::AutogradContext* ctx, torch::Tensor texture,
                                                  torch::Tensor background_color, torch::Tensor points,
                                                  torch::Tensor pose_tangents, torch::Tensor intrinsics,
                                                  torch::Tensor confidence, torch::Tensor dynamic_refinement,
                                                  torch::IValue info);
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                   torch::autograd::variable_list grad_output);
};

// Adam over groups of flat float tensors with one kernel per tensor and step: the update of torch::optim::MyAdam
// (src/lib/models/my_adam.cpp:25-104) as the reference sets it up for texture_raw, background_color_raw and confidence_raw,
// one group and learning rate each (src/lib/data/NeuralScene.cpp:238-281), stepped and cleared once per batch (:1247-1248).
class MyAdam
{
   public:
    struct Group
    {
        std::vector<torch::Tensor> params;
        double lr = 1e-3;
    };
    explicit MyAdam(std::vector<Group> groups, double beta1 = 0.9, double beta2 = 0.999, double eps = 1e-8,
                    double weight_decay = 0.0);
    // One step on every parameter that has a gradient; with zero_grad the gradients are cleared in the same pass
    // (texture_optimizer->step(); texture_optimizer->zero_grad();).
    void step(bool zero_grad = false);
    void zero_grad();

   private:
    struct State
    {
        torch::Tensor exp_avg, exp_avg_sq;
        int64_t step = 0;
    };
    std::vector<Group> groups_;
    std::vector<std::vector<State>> state_;
    double beta1_, beta2_, eps_, weight_decay_;
    std::unique_ptr<PointRendererCache> cache_;
};

// Render the scene into a batch of images; every image is a pyramid of layers: L tensors [B,C,h_l,w_l], then L depth
// tensors [B,1,h_l,w_l] if add_depth_to_network (all zero in the blend modes: the reference only fills them in its
// depth-test mode, src/lib/rendering/PointRenderer.cu:1061-1066), then L masks [B,1,h_l,w_l] if output_background_mask.
std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo* info);

// The caller of BlendPointCloud in VET: PointRenderModuleImpl::forward(NeuralRenderInfo*)
// (src/lib/rendering/RenderModule.cpp:45-245). It owns the cache, renders at twice the resolution and averages 2x2
// blocks when super_sampling is on (:60-68,102-127), splits the flat output list into images and (detached) masks
// (:74-100) and appends the masks to the images as an extra channel when cat_masks_to_color is on (:204-210).
// The environment-map branch (:129-202) is there too, with the map itself (a module outside the rasterizer) behind a
// callback: it receives layers[l][b] = a clone of the [1,1,h_l,w_l] slice of the cache's weight tensor, as
// EnvironmentMap::Sample2 does, and returns L tensors [B,C_env,h_l,w_l] that are appended as channels (cat_env_to_color)
// or added to the images, masked to the pixels whose weight is at most 0.001 when no_envmap_at_points is on (:180-196,
// literally: the reference zeroes the map where the weight EXCEEDS 0.001). With add_depth_to_network the (zero) depth
// tensors are appended to the images as a channel (:223-232).
class PointRenderModule
{
   public:
    using EnvironmentSampler =
        std::function<std::vector<torch::Tensor>(const std::vector<std::vector<torch::Tensor>>& layers, NeuralRenderInfo* nri)>;
    bool super_sampling     = false;  // RenderParams::super_sampling, src/lib/data/Settings.h:38
    bool cat_masks_to_color = false;  // PipelineParams::cat_masks_to_color, src/lib/data/Settings.h:295
    EnvironmentSampler environment_map;   // nri->scene->environment_map->Sample2(...), bound by the caller; empty = no map
    bool enable_environment_map = true;   // PipelineParams::enable_environment_map (only looked at with a sampler set)
    bool cat_env_to_color       = false;  // PipelineParams::cat_env_to_color
    bool no_envmap_at_points    = true;   // RenderParams::no_envmap_at_points, src/lib/data/Settings.h:73
    PointRenderModule() : cache(std::make_shared<PointRendererCache>()) {}
    // {images, masks}: L images [B,C(+1),h_l,w_l]; L masks [B,1,h_l,w_l] if output_background_mask, else none
    std::pair<std::vector<torch::Tensor>, std::vector<torch::Tensor>> forward(NeuralRenderInfo* nri);
    std::shared_ptr<PointRendererCache> cache;
};

// VET's scene checkpoints (NeuralScene::SaveCheckpoint / LoadCheckpoint, src/lib/data/NeuralScene.cpp:343-437) are four
// libtorch module archives, <prefix>points.pth, texture.pth, poses.pth and intrinsics.pth, whose entries carry the names
// the modules registered their tensors under:
//   points.pth      parameter "t_position" [N,4] f32, buffer "t_index" [N,1] i32   (src/lib/rendering/NeuralPointCloudCuda.cpp:71-72)
//   texture.pth     parameters "texture" [C,N], "background_color" [C], "confidence_value_of_point" [1,N]: the RAW tensors
//                   (before abs / sigmoid)                                          (src/lib/models/NeuralTexture.cpp:45-47)
//   poses.pth       parameter "tangent_poses" [F,6] f64, buffer "poses_se3" [F,8] f64 (src/lib/data/NeuralStructure.cpp:29-30)
//   intrinsics.pth  parameter "intrinsics" [Ncam,13] f32                             (src/lib/data/NeuralStructure.cpp:96)
// These two functions read and write exactly those entries into / from the tensor bundle the rasterizer takes, so a
// scene trained by VET renders here and the other way round. Entries of the reference's modules that the rasterizer
// does not read are carried along: points.pth also holds the buffers "t_original_color" [N,4] f32 (always; torch::load
// of the reference's module throws when a registered name is missing, so SaveSceneCheckpoint writes zeros when the bundle
// has none), "t_normal" and the four "t_cell_*" tensors when the bundle has them. The environment map and the neural
// camera have files of their own, which are not handled here. A missing file leaves the corresponding tensors undefined.
SceneTensors LoadSceneCheckpoint(const std::string& prefix, torch::Device device = torch::kCPU);
void SaveSceneCheckpoint(const std::string& prefix, const SceneTensors& scene);

// The order VET's scene preprocessing gives a point cloud before the rasterizer ever sees it
// (point_cloud.ReorderMorton64(); point_cloud.RandomBlockShuffle(256); src/lib/data/SceneData.cpp:105-106): points sorted
// by the 63-bit Morton code of their position inside the cloud's bounding box (21 bits per axis), then whole blocks of
// `block` consecutive points shuffled. It is what gives the binning passes their locality (neighbouring threads hit
// neighbouring pixels) while no pixel's fragments arrive from one workgroup only. positions: [N,3] or [N,4] float CPU
// tensor; returns the permutation [N] int64 (new index -> old index). The Morton part is deterministic; the block
// shuffle uses std::mt19937_64(seed) (saiga's generator is not part of the reference tree).
torch::Tensor MortonBlockShuffleOrder(torch::Tensor positions, int64_t block = 256, uint64_t seed = 0);

// SceneData::SortBlocksByRadius(256) (src/lib/data/SceneData.cpp:108,1005-1018), the step after the block shuffle:
// inside every complete block of `block` consecutive points the points are sorted by their drop-out radius, ascending, so
// that with drop_out_points_by_radius the points a layer drops are the leading lanes of every block. radius: [N] float
// CPU tensor in the order the cloud is in; returns the permutation [N] int64 (new index -> old index). Points of equal
// radius keep their order here (std::sort in the reference leaves it unspecified).
// The same kind of order (Morton code over the bounding box, then whole blocks shuffled) computed with tensor operations
// on the device the positions are on, without a host round trip: int32 [N]. For vetrast_forward_args.point_order.
torch::Tensor ProcessingOrderOnDevice(const torch::Tensor& positions, int64_t block = 256, uint64_t seed = 0);
torch::Tensor SortBlocksByRadiusOrder(torch::Tensor radius, int64_t block = 256);

// All of src/lib/data/SceneData.cpp:105-108 for a cloud given as [N,4] (x, y, z, drop-out radius): Morton order, block
// shuffle, blocks sorted by radius; the permutation [N] int64 (new index -> old index).
torch::Tensor ScenePreprocessOrder(torch::Tensor positions_radius, int64_t block = 256, uint64_t seed = 0);

}  // namespace vet_amd
