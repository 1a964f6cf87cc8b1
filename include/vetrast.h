/*
 * vetrast — C ABI of the MI355X (gfx950) blending point rasterizer.
 *
 * This header is the whole drop-in boundary: plain pointers, sizes and PODs, no torch or HIP types.
 * All `device` pointers are hipMalloc'ed (or torch-allocated) memory on the GPU the context was created
 * on; all `host` pointers are ordinary host memory that only has to stay valid for the duration of the call.
 * Every entry point returns 0 on success or a negative vetrast_status, never aborts, never allocates device
 * memory behind the caller's back (the caller owns inputs, outputs and the workspace) and, unless stated
 * otherwise, only enqueues work on the given stream (pass the hipStream_t as `void*`, NULL = default stream).
 * A context serves one host thread at a time.
 *
 * The reference has no C ABI; its seam is the libtorch function
 *   std::vector<torch::Tensor> BlendPointCloud(NeuralRenderInfo*)          src/lib/rendering/PointRenderer.h:53
 *   torch::autograd::PointRender::forward / ::backward                      src/lib/rendering/PointRenderer.h:39-47
 * implemented by BlendPointCloudForward / BlendPointCloudBackward            src/lib/rendering/PointRenderer.cu:657,1111
 * The entry points below are what a libtorch shim with that signature binds (see vet_amd/torch_ext).
 */
#ifndef VETRAST_H
#define VETRAST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VETRAST_MAX_LAYERS 5   /* max_layers, src/lib/rendering/RenderConstants.h:33 */
#define VETRAST_MAX_CHANNELS 4 /* CUDA_KERNEL_ASSERT(num_texture_channels <= 4), src/lib/rendering/RenderForward.cu:1322 */

typedef enum vetrast_status
{
    VETRAST_OK                  = 0,
    VETRAST_ERR_INVALID_ARG     = -1, /* null pointer, size out of range, misaligned workspace */
    VETRAST_ERR_WORKSPACE_SMALL = -2, /* workspace_bytes below vetrast_forward_workspace_bytes() */
    VETRAST_ERR_HIP             = -3, /* a HIP runtime call failed; see vetrast_last_hip_error() */
    VETRAST_ERR_UNSUPPORTED     = -4, /* a reference feature outside the blending path (OCam, normals, ...) */
    VETRAST_ERR_BAD_INPUT_DATA  = -5, /* device-side check failed (non-zero distortion that was not allowed), from
                                         vetrast_query_device_flags */
    VETRAST_ERR_TOO_LARGE       = -6  /* size beyond the fixed maximum of an entry point that allocates nothing */
} vetrast_status;

/* Camera model tag of a view. Mirrors enum CameraModel, src/lib/data/SceneData.h:30-35.
 * Only PINHOLE_DISTORTION is implemented; non-zero distortion coefficients need vetrast_params.allow_distortion. */
#define VETRAST_CAMERA_PINHOLE_DISTORTION 0
#define VETRAST_CAMERA_OCAM 1
#define VETRAST_CAMERA_SPHERICAL 2

/* One view of the batch. Mirrors struct ReducedImageInfo, src/lib/data/SceneData.h:39-50, field by field
 * (the Eigen members are spelled out as floats). The reference passes it by value as a kernel argument
 * (CountingPrepassMulti, src/lib/rendering/RenderForward.cu:807); so does this library. */
typedef struct vetrast_view
{
    int32_t w, h;              /* full-resolution size of layer 0; must be equal for all views of a call */
    int32_t image_index;       /* row of poses_se3 / pose gradient */
    int32_t camera_index;      /* row of intrinsics / intrinsics gradient */
    int32_t camera_model_type; /* VETRAST_CAMERA_* */
    float crop_transform[5];   /* fx, fy, cx, cy, s of IntrinsicsPinholef crop_transform */
    float crop_rotation[4];    /* r00, r01, r10, r11 (row-major; Eigen stores the 2x2 column-major) */
} vetrast_view;

/* Scalar parameters of the path. Mirrors the RenderParams fields the blending path reads
 * (src/lib/data/Settings.h:19-93, copied into DeviceRenderParams at src/lib/rendering/RenderConstants.h:105-126). */
typedef struct vetrast_params
{
    int32_t num_texture_channels;         /* C, 1..4 */
    int32_t num_layers;                   /* L, 1..5  (NeuralRenderInfo::num_layers) */
    int32_t debug_max_list_length;        /* K; <= 0 means no cut (reference default -1) */
    int32_t use_environment_map;          /* 0: the background colour is blended behind the last fragment */
    int32_t need_point_gradient;          /* backward: compute the position gradient */
    int32_t viewer_only;                  /* with it, points with confidence < stability_cutoff_value are skipped */
    float stability_cutoff_value;
    int32_t drop_out_points_by_radius;    /* stop descending layers once the splat radius falls below the threshold */
    float drop_out_radius_threshold;
    int32_t output_background_mask;       /* forward also writes out_mask = (weight == 0 ? mask_value : 1) */
    float output_background_mask_value;
    int32_t check_normal;                 /* must be 0 (needs saiga's UnpackNormal10Bit) */
    /* Two switches for behaviours of the reference that are accidents of its implementation: */
    int32_t quirk_background_confidence_leak; /* 1: the background pseudo-fragment also adds its alpha gradient to
                                                 grad_confidence[0], as src/lib/rendering/RenderBackward.cu:1157 does */
    int32_t point_gradient_normalization;     /* 0: leave sums and counts; 1: row i / count i;
                                                 2: literal reference (vec3 stride over the [N,4] buffer,
                                                 src/lib/rendering/PointRenderer.cu:1278-1279) */
    /* Pose / intrinsics gradients (only computed when the matching buffers of vetrast_backward_args are given): */
    float K_gradient_factor;                  /* RenderParams::K_gradient_factor, src/lib/data/Settings.h:55 */
    int32_t camera_gradient_normalization;    /* 0: leave sums and counts; 1: divide each pose / intrinsics row by its
                                                 count as src/lib/rendering/PointRenderer.cu:1253-1308 does (the count
                                                 grows by 1/1024 per fragment, so this is 1024 x the mean) */
    int32_t render_mode;                      /* RenderParams::render_mode, src/lib/data/Settings.h: 1 = FULL_BLEND
                                                 (a point lands in the pixel it rounds to), 3 = BILINEAR_BLEND (a point
                                                 lands in the 2x2 pixels around it, alpha = bilinear weight x confidence,
                                                 blending stops once the transmittance falls below 0.001), 2 =
                                                 FUZZY_BLEND (FULL_BLEND lists; the nearest fragments of a pixel that
                                                 lie within depth_accept_blend of the first one are averaged before
                                                 they are blended). Other values (0 = FUZZY_DT, the
                                                 depth-test mode, included) are refused. */
    /* The steps VET runs on the optimised tensors right before the rasterizer, fused into it
     * (NeuralPointTextureImpl::PrepareConfidence / PrepareTexture, src/lib/models/NeuralTexture.h:38-55; called from
     * src/lib/models/Pipeline.cpp:113-124). With them on, `confidence`, `texture` and `background` are the RAW tensors
     * and the gradients vetrast_backward returns are those of the raw tensors. */
    int32_t confidence_activation;            /* 0: confidence is used as given; 1: sigmoid(confidence_scale * confidence) */
    float confidence_scale;                   /* 10 + sigmoid_narrowing_factor * epoch in VET */
    int32_t texture_abs;                      /* 1: |texture| and |background| (PipelineParams::non_subzero_texture) */
    float depth_accept_blend;                 /* FUZZY_BLEND: depth range of a bucket, RenderParams::depth_accept_blend
                                                 (src/lib/data/Settings.h:42, default 0.01); must lie in (0, 1e4) */
    /* A hint for speed only; results do not depend on it. The pixels of a layer are cut into bins sized so that a bin
     * is expected to hold about a thousand fragments if EVERY point lands in the layer. A view that sees a part of the
     * cloud (VET trains on 512x512 crops, configs/config.ini:27) or drops points by radius at the coarse layers then
     * gets bins far too small. expected_fragments[l] > 0 says how many fragments ONE view is expected to leave in layer
     * l (e.g. what the previous call left there: offsets[layer_pixel_base[l + 1]] - offsets[layer_pixel_base[l]]); the
     * bins of that layer are sized for it. 0: every point. No counterpart in the reference. */
    float expected_fragments[VETRAST_MAX_LAYERS];
    /* Lens distortion. The reference distorts the normalised image point with saiga's distortNormalizedPoint
     * (src/lib/rendering/PointRendererHelper.h:207,348), which is not part of its source tree; cameras with non-zero
     * coefficients are therefore refused (VETRAST_ERR_BAD_INPUT_DATA through vetrast_query_device_flags) unless
     * allow_distortion is set. With it, columns 5..12 of `intrinsics` are taken as k1 k2 k3 k4 k5 k6 p1 p2 (the order
     * of src/lib/data/SceneData.cpp:464-478) of the rational model
     *   x' = x (1 + k1 r^2 + k2 r^4 + k3 r^6) / (1 + k4 r^2 + k5 r^4 + k6 r^6) + 2 p1 x y + p2 (r^2 + 2 x^2)
     *   y' = y (   same ratio   )                                              + p1 (r^2 + 2 y^2) + 2 p2 x y
     * and the backward pass returns their gradient scaled as src/lib/rendering/RenderBackward.cu:1440-1455 scales it
     * (k3 x 0.25, k4..k6 and p1, p2 x 0.1, everything x distortion_gradient_factor). PARITY WITH THE REFERENCE IS
     * UNPINNED for such cameras: the formula is the published one the coefficient layout implies, not saiga's code,
     * and RenderParams::dist_cutoff (points beyond the radius where the polynomial stops being monotonic are culled
     * by saiga) is not applied. */
    int32_t allow_distortion;
    float distortion_gradient_factor;         /* RenderParams::distortion_gradient_factor, src/lib/data/Settings.h:54 */
} vetrast_params;

#define VETRAST_RENDER_FULL_BLEND 1
#define VETRAST_RENDER_FUZZY_BLEND 2
#define VETRAST_RENDER_BILINEAR_BLEND 3

typedef struct vetrast_ctx vetrast_ctx;

/* Per-kernel timing scopes, named after the reference's CudaTimerSystem scopes
 * (src/lib/rendering/PointRenderer.cu:249,770,791,843,872,886,1222,1252). */
typedef enum vetrast_scope
{
    VETRAST_SCOPE_PREPARE = 0,      /* "Build Cache": zero-fill, view preparation */
    VETRAST_SCOPE_PACK,             /* "Build Cache": descriptor interleave; it rides along with the COUNT kernel of the
                                       first view, so this scope reports no launches of its own */
    VETRAST_SCOPE_COUNT,            /* "CountingPass": fragments per bin (a 16x16 pixel tile or a piece of one) and, in
                                       the same pass over the points, the fragment records written to their bins */
    VETRAST_SCOPE_SCAN,             /* "CreateAndAllocateBuffers" (prefix scan over the bins; no allocation here) */
    VETRAST_SCOPE_FILL,             /* "CollectionPass", first half: the records that did not fit their bin's own room
                                       are filed behind the scan (an almost empty kernel as a rule) */
    VETRAST_SCOPE_BUILD,            /* "CollectionPass" second half + "SortingPass" + "BlendingPass": one pass per bin */
    VETRAST_SCOPE_BACKWARD_PREPARE, /* "Prepare Backward": zero-fill of gradient buffers */
    VETRAST_SCOPE_BACKWARD_BLEND,   /* "BlendBackwards", per-pixel part */
    VETRAST_SCOPE_BACKWARD_GATHER,  /* "BlendBackwards", per-point sum of the stored fragment gradients */
    VETRAST_SCOPE_BACKWARD_POST,    /* "Post Process Gradient" */
    VETRAST_SCOPE_LIFT_ERROR,       /* vetrast_lift_error (the reference times FillSceneGridWithLoss in no scope) */
    VETRAST_SCOPE_COUNT_
} vetrast_scope;

/* Byte offsets of the arrays inside the forward workspace, so that a caller (or a test) can read the
 * per-pixel fragment lists. Pixels are numbered tile by tile: every layer is cut into 16x16 pixel tiles (the last
 * column / row of tiles may hang over the image; those pixels exist in the numbering and have empty lists), and
 *   q = 256 * (layer_tile_base[l] + (y / 16) * layer_tiles_x[l] + x / 16) + 16 * (y % 16) + x % 16. */
typedef struct vetrast_workspace_layout
{
    int32_t layer_w[VETRAST_MAX_LAYERS];
    int32_t layer_h[VETRAST_MAX_LAYERS];
    int32_t layer_tiles_x[VETRAST_MAX_LAYERS];        /* tiles per row of the layer = ceil(w_l / 16) */
    int32_t reserved0;
    int64_t layer_tile_base[VETRAST_MAX_LAYERS + 1];  /* first tile of the layer; [L] = number of tiles T */
    int64_t layer_pixel_base[VETRAST_MAX_LAYERS + 1]; /* 256 * layer_tile_base; [L] = pixel numbers P of one view */
    int64_t fragment_capacity;                        /* N * L * hits_per_layer, the per-view upper bound on fragments */
    int32_t hits_per_layer;                           /* 1 (FULL_BLEND) or 4 (BILINEAR_BLEND): fragments of a point per layer */
    int32_t reserved1;
    size_t total_bytes;
    /* per-view arrays: offset of view b = base + b * stride */
    size_t offsets_base, offsets_stride;     /* uint32 [P+1]: exclusive scan of per-pixel counts; [P] = fragments of the view */
    size_t fragments_base, fragments_stride; /* uint64 [N*L]: (depth_bits << 32) | point_id, per pixel ascending; only the
                                                first min(count, K) entries of a pixel's list are sorted and meaningful */
    size_t transmittance_base, transmittance_stride; /* float [N*L]: transmittance in front of each kept fragment */
    size_t weight_base, weight_stride;       /* float [P]: final transmittance per pixel (the reference's `weight` image) */
    size_t kept_base, kept_stride;           /* uint32 [P], BILINEAR_BLEND only: fragments of the pixel's list that took part in
                                                the blend (FULL_BLEND: min(count, K), not stored) */
    size_t cut_flags_base, cut_flags_stride; /* uint8 [P]: 1 where some fragments of the pixel's list did not (top-K cut, saturation) */
    /* shared by all views */
    size_t packed_base;    /* float [N][8]: descriptor (4, zero padded), confidence, 3 pad */
    size_t slots_base;     /* uint32, shaped like the log: rank inside its bin of every logged record (scratch) */
    size_t views_base;     /* prepared per-view camera constants */
    size_t scan_partials_base;
    int64_t num_bins;      /* bins of one view: runs of 256 / 64 / 16 / 4 consecutive pixel numbers, chosen per layer from N */
    size_t bin_counts_base, bin_counts_stride; /* per view, uint32 [2][num_bins+1 padded]: fragments per bin, and their
                                                  exclusive scan (in place of the counts where a view has more than
                                                  15 360 bins) */
    size_t binned_base;    /* uint32 [N*L*hits][4]: compact array of fragment records (key low, key high, pixel in bin, 0),
                              only used for the records beyond a bin's own room; scratch. In FULL_BLEND / FUZZY_BLEND with
                              N <= 2^24 a record is uint32 [2]: (depth bits, point id << 8 | pixel in bin) */
    size_t flags_base;     /* uint32 [4] device status flags, then at +64 bytes float [4]: the background as it is blended */
    size_t forward_only_bytes; /* a forward call with save_for_backward = 0 needs only this much */
    size_t partial_base;   /* float [L][N][8]: backward scratch, gradient record of the fragment of point i in layer l */
    size_t background_partial_base; /* float [workgroups][8]: backward scratch, per-workgroup background-gradient sums */
    size_t camera_partial_base;     /* double [ceil(N/256)][12]: backward scratch, per-workgroup pose / intrinsics sums */
    /* scratch shared by all views: the scatter pass writes the records of a bin to the bin's own room while their rank
     * is below the room's size (2048 records where about a thousand are expected per bin, 1024 where at most 512 are);
     * records beyond that go to a log of 256 segments (record + bin, rank in the slots array) and are filed into the
     * compact array after the scan. log_cursor: per view, 256 uint32 64 bytes apart, entries in every segment.
     * The log and the slots array only live inside a forward call: partial_base == log_base, the scratch of the
     * backward call lies on top of them (forward_only_bytes covers the log, total_bytes both). */
    size_t primary_base;   /* the rooms, layer after layer, bin after bin: 16-byte records, or 8-byte ones (see binned_base) */
    size_t log_base;       /* uint32 [256][ceil(ceil(N/256)/256)*256*L*hits][4] */
    size_t log_cursor_base;
    size_t last_key_base, last_key_stride;   /* per view, uint64 [P]: where cut_flags is 1, the key of the last fragment of
                                                the pixel's list that took part in the blend (0 if none did) */
    size_t projected_base, projected_stride; /* per view, float [N][2], BILINEAR_BLEND only (stride 0 otherwise): image
                                                position of every visible point at layer 0, from which the blend and its
                                                backward pass form the bilinear weights */
    /* A call with several views takes them view_lanes = min(num_views, 4) at a time: every kernel of the call is one
     * launch for the views of such a round (view b of the call on lane b % view_lanes), so the scratch that one view
     * needs exists once per lane: lane k's copy of binned, primary and scan_partials lies k * the stride behind the
     * base, its copy of the log / slots / partial / background_partial block k * lane_scratch_stride behind theirs. */
    int32_t view_lanes;
    int32_t reserved2;
    size_t binned_stride, primary_stride, scan_partials_stride, lane_scratch_stride;
} vetrast_workspace_layout;

/* Arguments of the forward pass. Replaces the inputs PointRender::forward receives
 * (src/lib/rendering/RenderInfo.cpp:25-29,34-43) plus what it reads through info->scene. */
typedef struct vetrast_forward_args
{
    int32_t num_points; /* N */
    int32_t num_views;  /* B = info->images.size() */
    int32_t num_poses;  /* F, rows of poses_se3 */
    int32_t num_cameras;
    const float* position;    /* device [N,4] x,y,z,drop-out radius (t_position, src/lib/rendering/NeuralPointCloudCuda.h:193-224) */
    const int32_t* index;     /* device [N] texture index of a point (t_index) or NULL for the identity */
    const float* texture;     /* device [C,N] planar descriptors */
    const float* confidence;  /* device [N] (the reference's [1,N]) already in (0,1) */
    const float* background;  /* device [C] */
    const float* dropout;     /* device [B,N], a point is skipped in view b where the value == 1; NULL = none */
    const double* poses_se3;  /* device [F,8] world->camera: unit quaternion x,y,z,w, translation, 1 pad
                                 (src/lib/data/NeuralStructure.cpp:15-28) */
    const float* intrinsics;  /* device [num_cameras,13]: fx,fy,cx,cy,s,k1..k6,p1,p2 (src/lib/data/NeuralStructure.cpp:65-99) */
    const vetrast_view* views; /* host [B] */
    vetrast_params params;
    int32_t save_for_backward; /* also store the per-fragment transmittance the backward pass reads */
    float* out[VETRAST_MAX_LAYERS];      /* device, layer l: [B,C,h_l,w_l] contiguous NCHW; fully overwritten */
    float* out_mask[VETRAST_MAX_LAYERS]; /* device, layer l: [B,1,h_l,w_l]; only with output_background_mask */
    void* workspace;                     /* device, 256-byte aligned */
    size_t workspace_bytes;
    /* Optional, layer l: device [B,1,h_l,w_l], the transmittance left behind the last blended fragment of every pixel
     * (1 where no point landed): the `weight` tensor of the reference's layer cache
     * (src/lib/rendering/RenderForward.cu:1355-1356), which PointRenderModuleImpl::forward hands to the environment map
     * (src/lib/rendering/RenderModule.cpp:132-196). NULL = not wanted. */
    float* out_weight[VETRAST_MAX_LAYERS];
    /* Optional, device [N]: a permutation of 0..N-1, the order in which the binning pass walks the points (thread i
     * takes point point_order[i]). Results do not depend on it, bit for bit; the time of the binning pass does: it
     * groups the points of a wave by bin before it touches global counters, so it wants neighbours in the array to be
     * neighbours in space. A cloud in the order of VET's preprocessing (src/lib/data/SceneData.cpp:105-108) needs none;
     * one that has grown since (NeuralScene::AddNewPoints appends, src/lib/data/NeuralScene.cpp:1013) or comes in
     * file order does. Point ids everywhere else (index, gradients, dropout) stay the caller's. NULL = array order.
     * No counterpart in the reference. */
    const int32_t* point_order;
    /* Optional, device float [N][8], 32-byte aligned: the descriptor records vetrast_pack_descriptors wrote from THIS
     * texture and confidence under THESE params (num_texture_channels, confidence_activation, confidence_scale,
     * texture_abs). The call then reads a fragment's descriptor and confidence from it and leaves out the interleave
     * it otherwise does on the side in every call: for callers that render a scene more than once between changes of
     * its texture (a viewer; evaluation). The caller vouches that the records are current; vetrast_backward reads the
     * same array. NULL = the call interleaves for itself, into the workspace. No counterpart in the reference, which
     * reads the planar tensors per channel (src/lib/rendering/RenderForward.cu:1338-1342). */
    const float* packed_descriptors;
} vetrast_forward_args;

/* Arguments of the backward pass. Replaces BlendPointCloudBackward's inputs and its seven returned tensors
 * (src/lib/rendering/PointRenderer.cu:1111-1323). The workspace and `out` must be those of the matching forward call
 * (made with save_for_backward = 1) and unchanged since; this is the saved state of
 * src/lib/rendering/PointRenderer.cu:1027-1059. fwd.out_mask is not used and may be left NULL. */
typedef struct vetrast_backward_args
{
    vetrast_forward_args fwd;                      /* same values as passed to vetrast_forward */
    const float* grad_out[VETRAST_MAX_LAYERS];     /* device, layer l: [B,C,h_l,w_l] upstream gradient */
    float* grad_texture;     /* device [C,N]; overwritten */
    float* grad_confidence;  /* device [N]; overwritten */
    float* grad_background;  /* device [C]; overwritten */
    float* grad_points;      /* device [N,4] or NULL (points do not require grad); xyz sums (w stays 0); overwritten */
    float* grad_point_count; /* device [N]; number of fragments that contributed to a point; required with grad_points */
    /* Optional camera gradients, accumulated over every fragment that gets a position gradient
     * (src/lib/rendering/RenderBackward.cu:1418-1459). NULL = not wanted. */
    double* grad_pose;           /* device [F,6]: d/d(se3 tangent: translation, rotation) of pose row image_index; overwritten */
    float* grad_pose_count;      /* device [F]: fragments / 1024 per pose row; required with grad_pose */
    float* grad_intrinsics;      /* device [num_cameras,13]: fx,fy,cx,cy scaled by K_gradient_factor; the skew column is
                                    zeroed as in the reference; the 8 distortion columns are filled where
                                    vetrast_params.allow_distortion is set, else stay 0; overwritten */
    float* grad_intrinsics_count; /* device [num_cameras]: fragments / 1024 per camera row; required with grad_intrinsics */
} vetrast_backward_args;

/* Create / destroy a context bound to the current HIP device. The context owns only a few HIP events. */
int vetrast_create(vetrast_ctx** out_ctx);
void vetrast_destroy(vetrast_ctx* ctx);

/* Layer pyramid by repeated integer halving (src/lib/rendering/PointRenderer.cu:351-381). Pure host arithmetic. */
int vetrast_layer_sizes(int32_t w, int32_t h, int32_t num_layers, int32_t* layer_w, int32_t* layer_h);

/* Size and layout of the workspace a forward call with these dimensions needs. Pure host arithmetic. The reference
 * sizes its fragment buffers from a device->host read of the scan total (src/lib/rendering/PointRenderer.cu:811-821);
 * here the buffer has the upper bound N*L entries per view instead, so no read-back is needed. */
int vetrast_workspace_layout_for(int32_t num_points, int32_t num_views, int32_t num_layers, int32_t w, int32_t h,
                                 vetrast_workspace_layout* layout);
/* The same for a given render mode (BILINEAR_BLEND needs room for four fragments per point and layer);
 * vetrast_workspace_layout_for and vetrast_forward_workspace_bytes are the FULL_BLEND case. */
int vetrast_workspace_layout_for_mode(int32_t num_points, int32_t num_views, int32_t num_layers, int32_t w, int32_t h,
                                      int32_t render_mode, vetrast_workspace_layout* layout);
size_t vetrast_forward_workspace_bytes(int32_t num_points, int32_t num_views, int32_t num_layers, int32_t w, int32_t h);

/* Forward: project, count, scan, fill, per-pixel sort by (depth bits, point id), top-K cut, front-to-back blend.
 * Replaces BlendPointCloudForward in FULL_BLEND mode (src/lib/rendering/PointRenderer.cu:657-1069). */
int vetrast_forward(vetrast_ctx* ctx, const vetrast_forward_args* args, void* stream);

/* Backward: gradients to descriptors, confidence, background and point positions.
 * Replaces BlendPointCloudBackward in FULL_BLEND mode (src/lib/rendering/PointRenderer.cu:1111-1323). */
int vetrast_backward(vetrast_ctx* ctx, const vetrast_backward_args* args, void* stream);

/* Blocking: waits for the stream, then reads the device flag word of the workspace. Returns VETRAST_OK or
 * VETRAST_ERR_BAD_INPUT_DATA (a camera with non-zero distortion coefficients was used; the reference's saiga
 * distortion model is not available, so such input is flagged instead of guessed). */
int vetrast_query_device_flags(vetrast_ctx* ctx, const void* workspace, const vetrast_workspace_layout* layout,
                               void* stream);

/* Writes the descriptor records of vetrast_forward_args.packed_descriptors: row i = texture[0..C-1][i] (|.| with
 * texture_abs), then confidence[i] (sigmoid(confidence_scale * .) with confidence_activation), then zeros; the steps
 * of NeuralPointTextureImpl::PrepareTexture / PrepareConfidence (src/lib/models/NeuralTexture.h:38-55) and the
 * interleave in one pass. Of `params` only those four members are read. One streaming kernel, 52 bytes per point. */
typedef struct vetrast_pack_args
{
    int32_t num_points;
    const float* texture;    /* device [C,N] */
    const float* confidence; /* device [N] */
    vetrast_params params;
    float* packed;           /* device [N][8], 32-byte aligned; fully overwritten */
} vetrast_pack_args;
size_t vetrast_packed_descriptor_bytes(int32_t num_points);
int vetrast_pack_descriptors(vetrast_ctx* ctx, const vetrast_pack_args* args, void* stream);

/* One Adam step on a flat float tensor, the update MyAdam::step applies to texture_raw, confidence_raw and
 * background_color_raw after every batch (src/lib/models/my_adam.cpp:25-104 = torch's Adam without amsgrad; options as
 * in src/lib/data/NeuralScene.cpp:238-281): one kernel instead of the ~10 elementwise launches of the tensor-op form.
 *   g = grad + weight_decay * param;  m = beta1 * m + (1 - beta1) * g;  v = beta2 * v + (1 - beta2) * g * g;
 *   param -= lr / (1 - beta1^step) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps)
 * `step` is the state's step count after the increment (1 on the first call). With zero_grad the gradient is cleared
 * in the same pass (texture_optimizer->zero_grad(), src/lib/data/NeuralScene.cpp:1247-1248). */
typedef struct vetrast_adam_args
{
    float* param;      /* device [n] */
    float* grad;       /* device [n] */
    float* exp_avg;    /* device [n], zero before the first step */
    float* exp_avg_sq; /* device [n], zero before the first step */
    int64_t n;
    int64_t step;
    double lr, beta1, beta2, eps, weight_decay; /* doubles as in torch's AdamOptions: 1 - beta2 must not be formed in float */
    int32_t zero_grad;
} vetrast_adam_args;
int vetrast_adam_step(vetrast_ctx* ctx, const vetrast_adam_args* args, void* stream);

/* Error lifting: adds the per-pixel error of one rendered view to every cell of the scene grid whose projection covers
 * the pixel. Replaces PointRendererCache::FillSceneGridWithLoss and its kernel FillSceneGridWithLossRasterize
 * (src/lib/rendering/RenderForward.cu:605-632,639-791; called once per view of a batch in the epoch before points are
 * added, src/apps/train.cpp:1069-1078; cell tensors: src/lib/rendering/NeuralPointCloudCuda.h:100-106,166-191,
 * built by UpdateCellStructureForPointOptim, src/lib/rendering/NeuralPointCloudCuda.cpp:95-147).
 *
 * For every cell: the 8 corners bb_min + bb_length * {000,100,010,001,110,101,011,111} are projected like points
 * (pinhole, zero distortion, crop transform and rotation of `view`); a cell with a corner at or behind the camera
 * plane is skipped; the pixel box of the 8 projections is cut to the image minus a border of `border_pixels`
 * (VETRAST_LIFT_BORDER_PIXELS in the reference); every integer pixel of the box that lies in one of the 12 projected
 * face triangles adds sum_c |loss_image[c][y][x]| to cell_value and 1 to cell_access_count.
 *
 * The reference adds the float terms with atomics in arrival order; here the terms of a cell are summed in double and
 * added to cell_value with one rounding, which makes the call reproducible. cell_value and cell_access_count are
 * accumulated into, not cleared (ResetCellValues / NormalizeBBCellValue stay with the caller,
 * src/lib/rendering/NeuralPointCloudCuda.h:42-52). */
#define VETRAST_LIFT_BORDER_PIXELS 32
/* Byte offset inside the workspace of a uint32 that is 1 after the call if the camera row holds non-zero distortion
 * coefficients (they are ignored, as in vetrast_forward), else 0. */
#define VETRAST_LIFT_FLAGS_OFFSET 192
/* Byte offset inside the workspace of a uint32 that holds, after the call, how many cells were too large on screen for
 * one wave and went through the shared path (a diagnostic; nothing has to read it). */
#define VETRAST_LIFT_QUEUE_LENGTH_OFFSET 176
typedef struct vetrast_lift_args
{
    int64_t num_cells;
    const float* cell_bb_min;    /* device [num_cells,3] (t_cell_bb_min) */
    const float* cell_bb_length; /* device [num_cells,3] (t_cell_bb_length) */
    float* cell_value;           /* device [num_cells] (t_cell_value, [num_cells,1]); accumulated into */
    int32_t* cell_access_count;  /* device [num_cells] (t_cell_access_count); accumulated into */
    int32_t num_poses;           /* rows of poses_se3 */
    int32_t num_cameras;
    const double* poses_se3;     /* device [num_poses,8], as in vetrast_forward_args */
    const float* intrinsics;     /* device [num_cameras,13], as in vetrast_forward_args */
    vetrast_view view;           /* the view the error image belongs to (images[batch]); w / 2, h / 2 is the crop rotation centre */
    const float* loss_image;     /* device [channels,height,width], e.g. |target - output| of that view */
    int32_t channels, height, width;
    int32_t border_pixels;       /* >= 0; the reference's constant is VETRAST_LIFT_BORDER_PIXELS */
    void* workspace;             /* device, 256-byte aligned, vetrast_lift_workspace_bytes(num_cells) bytes */
    size_t workspace_bytes;
} vetrast_lift_args;
size_t vetrast_lift_workspace_bytes(int64_t num_cells);
int vetrast_lift_error(vetrast_ctx* ctx, const vetrast_lift_args* args, void* stream);

/* vetrast_lift_error for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same arguments, same kernels and
 * same results as vetrast_lift_error, but `workspace` / `workspace_bytes` are ignored: the scratch is an array inside
 * the library (about 12.6 MB of device memory per GPU, held until the process ends), whose address on the context's
 * device vetrast_create looks up once. The call itself allocates and frees nothing, creates no events (it reports no
 * timing scope) and only launches kernels.
 *   - num_cells > VETRAST_LIFT_STATIC_MAX_CELLS is refused with VETRAST_ERR_TOO_LARGE.
 *   - The context's device must be the current device, else VETRAST_ERR_INVALID_ARG.
 *   - All calls on one GPU share that GPU's array (every call rewrites what it reads, nothing has to be cleared in
 *     between): calls that overlap on one GPU, on different streams or from different contexts, race. Calls on one
 *     stream are safe.
 *   - The distortion flag word of vetrast_lift_error lives in the scratch and cannot be read back here; check the
 *     intrinsics beforehand. */
#define VETRAST_LIFT_STATIC_MAX_CELLS (1 << 19)
int vetrast_lift_error_static(vetrast_ctx* ctx, const vetrast_lift_args* args, void* stream);

/* Per-kernel timing, the counterpart of NeuralRenderInfo::timer_system (src/lib/rendering/PointRenderer.h:32).
 * With profiling enabled every launch is bracketed by HIP events on the call's stream; vetrast_scope_times
 * synchronises on them and returns, per scope, the summed kernel time in milliseconds and the number of launches
 * since the last vetrast_reset_scope_times. */
int vetrast_set_profiling(vetrast_ctx* ctx, int32_t enabled);
int vetrast_reset_scope_times(vetrast_ctx* ctx);
int vetrast_scope_times(vetrast_ctx* ctx, float* ms /* [VETRAST_SCOPE_COUNT_] */,
                        int32_t* launches /* [VETRAST_SCOPE_COUNT_] */);
const char* vetrast_scope_name(int32_t scope);

const char* vetrast_status_string(int status);
/* hipError_t value of the last failed HIP call of this context (0 if none). */
int vetrast_last_hip_error(const vetrast_ctx* ctx);

#ifdef __cplusplus
}
#endif
#endif /* VETRAST_H */
