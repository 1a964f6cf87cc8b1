// C ABI of the gfx950 blending point rasterizer: argument checks, workspace layout and the launch sequence.
// Host-side counterpart of BlendPointCloudForward / BlendPointCloudBackward and PointRendererCache
// (src/lib/rendering/PointRenderer.cu:238-470,657-1069,1111-1323 of the reference), without its per-layer
// device->host reads, per-frame allocations and __constant__ uploads.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstring>
#include <type_traits>
#include <mutex>
#include <new>
#include <vector>

#include "common.h"
#include "forward_kernels.h"
#include "sort_kernels.h"
#include "build_kernels.h"
#include "backward_kernels.h"
#include "lift_kernels.h"

using namespace vetrast;

struct vetrast_ctx
{
    int device         = 0;
    int profiling      = 0;
    int last_hip_error = 0;
    struct Span
    {
        int scope;
        hipEvent_t start, stop;
    };
    std::vector<Span> spans;             // recorded since the last reset
    std::vector<hipEvent_t> free_events;  // recycled events
    float acc_ms[VETRAST_SCOPE_COUNT_]      = {};
    int32_t acc_launches[VETRAST_SCOPE_COUNT_] = {};
    char* lift_scratch = nullptr;  // this device's copy of the file-scope scratch array (vetrast_lift_error_static)
};

namespace
{
constexpr size_t kAlign = 256;
constexpr double kSplitListLength = 8.0;  // layers that blend at least this many fragments per pixel are split
inline size_t align_up(size_t v, size_t a)
{
    return (v + a - 1) / a * a;
}

// Bytes of error-lifting scratch for num_cells cells: header (camera constants, queue length, flag word), queue
// entries, one double per queue slot, chunk prefix sums.
constexpr size_t align_up_c(size_t v, size_t a) { return (v + a - 1) / a * a; }
constexpr size_t lift_workspace_bytes_for(size_t num_cells)
{
    return kLiftHeader + align_up_c(num_cells * sizeof(uint2), kAlign) + align_up_c(num_cells * sizeof(double), kAlign) +
           align_up_c((num_cells + 1) * sizeof(unsigned long long), kAlign);
}

#define VET_HIP(ctx, expr)                               \
    do                                                   \
    {                                                    \
        hipError_t e_ = (expr);                          \
        if (e_ != hipSuccess)                            \
        {                                                \
            if (ctx) (ctx)->last_hip_error = (int)e_;    \
            return VETRAST_ERR_HIP;                      \
        }                                                \
    } while (0)

// Brackets the launches of one scope with events when profiling is on.
struct ScopeTimer
{
    vetrast_ctx* ctx;
    hipStream_t stream;
    int scope;
    hipEvent_t start = nullptr, stop = nullptr;
    bool on          = false;
    ScopeTimer(vetrast_ctx* c, hipStream_t s, int sc) : ctx(c), stream(s), scope(sc)
    {
        if (!ctx->profiling) return;
        start = take();
        stop  = take();
        if (!start || !stop) return;
        on = hipEventRecord(start, stream) == hipSuccess;
    }
    ~ScopeTimer()
    {
        if (!on) return;
        (void)hipEventRecord(stop, stream);
        ctx->spans.push_back({scope, start, stop});
    }
    hipEvent_t take()
    {
        if (!ctx->free_events.empty())
        {
            hipEvent_t e = ctx->free_events.back();
            ctx->free_events.pop_back();
            return e;
        }
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return nullptr;
        return e;
    }
};

inline int grid_for(size_t n, int block = kBlock)
{
    return (int)((n + block - 1) / block);
}

// N only steers the bin sizes: N / pixels bounds the mean list length of a layer from above without any device read.
LayerTable make_layer_table(int w, int h, int L, int64_t N, const float* expected_fragments = nullptr)
{
    LayerTable t;
    std::memset(&t, 0, sizeof(t));
    t.L           = L;
    uint32_t tile = 0, bin = 0, room = 0;
    for (int l = 0; l < L; ++l)
    {
        t.w[l]         = w;
        t.h[l]         = h;
        t.tiles_x[l]   = (w + kTile - 1) / kTile;
        t.tiles_y[l]   = (h + kTile - 1) / kTile;
        t.tile_base[l] = tile;
        t.base[l]      = tile * kTilePixels;
        const uint32_t tiles = (uint32_t)t.tiles_x[l] * (uint32_t)t.tiles_y[l];
        tile += tiles;
        // largest bin of 256, 64, 16 or 4 pixels expected to hold at most 1024 fragments
        // Fragments the bins of the layer are sized for: every point, unless the caller knows how many a view leaves
        // there. Then twice that number: the rule below was tuned on full frames, sized for every point, of which about
        // half were in view (surfaces put a multiple of the mean into many bins).
        double in_layer = (double)N;
        if (expected_fragments && expected_fragments[l] > 0.f && 2.0 * (double)expected_fragments[l] < in_layer)
            in_layer = 2.0 * (double)expected_fragments[l];
        const double mean_len = in_layer / ((double)w * (double)h);
        int shift             = 8;
        while (shift > 2 && mean_len * (double)(1 << shift) > 1024.0) shift -= 2;
        // ... and small enough for the layer to have a thousand bins where it has the pixels for them: every bin is one
        // workgroup's chain of dependent steps, and a layer of a few dozen big bins (a coarse layer of a 512x512
        // training crop) runs them on a few dozen compute units while the others wait
        while (shift > 2 && (tiles << (8 - shift)) < 1024u) shift -= 2;
        t.bin_shift[l] = shift;
        t.bin_base[l]  = bin;
        t.room_cap[l]  = mean_len * (double)(1 << shift) > 512.0 ? kPrimaryCap : kPrimaryCapSmall;
        t.room_base[l] = room;
        room += (tiles << (8 - shift)) * t.room_cap[l];
        bin += tiles << (8 - shift);
        w /= 2;
        h /= 2;
    }
    for (int l = L; l <= VETRAST_MAX_LAYERS; ++l)
    {
        t.tile_base[l] = tile;
        t.base[l]      = tile * kTilePixels;
        t.bin_base[l]  = bin;
        t.room_base[l] = room;
    }
    return t;
}

// The layer table the kernels of a call work with: bins sized for the fragments the caller expects a view to leave in
// every layer (vetrast_params.expected_fragments), but never more bins or more room than the table the workspace was
// laid out for (every point in every layer), which smaller expectations cannot exceed: coarser bins are fewer, and a
// bin's room at most doubles where its pixels quadruple.
LayerTable make_call_layer_table(int w, int h, int L, int64_t hits_if_all_visible, const float* expected_fragments)
{
    const LayerTable full = make_layer_table(w, h, L, hits_if_all_visible);
    const LayerTable t    = make_layer_table(w, h, L, hits_if_all_visible, expected_fragments);
    if (t.bin_base[L] > full.bin_base[L] || t.room_base[L] > full.room_base[L]) return full;
    return t;
}

// Fragments a point can leave in one layer: 1 (the pixel it rounds to) or the 2x2 pixels around it.
inline int hits_of_mode(int render_mode)
{
    return render_mode == VETRAST_RENDER_BILINEAR_BLEND ? 4 : 1;
}

// Fragment records of 8 instead of 16 bytes: the low key word (point id, or point id << 2 | corner of the 2x2 splat)
// fits 24 bits.
inline bool compact_records(int64_t N, int hits)
{
    return N * hits <= (int64_t)(1 << 24);
}

inline int check_mode(int render_mode)
{
    return (render_mode == VETRAST_RENDER_FULL_BLEND || render_mode == VETRAST_RENDER_FUZZY_BLEND ||
            render_mode == VETRAST_RENDER_BILINEAR_BLEND)
               ? VETRAST_OK
               : VETRAST_ERR_UNSUPPORTED;
}

int check_dims(int64_t N, int B, int L, int w, int h, int hits)
{
    if (N < 0 || B < 1 || L < 1 || L > VETRAST_MAX_LAYERS || w < 1 || h < 1) return VETRAST_ERR_INVALID_ARG;
    if ((w >> (L - 1)) < 1 || (h >> (L - 1)) < 1) return VETRAST_ERR_INVALID_ARG;  // coarsest layer must not be empty
    // fragment positions and pixel numbers are 32-bit; with 4 hits the point id shares a key word with the corner
    if (N * L * hits >= (int64_t)0xFFFFFFF0ll) return VETRAST_ERR_INVALID_ARG;
    if (hits > 1 && N > (int64_t)(1 << 30)) return VETRAST_ERR_INVALID_ARG;
    int64_t P = 0;
    int lw = w, lh = h;
    for (int l = 0; l < L; ++l, lw /= 2, lh /= 2)
        P += (int64_t)((lw + kTile - 1) / kTile) * ((lh + kTile - 1) / kTile) * kTilePixels;
    if (P + kScanPerBlock >= (int64_t)0x7FFFFFFFll) return VETRAST_ERR_INVALID_ARG;
    return VETRAST_OK;
}

// `for_backward`: the masks are not read or written by the backward pass, so their pointers may be missing there.
int validate_forward(const vetrast_forward_args* a, vetrast_workspace_layout* lay, bool for_backward = false)
{
    if (!a) return VETRAST_ERR_INVALID_ARG;
    const vetrast_params& p = a->params;
    if (!a->position || !a->texture || !a->confidence || !a->background || !a->poses_se3 || !a->intrinsics ||
        !a->views || !a->workspace)
        return VETRAST_ERR_INVALID_ARG;
    if (a->num_views < 1 || a->num_poses < 1 || a->num_cameras < 1) return VETRAST_ERR_INVALID_ARG;
    if (p.num_texture_channels < 1 || p.num_texture_channels > VETRAST_MAX_CHANNELS) return VETRAST_ERR_INVALID_ARG;
    if (p.check_normal) return VETRAST_ERR_UNSUPPORTED;
    int st = check_mode(p.render_mode);
    if (st != VETRAST_OK) return st;
    // FUZZY_BLEND: a range <= 0 divides 0 by 0 in the reference's first bucket; the kernels rely on range < 1e4
    if (p.render_mode == VETRAST_RENDER_FUZZY_BLEND && !(p.depth_accept_blend > 0.f && p.depth_accept_blend < 1e4f))
        return VETRAST_ERR_INVALID_ARG;
    const int w = a->views[0].w, h = a->views[0].h;
    st          = check_dims(a->num_points, a->num_views, p.num_layers, w, h, hits_of_mode(p.render_mode));
    if (st != VETRAST_OK) return st;
    for (int b = 0; b < a->num_views; ++b)
    {
        const vetrast_view& v = a->views[b];
        if (v.camera_model_type != VETRAST_CAMERA_PINHOLE_DISTORTION) return VETRAST_ERR_UNSUPPORTED;
        if (v.w != w || v.h != h) return VETRAST_ERR_INVALID_ARG;
        if (v.image_index < 0 || v.image_index >= a->num_poses) return VETRAST_ERR_INVALID_ARG;
        if (v.camera_index < 0 || v.camera_index >= a->num_cameras) return VETRAST_ERR_INVALID_ARG;
    }
    for (int l = 0; l < p.num_layers; ++l)
    {
        if (!a->out[l]) return VETRAST_ERR_INVALID_ARG;
        if (p.output_background_mask && !for_backward && !a->out_mask[l]) return VETRAST_ERR_INVALID_ARG;
    }
    if (((uintptr_t)a->workspace % kAlign) != 0 || ((uintptr_t)a->position % 16) != 0) return VETRAST_ERR_INVALID_ARG;
    if (((uintptr_t)a->packed_descriptors % 32) != 0) return VETRAST_ERR_INVALID_ARG;
    st = vetrast_workspace_layout_for_mode(a->num_points, a->num_views, p.num_layers, w, h, p.render_mode, lay);
    if (st != VETRAST_OK) return st;
    const size_t need = a->save_for_backward ? lay->total_bytes : lay->forward_only_bytes;
    if (a->workspace_bytes < need) return VETRAST_ERR_WORKSPACE_SMALL;
    return VETRAST_OK;
}

template <class T>
inline T* ws_ptr(void* ws, size_t off)
{
    return reinterpret_cast<T*>(static_cast<char*>(ws) + off);
}

// `list_bound[l]`: an upper bound of the mean number of fragments a pixel of layer l blends (null: no layer is split;
// `split_all`: every layer is, which is what buffers are sized for).
// The overflow log: workgroup w of the scatter pass appends to segment w % kLogSegments, so a segment needs room for
// every hit of ceil(workgroups / kLogSegments) workgroups.
uint32_t log_segment_records(int64_t N, int L, int hits)
{
    const int64_t groups = (N + kBlock - 1) / kBlock;
    return (uint32_t)((groups + kLogSegments - 1) / kLogSegments * kBlock * L * hits);
}
size_t log_records(int64_t N, int L, int hits) { return (size_t)log_segment_records(N, L, hits) * kLogSegments; }
size_t log_cursor_bytes(int B) { return (size_t)B * kLogSegments * kLogCursorStride * sizeof(uint32_t); }

// Per-workgroup pose / intrinsics rows one view's per-point backward pass leaves.
size_t camera_rows_bytes(int64_t N)
{
    return align_up(((size_t)N + kBlock - 1) / kBlock * kCameraRow * sizeof(double), kAlign);
}

TileMap make_tile_map(const LayerTable& ly, const double* list_bound = nullptr, bool split_all = false)
{
    TileMap m;
    std::memset(&m, 0, sizeof(m));
    m.L = ly.L;
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
        m.split[l] = (split_all || (list_bound && l < ly.L && list_bound[l] >= kSplitListLength)) ? 4u : 1u;
    // a region is one 16x16 tile of the coarsest layer; over the finer layers it covers (16 << k)^2 pixels. Layer sizes
    // come from integer halving, so the finest layer can be a few pixels larger than 2^(L-1) times the coarsest one:
    // size the region grid from the finest layer.
    const uint32_t span = (uint32_t)kTile << (ly.L - 1);
    m.regions_x         = ((uint32_t)ly.w[0] + span - 1) / span;
    m.regions           = m.regions_x * (((uint32_t)ly.h[0] + span - 1) / span);
    uint32_t tiles      = 0;
    for (int k = 0; k < ly.L; ++k) tiles += 1u << (2 * k);
    m.tiles_per_region = tiles;
    m.regions_per_xcd  = (m.regions + kXcds - 1) / kXcds;
    m.groups_per_region = 0;
    for (int l = 0; l < ly.L; ++l) m.groups_per_region += (1u << (2 * (ly.L - 1 - l))) * m.split[l];
    return m;
}

uint32_t tile_grid(const TileMap& m)
{
    return m.regions_per_xcd * m.groups_per_region * kXcds;
}

ViewPass make_view_pass(const vetrast_forward_args* a, const vetrast_workspace_layout& lay, const LayerTable& ly, int b)
{
    ViewPass vp;
    vp.position         = reinterpret_cast<const float4*>(a->position);
    vp.index            = a->index;
    vp.confidence       = a->confidence;
    vp.dropout          = a->dropout ? a->dropout + (size_t)b * a->num_points : nullptr;
    vp.view             = ws_ptr<DeviceView>(a->workspace, lay.views_base) + b;
    vp.ly               = ly;
    vp.N                = a->num_points;
    vp.drop_by_radius   = a->params.drop_out_points_by_radius;
    vp.radius_threshold = a->params.drop_out_radius_threshold;
    vp.viewer_only      = a->params.viewer_only;
    vp.stability_cutoff = a->params.stability_cutoff_value;
    vp.confidence_activation = a->params.confidence_activation;
    vp.confidence_scale      = a->params.confidence_scale;
    vp.point_order = a->point_order;
    vp.projected = lay.projected_stride ? ws_ptr<float2>(a->workspace, lay.projected_base + lay.projected_stride * b) : nullptr;
    return vp;
}

// Scratch of vetrast_lift_error_static: the workspace vetrast_lift_error takes from its caller, as an array of the
// library's own, sized for VETRAST_LIFT_STATIC_MAX_CELLS cells. Every GPU the library runs on holds a copy of its own
// until the process ends. In host code this name only stands for the symbol: the device address is looked up once per
// device (scratch_of_device) and only that pointer is handed to kernels.
constexpr size_t kLiftStaticBytes = lift_workspace_bytes_for((size_t)VETRAST_LIFT_STATIC_MAX_CELLS);
static __device__ __align__(256) unsigned char scratch[kLiftStaticBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
char* g_scratch_ptr[kMaxDevices] = {};

// Address of the scratch array on `device`, which must be the current device. hipSuccess and a non-null pointer on
// success.
hipError_t scratch_of_device(int device, char** out)
{
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device])
    {
        void* p      = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p || (reinterpret_cast<uintptr_t>(p) % kAlign) != 0) return hipErrorInvalidSymbol;
        g_scratch_ptr[device] = static_cast<char*>(p);
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

// Argument checks of the error lifting that do not concern the workspace. VETRAST_OK with *nothing_to_do set for an
// empty grid.
int validate_lift(const vetrast_lift_args* a, bool* nothing_to_do)
{
    *nothing_to_do = false;
    if (a->num_cells < 0 || a->num_cells > (int64_t)1 << 30) return VETRAST_ERR_INVALID_ARG;
    if (a->channels < 1 || a->height < 1 || a->width < 1 || a->border_pixels < 0) return VETRAST_ERR_INVALID_ARG;
    // pixel numbers inside a cell's box go through float arithmetic that is exact below 2^24
    if ((int64_t)a->height * a->width >= (int64_t)1 << 24) return VETRAST_ERR_INVALID_ARG;
    const vetrast_view& v = a->view;
    if (v.camera_model_type != VETRAST_CAMERA_PINHOLE_DISTORTION) return VETRAST_ERR_UNSUPPORTED;
    if (v.image_index < 0 || v.image_index >= a->num_poses) return VETRAST_ERR_INVALID_ARG;
    if (v.camera_index < 0 || v.camera_index >= a->num_cameras) return VETRAST_ERR_INVALID_ARG;
    if (a->num_cells == 0)
    {
        *nothing_to_do = true;
        return VETRAST_OK;
    }
    if (!a->cell_bb_min || !a->cell_bb_length || !a->cell_value || !a->cell_access_count || !a->poses_se3 ||
        !a->intrinsics || !a->loss_image)
        return VETRAST_ERR_INVALID_ARG;
    return VETRAST_OK;
}

// The five launches of the error lifting with their scratch at `ws` (lift_workspace_bytes_for(num_cells) bytes,
// 256-byte aligned). Every word of the scratch a kernel reads has been written by an earlier kernel of the same call
// (the prepare kernel empties the queue, a slot's sum is cleared when the slot is taken), so nothing needs clearing
// between calls that share one scratch.
void launch_lift(const vetrast_lift_args* a, char* ws, hipStream_t stream)
{
    const vetrast_view& v = a->view;
    LiftPass lp;
    lp.bb_min       = a->cell_bb_min;
    lp.bb_length    = a->cell_bb_length;
    lp.value        = a->cell_value;
    lp.access_count = a->cell_access_count;
    lp.loss         = a->loss_image;
    lp.num_cells    = a->num_cells;
    lp.channels     = a->channels;
    lp.height       = a->height;
    lp.width        = a->width;
    lp.border       = a->border_pixels;
    lp.view         = reinterpret_cast<const DeviceView*>(ws);
    lp.queue_length = reinterpret_cast<uint32_t*>(ws + VETRAST_LIFT_QUEUE_LENGTH_OFFSET);
    lp.queue        = reinterpret_cast<uint2*>(ws + kLiftHeader);
    lp.sums = reinterpret_cast<double*>(ws + kLiftHeader + align_up((size_t)a->num_cells * sizeof(uint2), kAlign));
    lp.starts = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(lp.sums) +
                                                      align_up((size_t)a->num_cells * sizeof(double), kAlign));
    uint32_t* flags = reinterpret_cast<uint32_t*>(ws + VETRAST_LIFT_FLAGS_OFFSET);

    ViewSource src;
    src.image_index  = v.image_index;
    src.camera_index = v.camera_index;
    src.w            = v.w;
    src.h            = v.h;
    for (int j = 0; j < 5; ++j) src.crop[j] = v.crop_transform[j];
    for (int j = 0; j < 4; ++j) src.rot[j] = v.crop_rotation[j];

    hipLaunchKernelGGL(lift_prepare_kernel, dim3(1), dim3(kWave), 0, stream, src, a->poses_se3, a->intrinsics,
                       reinterpret_cast<DeviceView*>(ws), lp.queue_length, flags);
    const int waves_per_block = kBlock / kWave;
    hipLaunchKernelGGL(lift_cells_kernel, dim3((unsigned)((a->num_cells + waves_per_block - 1) / waves_per_block)),
                       dim3(kBlock), 0, stream, lp);
    // The queue length stays on the device, so the shared pass is launched at a fixed width and splits the chunks
    // it finds evenly.
    hipLaunchKernelGGL(lift_scan_kernel, dim3(1), dim3(kLiftScanBlock), 0, stream, lp);
    hipLaunchKernelGGL(lift_queued_kernel, dim3(2048), dim3(kBlock), 0, stream, lp);
    hipLaunchKernelGGL(lift_finish_kernel, dim3((unsigned)std::min<int64_t>(grid_for((size_t)a->num_cells), 256)),
                       dim3(kBlock), 0, stream, lp);
}

}  // namespace

extern "C" {

int vetrast_create(vetrast_ctx** out_ctx)
{
    if (!out_ctx) return VETRAST_ERR_INVALID_ARG;
    *out_ctx         = nullptr;
    vetrast_ctx* ctx = new (std::nothrow) vetrast_ctx();
    if (!ctx) return VETRAST_ERR_INVALID_ARG;
    hipError_t e = hipGetDevice(&ctx->device);
    if (e != hipSuccess)
    {
        vetrast_destroy(ctx);
        return VETRAST_ERR_HIP;
    }
    // this device's address of the scratch array of vetrast_lift_error_static, looked up once per device
    e = scratch_of_device(ctx->device, &ctx->lift_scratch);
    if (e != hipSuccess)
    {
        vetrast_destroy(ctx);
        return VETRAST_ERR_HIP;
    }
    *out_ctx = ctx;
    return VETRAST_OK;
}

void vetrast_destroy(vetrast_ctx* ctx)
{
    if (!ctx) return;
    for (auto& s : ctx->spans)
    {
        (void)hipEventDestroy(s.start);
        (void)hipEventDestroy(s.stop);
    }
    for (auto e : ctx->free_events) (void)hipEventDestroy(e);
    delete ctx;
}

int vetrast_layer_sizes(int32_t w, int32_t h, int32_t num_layers, int32_t* layer_w, int32_t* layer_h)
{
    if (!layer_w || !layer_h || num_layers < 1 || num_layers > VETRAST_MAX_LAYERS || w < 1 || h < 1)
        return VETRAST_ERR_INVALID_ARG;
    for (int l = 0; l < num_layers; ++l)
    {
        layer_w[l] = w;
        layer_h[l] = h;
        w /= 2;
        h /= 2;
    }
    return VETRAST_OK;
}

int vetrast_workspace_layout_for(int32_t N, int32_t B, int32_t L, int32_t w, int32_t h, vetrast_workspace_layout* lay)
{
    return vetrast_workspace_layout_for_mode(N, B, L, w, h, VETRAST_RENDER_FULL_BLEND, lay);
}

int vetrast_workspace_layout_for_mode(int32_t N, int32_t B, int32_t L, int32_t w, int32_t h, int32_t render_mode,
                                      vetrast_workspace_layout* lay)
{
    if (!lay) return VETRAST_ERR_INVALID_ARG;
    int st = check_mode(render_mode);
    if (st != VETRAST_OK) return st;
    const int hits = hits_of_mode(render_mode);
    st             = check_dims(N, B, L, w, h, hits);
    if (st != VETRAST_OK) return st;
    std::memset(lay, 0, sizeof(*lay));
    LayerTable t = make_layer_table(w, h, L, (int64_t)N * hits);
    for (int l = 0; l < L; ++l)
    {
        lay->layer_w[l] = t.w[l];
        lay->layer_h[l] = t.h[l];
    }
    for (int l = 0; l < L; ++l) lay->layer_tiles_x[l] = t.tiles_x[l];
    for (int l = 0; l <= VETRAST_MAX_LAYERS; ++l)
    {
        lay->layer_tile_base[l]  = t.tile_base[l < L ? l : L];
        lay->layer_pixel_base[l] = t.base[l < L ? l : L];
    }
    const size_t P         = t.base[L];
    const size_t bins      = t.bin_base[L];
    const size_t Tpad      = align_up(bins + 1, kScanPerBlock);
    lay->num_bins          = (int64_t)bins;
    const size_t cap       = (size_t)N * L * hits;
    lay->fragment_capacity = (int64_t)cap;
    lay->hits_per_layer    = hits;
    size_t at              = 0;
    lay->flags_base        = at;
    at += kAlign;
    lay->bin_counts_base   = at;
    lay->bin_counts_stride = 2 * Tpad * sizeof(uint32_t);  // the counts, and behind them room for their scan
    at += lay->bin_counts_stride * B;
    lay->log_cursor_base = at;  // right behind the bin counters: one zero-fill covers both
    at += log_cursor_bytes(B);
    // scratch that exists once per lane (the views that share a launch), see vetrast_workspace_layout::view_lanes
    const int lanes            = std::min(B, kViewLanes);
    lay->view_lanes            = lanes;
    lay->scan_partials_base    = at;
    lay->scan_partials_stride  = align_up((Tpad / kScanPerBlock) * sizeof(uint32_t), kAlign);
    at += lay->scan_partials_stride * lanes;
    lay->offsets_base   = at;
    lay->offsets_stride = align_up((P + 1) * sizeof(uint32_t), kAlign);
    at += lay->offsets_stride * B;
    const size_t record_bytes = compact_records(N, hits) ? sizeof(uint2) : sizeof(uint4);
    lay->binned_base   = at;
    lay->binned_stride = align_up(cap * record_bytes, kAlign);
    at += lay->binned_stride * lanes;
    lay->primary_base   = at;
    lay->primary_stride = align_up((size_t)t.room_base[L] * record_bytes, kAlign);
    at += lay->primary_stride * lanes;
    lay->views_base = at;
    at += align_up((size_t)B * sizeof(DeviceView), kAlign);
    lay->packed_base = at;
    at += align_up((size_t)N * kPackedFloats * sizeof(float), kAlign);
    lay->weight_base   = at;
    lay->weight_stride = align_up(P * sizeof(float), kAlign);
    at += lay->weight_stride * B;
    lay->kept_base   = at;
    lay->kept_stride = align_up(P * sizeof(uint32_t), kAlign);
    at += lay->kept_stride * B;
    lay->cut_flags_base   = at;
    lay->cut_flags_stride = align_up(P, kAlign);
    at += lay->cut_flags_stride * B;
    lay->fragments_base   = at;
    lay->fragments_stride = align_up(cap * sizeof(uint64_t), kAlign);
    at += lay->fragments_stride * B;
    lay->transmittance_base   = at;
    lay->transmittance_stride = align_up(cap * sizeof(float), kAlign);
    at += lay->transmittance_stride * B;
    lay->last_key_base   = at;
    lay->last_key_stride = align_up(P * sizeof(uint64_t), kAlign);
    at += lay->last_key_stride * B;
    lay->projected_base   = at;
    lay->projected_stride = hits == 4 ? align_up((size_t)N * sizeof(float2), kAlign) : 0;
    at += lay->projected_stride * B;
    // The overflow log (written by the scatter pass, emptied by overflow_move_kernel before the build pass of the same
    // view) is dead once the forward call is over: the scratch of the backward call lies on top of it.
    // One such block per lane, lane_scratch_stride apart.
    const size_t shared_base = align_up(at, kAlign);
    lay->log_base            = shared_base;
    at                       = shared_base + align_up(log_records(N, L, hits) * sizeof(uint4), kAlign);
    lay->slots_base          = at;
    at += align_up(log_records(N, L, hits) * sizeof(uint32_t), kAlign);
    const size_t forward_block = align_up(at, kAlign) - shared_base;
    at                         = shared_base;
    lay->partial_base          = at;
    at += align_up(cap * 8 * sizeof(float), kAlign);
    lay->background_partial_base = at;
    // (the FUZZY_BLEND kernel that takes a wave per list keeps rows per replica and kFuzzyFoldRows rows they are folded into)
    at += align_up(((size_t)tile_grid(make_tile_map(t, nullptr, true)) * kFuzzyReplicas + kFuzzyFoldRows) * kBackgroundRow * sizeof(float), kAlign);
    const size_t backward_block = align_up(at, kAlign) - shared_base;
    lay->lane_scratch_stride    = std::max(forward_block, backward_block);
    lay->forward_only_bytes     = shared_base + lay->lane_scratch_stride * (lanes - 1) + forward_block;
    at                          = shared_base + lay->lane_scratch_stride * lanes;
    lay->camera_partial_base = at;  // (a block of rows per view of a round, see camera_rows_bytes)
    at += camera_rows_bytes(N) * lanes;
    lay->total_bytes = std::max(align_up(at, kAlign), lay->forward_only_bytes);
    return VETRAST_OK;
}

size_t vetrast_forward_workspace_bytes(int32_t N, int32_t B, int32_t L, int32_t w, int32_t h)
{
    vetrast_workspace_layout lay;
    if (vetrast_workspace_layout_for(N, B, L, w, h, &lay) != VETRAST_OK) return 0;
    return lay.total_bytes;
}

namespace
{
// Whether the caller expects a view of the call to see a small part of the cloud: a third of the fragments every
// point in every layer would leave, or less. False where it has not said (expected_fragments).
bool views_see_little(const vetrast_params& p, int N, int hits)
{
    double expected = 0.0;
    for (int l = 0; l < p.num_layers; ++l)
    {
        if (!(p.expected_fragments[l] > 0.f)) return false;
        expected += p.expected_fragments[l];
    }
    return expected < (double)N * hits * p.num_layers / 3.0;
}
}  // namespace

int vetrast_forward(vetrast_ctx* ctx, const vetrast_forward_args* a, void* stream_)
{
    if (!ctx) return VETRAST_ERR_INVALID_ARG;
    vetrast_workspace_layout lay;
    int st = validate_forward(a, &lay);
    if (st != VETRAST_OK) return st;
    hipStream_t stream      = (hipStream_t)stream_;
    const vetrast_params& p = a->params;
    const int N = a->num_points, B = a->num_views, L = p.num_layers, C = p.num_texture_channels;
    const int hits      = hits_of_mode(p.render_mode);
    const LayerTable ly = make_call_layer_table(a->views[0].w, a->views[0].h, L, (int64_t)N * hits, p.expected_fragments);
    const uint32_t bins = ly.bin_base[L];
    const size_t Tpad   = lay.bin_counts_stride / sizeof(uint32_t) / 2;  // counts per view; as many words behind them
    void* ws            = a->workspace;
    uint32_t* flags     = ws_ptr<uint32_t>(ws, lay.flags_base);
    // the caller's descriptor records where it keeps them current itself, else the workspace's, written by this call
    const bool own_pack  = a->packed_descriptors == nullptr;
    float4* packed       = own_pack ? ws_ptr<float4>(ws, lay.packed_base)
                                    : reinterpret_cast<float4*>(const_cast<float*>(a->packed_descriptors));
    DeviceView* views   = ws_ptr<DeviceView>(ws, lay.views_base);

    {
        ScopeTimer tm(ctx, stream, VETRAST_SCOPE_PREPARE);
        // per-bin counters of all views (contiguous) start at zero; InitializeData, PointRenderer.cu:402-470
        const size_t n4  = (2 * Tpad * B * sizeof(uint32_t) + log_cursor_bytes(B)) / sizeof(uint4);
        uint4* counters4 = ws_ptr<uint4>(ws, lay.bin_counts_base);
        const int zero_blocks = std::min(grid_for(n4), 1024);
        for (int first = 0; first < B; first += 16)
        {
            PrepareViewsArgs pv;
            const int cnt = std::min(16, B - first);
            for (int k = 0; k < cnt; ++k)
            {
                const vetrast_view& v = a->views[first + k];
                ViewSource& s         = pv.src[k];
                s.image_index         = v.image_index;
                s.camera_index        = v.camera_index;
                s.w                   = v.w;
                s.h                   = v.h;
                for (int j = 0; j < 5; ++j) s.crop[j] = v.crop_transform[j];
                for (int j = 0; j < 4; ++j) s.rot[j] = v.crop_rotation[j];
            }
            hipLaunchKernelGGL(prepare_views_kernel, dim3(1 + (first == 0 ? zero_blocks : 0)), dim3(kBlock), 0, stream, pv,
                               first, cnt, a->poses_se3, a->intrinsics, views, flags, counters4, n4, a->background, C,
                               p.texture_abs, p.allow_distortion);
        }
    }

    // Views in rounds of up to view_lanes: every kernel takes the views of a round in one launch (each view with the
    // scratch of its lane).
    const int lanes          = std::max(1, lay.view_lanes);
    const bool scan_and_move = bins + 1 <= (uint32_t)kScanMoveMax;
    // The descriptor interleave rides on the scatter pass of the first view, which takes every row; or, where row,
    // point and thread are the same number (no texture index, no processing order), on that of every view, each for
    // the rows of the points it sees (only fragments ever read a row; views that see the same point write the same
    // bytes): with one view, and with several where the caller expects each to see little of the cloud.
    const bool rows_of_visible_points =
        a->index == nullptr && a->point_order == nullptr && (B == 1 || views_see_little(p, N, hits));
    for (int first = 0; first < B; first += lanes)
    {
        const int last = std::min(B, first + lanes), count = last - first;
        const bool one = count == 1;
        PerView<ScatterArgs> scatter{};
        PerView<ScanArgs> scan{};
        PerView<BuildPass> build{};
        for (int b = first; b < last; ++b)
        {
            const size_t lane = (size_t)(b - first);
            ScatterArgs& sc   = scatter.v[lane];
            sc.view           = make_view_pass(a, lay, ly, b);
            sc.bin_counts     = ws_ptr<uint32_t>(ws, lay.bin_counts_base + lay.bin_counts_stride * b);
            ScatterTargets& targets  = sc.out;
            targets.primary          = ws_ptr<uint4>(ws, lay.primary_base + lay.primary_stride * lane);
            targets.compact          = compact_records(N, hits) ? 1 : 0;
            targets.log              = ws_ptr<uint4>(ws, lay.log_base + lay.lane_scratch_stride * lane);
            targets.log_rank         = ws_ptr<uint32_t>(ws, lay.slots_base + lay.lane_scratch_stride * lane);
            targets.log_cursor       = ws_ptr<uint32_t>(ws, lay.log_cursor_base) + (size_t)b * kLogSegments * kLogCursorStride;
            targets.segment_capacity = log_segment_records(N, L, hits);
            // the scatter pass of the first view also interleaves the descriptors (PrepareTexture / PrepareConfidence included)
            PackJob& pack              = sc.pack;
            pack.texture               = a->texture;
            pack.confidence            = a->confidence;
            pack.packed                = (own_pack && (b == 0 || rows_of_visible_points)) ? packed : nullptr;
            pack.N                     = N;
            pack.C                     = C;
            pack.confidence_activation = p.confidence_activation;
            pack.confidence_scale      = p.confidence_scale;
            pack.texture_abs           = p.texture_abs;
            pack.visible_only          = rows_of_visible_points ? 1 : 0;

            // Where the bins of a view are few enough, one launch scans their counts and files the logged records (the
            // scan lands behind the counts); otherwise the scan runs in place and the move kernel follows.
            ScanArgs& sa      = scan.v[lane];
            sa.bin_counts     = sc.bin_counts;
            sa.scanned_behind = (uint32_t)Tpad;
            sa.n              = bins + 1;
            sa.partials       = ws_ptr<uint32_t>(ws, lay.scan_partials_base + lay.scan_partials_stride * lane);
            sa.in             = targets;
            sa.binned         = ws_ptr<uint4>(ws, lay.binned_base + lay.binned_stride * lane);
            sa.capacity       = (uint32_t)lay.fragment_capacity;

            BuildPass& bp          = build.v[lane];
            bp.bin_offsets         = scan_and_move ? sc.bin_counts + Tpad : sc.bin_counts;
            bp.primary             = targets.primary;
            bp.binned              = sa.binned;
            bp.compact_records     = targets.compact;
            bp.offsets             = ws_ptr<uint32_t>(ws, lay.offsets_base + lay.offsets_stride * b);
            bp.fragments           = ws_ptr<uint64_t>(ws, lay.fragments_base + lay.fragments_stride * b);
            bp.list_is_cut         = ws_ptr<uint8_t>(ws, lay.cut_flags_base + lay.cut_flags_stride * b);
            bp.last_key            = ws_ptr<uint64_t>(ws, lay.last_key_base + lay.last_key_stride * b);
            bp.kept                = ws_ptr<uint32_t>(ws, lay.kept_base + lay.kept_stride * b);
            bp.projected           = sc.view.projected;
            bp.index               = a->index;
            bp.packed              = packed;
            bp.background          = reinterpret_cast<const float*>(flags) + kPreparedBackgroundOffset;
            bp.transmittance       = a->save_for_backward ? ws_ptr<float>(ws, lay.transmittance_base + lay.transmittance_stride * b) : nullptr;
            bp.weight              = ws_ptr<float>(ws, lay.weight_base + lay.weight_stride * b);
            bp.ly                  = ly;
            bp.num_bins            = bins;
            bp.N                   = N;
            bp.K                   = p.debug_max_list_length;
            bp.use_environment_map = p.use_environment_map;
            bp.mask_value          = p.output_background_mask_value;
            bp.depth_accept        = p.depth_accept_blend;
            for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
            {
                bp.out[l] = bp.out_mask[l] = bp.out_weight[l] = nullptr;
                if (l >= L) continue;
                const size_t plane = (size_t)ly.w[l] * ly.h[l];
                bp.out[l]          = a->out[l] + (size_t)b * C * plane;
                if (p.output_background_mask) bp.out_mask[l] = a->out_mask[l] + (size_t)b * plane;
                if (a->out_weight[l]) bp.out_weight[l] = a->out_weight[l] + (size_t)b * plane;
            }
        }
        const dim3 blk(kBlock);
        const unsigned views_y = (unsigned)count;
        if (N > 0)
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_COUNT);
            const ScatterArgs& sc = scatter.v[0];
            const dim3 g(grid_for(N)), gv(grid_for(N), views_y);
            if (hits == 1 && one)
                hipLaunchKernelGGL(bin_scatter_kernel<1>, g, blk, 0, stream, sc.view, sc.bin_counts, sc.out, sc.pack);
            else if (hits == 1)
                hipLaunchKernelGGL(bin_scatter_views_kernel<1>, gv, blk, 0, stream, scatter);
            else if (one)
                hipLaunchKernelGGL(bin_scatter_kernel<4>, g, blk, 0, stream, sc.view, sc.bin_counts, sc.out, sc.pack);
            else
                hipLaunchKernelGGL(bin_scatter_views_kernel<4>, gv, blk, 0, stream, scatter);
        }
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_SCAN);
            const ScanArgs& sa = scan.v[0];
            if (scan_and_move)
            {
                if (one)
                    hipLaunchKernelGGL(scan_move_kernel, dim3(kLogSegments), blk, 0, stream,
                                       reinterpret_cast<const uint4*>(sa.bin_counts), sa.n,
                                       reinterpret_cast<uint4*>(sa.bin_counts + Tpad), sa.in, sa.binned, sa.capacity);
                else
                    hipLaunchKernelGGL(scan_move_views_kernel, dim3(kLogSegments, views_y), blk, 0, stream, scan);
            }
            else
            {
                const unsigned blocks = (unsigned)(Tpad / kScanPerBlock);
                if (one)
                {
                    hipLaunchKernelGGL(scan_partials_kernel, dim3(blocks), blk, 0, stream,
                                       reinterpret_cast<const uint4*>(sa.bin_counts), sa.partials);
                    hipLaunchKernelGGL(scan_apply_kernel, dim3(blocks), blk, 0, stream,
                                       reinterpret_cast<uint4*>(sa.bin_counts), sa.partials);
                }
                else
                {
                    hipLaunchKernelGGL(scan_partials_views_kernel, dim3(blocks, views_y), blk, 0, stream, scan);
                    hipLaunchKernelGGL(scan_apply_views_kernel, dim3(blocks, views_y), blk, 0, stream, scan);
                }
            }
        }
        if (N > 0 && !scan_and_move)
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_FILL);
            // the few records beyond their bin's own room, if any
            const ScanArgs& sa = scan.v[0];
            if (one)
                hipLaunchKernelGGL(overflow_move_kernel, dim3(256), blk, 0, stream, sa.in, sa.bin_counts, sa.binned, sa.capacity);
            else
                hipLaunchKernelGGL(overflow_move_views_kernel, dim3(256, views_y), blk, 0, stream, scan);
        }
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BUILD);
            const BuildPass& bp = build.v[0];
            const dim3 g(bins), gv(bins, views_y);
            auto launch = [&](auto channels, auto bilinear, auto fuzzy) {
                constexpr int kC         = decltype(channels)::value;
                constexpr bool kBilinear = decltype(bilinear)::value, kFuzzy = decltype(fuzzy)::value;
                if (one)
                    hipLaunchKernelGGL((bin_build_kernel<kC, kBilinear, kFuzzy>), g, blk, 0, stream, bp);
                else
                    hipLaunchKernelGGL((bin_build_views_kernel<kC, kBilinear, kFuzzy>), gv, blk, 0, stream, build);
            };
            auto with_channels = [&](auto bilinear, auto fuzzy) {
                switch (C)
                {
                    case 1: launch(std::integral_constant<int, 1>{}, bilinear, fuzzy); break;
                    case 2: launch(std::integral_constant<int, 2>{}, bilinear, fuzzy); break;
                    case 3: launch(std::integral_constant<int, 3>{}, bilinear, fuzzy); break;
                    default: launch(std::integral_constant<int, 4>{}, bilinear, fuzzy); break;
                }
            };
            if (p.render_mode == VETRAST_RENDER_FUZZY_BLEND)
                with_channels(std::false_type{}, std::true_type{});
            else if (hits == 1)
                with_channels(std::false_type{}, std::false_type{});
            else
                with_channels(std::true_type{}, std::false_type{});
        }
    }
    VET_HIP(ctx, hipGetLastError());
    return VETRAST_OK;
}

int vetrast_backward(vetrast_ctx* ctx, const vetrast_backward_args* g, void* stream_)
{
    if (!ctx || !g) return VETRAST_ERR_INVALID_ARG;
    const vetrast_forward_args* a = &g->fwd;
    vetrast_workspace_layout lay;
    int st = validate_forward(a, &lay, /*for_backward=*/true);
    if (st != VETRAST_OK) return st;
    if (!a->save_for_backward) return VETRAST_ERR_INVALID_ARG;
    if (!g->grad_texture || !g->grad_confidence || !g->grad_background) return VETRAST_ERR_INVALID_ARG;
    if (g->grad_points && !g->grad_point_count) return VETRAST_ERR_INVALID_ARG;
    if (g->grad_points && ((uintptr_t)g->grad_points % 16) != 0) return VETRAST_ERR_INVALID_ARG;
    if (g->grad_pose && !g->grad_pose_count) return VETRAST_ERR_INVALID_ARG;
    if (g->grad_intrinsics && !g->grad_intrinsics_count) return VETRAST_ERR_INVALID_ARG;
    const vetrast_params& p = a->params;
    for (int l = 0; l < p.num_layers; ++l)
        if (!g->grad_out[l]) return VETRAST_ERR_INVALID_ARG;
    hipStream_t stream = (hipStream_t)stream_;
    const int N = a->num_points, B = a->num_views, L = p.num_layers, C = p.num_texture_channels;
    const int hits      = hits_of_mode(p.render_mode);
    const LayerTable ly = make_call_layer_table(a->views[0].w, a->views[0].h, L, (int64_t)N * hits, p.expected_fragments);
    // fragments a pixel of layer l blends, bounded from above without a device read: all points land in the layer, the
    // top-K cut
    double list_bound[VETRAST_MAX_LAYERS] = {};
    for (int l = 0; l < L; ++l)
    {
        list_bound[l] = (double)N * hits / ((double)ly.w[l] * ly.h[l]);
        if (p.debug_max_list_length > 0) list_bound[l] = std::min(list_bound[l], (double)p.debug_max_list_length);
    }
    const TileMap tiles = make_tile_map(ly, list_bound);
    void* ws            = a->workspace;

    // The per-point kernel overwrites every gradient row in the first view, so the zeros_like fills of
    // PointRenderer.cu:267-277 are only needed where rows are added to with atomics: with a texture index
    // indirection, where several points may share a row.
    const bool add_to_rows = a->index != nullptr;
    ClearJob clear          = {};
    constexpr size_t kClearByKernel = 16384;  // words one workgroup clears in passing
    {
        ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_PREPARE);
        auto zero = [&](float* ptr, size_t n) {
            if (!ptr || n == 0) return;
            hipLaunchKernelGGL(fill_u32_kernel, dim3(std::min(grid_for(n), 8192)), dim3(kBlock), 0, stream,
                               reinterpret_cast<uint32_t*>(ptr), n, 0u);
        };
        // the pose and intrinsics accumulators: by the first view's per-pixel kernel where they are small (ClearJob)
        const size_t pose_words = (size_t)12 * a->num_poses, camera_words = (size_t)13 * a->num_cameras;
        if (g->grad_pose)
        {
            if (pose_words <= kClearByKernel)
            {
                clear.ptr[0] = reinterpret_cast<uint32_t*>(g->grad_pose), clear.count[0] = (uint32_t)pose_words;
                clear.ptr[1] = reinterpret_cast<uint32_t*>(g->grad_pose_count), clear.count[1] = (uint32_t)a->num_poses;
            }
            else
            {
                zero(reinterpret_cast<float*>(g->grad_pose), pose_words);
                zero(g->grad_pose_count, (size_t)a->num_poses);
            }
        }
        if (g->grad_intrinsics)
        {
            if (camera_words <= kClearByKernel)
            {
                clear.ptr[2] = reinterpret_cast<uint32_t*>(g->grad_intrinsics), clear.count[2] = (uint32_t)camera_words;
                clear.ptr[3] = reinterpret_cast<uint32_t*>(g->grad_intrinsics_count), clear.count[3] = (uint32_t)a->num_cameras;
            }
            else
            {
                zero(g->grad_intrinsics, camera_words);
                zero(g->grad_intrinsics_count, (size_t)a->num_cameras);
            }
        }
        if (add_to_rows)
        {
            zero(g->grad_texture, (size_t)C * N);
            zero(g->grad_confidence, (size_t)N);
            if (g->grad_points)
            {
                zero(g->grad_points, (size_t)4 * N);
                zero(g->grad_point_count, (size_t)N);
            }
        }
    }
    // position, pose and intrinsics gradients all hang off the per-fragment image-space gradient
    // (src/lib/rendering/RenderBackward.cu:1183, 1401-1459)
    const bool want_camera         = p.need_point_gradient && (g->grad_pose || g->grad_intrinsics) && N > 0;
    const bool want_image_gradient = p.need_point_gradient && (g->grad_points || g->grad_pose || g->grad_intrinsics);
    double* camera_rows            = ws_ptr<double>(ws, lay.camera_partial_base);
    const bool fuzzy_long  = p.render_mode == VETRAST_RENDER_FUZZY_BLEND &&
                            (p.debug_max_list_length <= 0 || p.debug_max_list_length > kFuzzyDense);
    // Layout of the gradient records (gradient_record): point after point where the caller expects the views to see a
    // small part of the cloud, layer after layer otherwise and where nothing is known.
    const int point_major_records = views_see_little(p, N, hits) ? 1 : 0;
    // Views in rounds of up to view_lanes: the per-pixel kernel takes the views of a round in one launch, each into its
    // lane's record array, and the per-point kernel behind it reads them all, again in one launch (the views add to
    // the same gradient rows).
    const int lanes = std::max(1, lay.view_lanes);
    const float4* packed = a->packed_descriptors ? reinterpret_cast<const float4*>(a->packed_descriptors)
                                                 : ws_ptr<float4>(ws, lay.packed_base);
    const int background_rows_count = (int)tile_grid(tiles) + (fuzzy_long ? kFuzzyFoldRows : 0);
    for (int first = 0; first < B; first += lanes)
    {
        const int last = std::min(B, first + lanes), count = last - first;
        float4* partial        = ws_ptr<float4>(ws, lay.partial_base);
        float* background_rows = ws_ptr<float>(ws, lay.background_partial_base);
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_BLEND);
            PerView<BackwardPass> views{};
            for (int b = first; b < last; ++b)
            {
                const size_t lane = (size_t)(b - first);
                BackwardPass& bp  = views.v[lane];
                bp.offsets          = ws_ptr<uint32_t>(ws, lay.offsets_base + lay.offsets_stride * b);
                bp.kept             = ws_ptr<uint32_t>(ws, lay.kept_base + lay.kept_stride * b);
                bp.projected        = lay.projected_stride ? ws_ptr<float2>(ws, lay.projected_base + lay.projected_stride * b) : nullptr;
                bp.fragments        = ws_ptr<uint64_t>(ws, lay.fragments_base + lay.fragments_stride * b);
                bp.transmittance    = ws_ptr<float>(ws, lay.transmittance_base + lay.transmittance_stride * b);
                bp.weight           = ws_ptr<float>(ws, lay.weight_base + lay.weight_stride * b);
                bp.index            = a->index;
                bp.packed           = packed;
                bp.background       = ws_ptr<const float>(ws, lay.flags_base) + kPreparedBackgroundOffset;
                bp.partial          = ws_ptr<float4>(ws, lay.partial_base + lay.lane_scratch_stride * lane);
                bp.point_major_records = point_major_records;
                bp.background_partial  = ws_ptr<float>(ws, lay.background_partial_base + lay.lane_scratch_stride * lane);
                bp.ly               = ly;
                bp.tiles            = tiles;
                bp.N                = N;
                bp.K                = p.debug_max_list_length;
                bp.use_environment_map              = p.use_environment_map;
                bp.need_point_gradient              = want_image_gradient ? 1 : 0;
                bp.quirk_background_confidence_leak = p.quirk_background_confidence_leak;
                bp.clear                            = b == 0 ? clear : ClearJob{};
                for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
                {
                    bp.grad_out[l] = nullptr;
                    bp.out[l]      = nullptr;
                    if (l >= L) continue;
                    const size_t plane = (size_t)ly.w[l] * ly.h[l];
                    bp.grad_out[l]     = g->grad_out[l] + (size_t)b * C * plane;
                    bp.out[l]          = a->out[l] + (size_t)b * C * plane;
                }
            }
            const BackwardPass& bp = views.v[0];
            const unsigned tiles_x = tile_grid(tiles);
            const dim3 grid(tiles_x), grid_views(tiles_x, (unsigned)count), blk(kBlock);
            const bool one = count == 1;
            if (p.render_mode == VETRAST_RENDER_FUZZY_BLEND)
            {
                // Lists of more than kFuzzyDense fragments exist only where the cut allows them; each is taken by a whole
                // wave, in a second kernel.
                const bool beyond_dense = bp.K <= 0 || bp.K > kFuzzyDense;
                // With longer lists about, the narrow dense kernel in front of that one is faster than the wide one (measured).
                const bool wide    = !beyond_dense && bp.K > kFuzzyNarrow;
                const float accept = p.depth_accept_blend;
                auto launch = [&](auto channels) {
                    constexpr int kC = decltype(channels)::value;
                    if (wide && one)
                        hipLaunchKernelGGL((blend_backward_fuzzy_kernel<kC, kFuzzyDense>), grid, blk, 0, stream, bp, accept);
                    else if (wide)
                        hipLaunchKernelGGL((blend_backward_fuzzy_views_kernel<kC, kFuzzyDense>), grid_views, blk, 0, stream, views, accept);
                    else if (one)
                        hipLaunchKernelGGL((blend_backward_fuzzy_kernel<kC, kFuzzyNarrow>), grid, blk, 0, stream, bp, accept);
                    else
                        hipLaunchKernelGGL((blend_backward_fuzzy_views_kernel<kC, kFuzzyNarrow>), grid_views, blk, 0, stream, views, accept);
                    if (beyond_dense)
                    {
                        const uint32_t dense_max = (uint32_t)(wide ? kFuzzyDense : kFuzzyNarrow);
                        // the rows of replicas 1 .. into kFuzzyFoldRows rows behind the per-workgroup ones
                        PerView<FoldArgs> folds{};
                        for (int k = 0; k < count; ++k)
                        {
                            folds.v[k].rows     = views.v[k].background_partial + ((size_t)kFuzzyFoldRows + tiles_x) * kBackgroundRow;
                            folds.v[k].num_rows = (int)((kFuzzyReplicas - 1) * tiles_x);
                            folds.v[k].folded   = views.v[k].background_partial + (size_t)tiles_x * kBackgroundRow;
                        }
                        if (one)
                        {
                            hipLaunchKernelGGL(blend_backward_fuzzy_long_kernel<kC>, dim3(tiles_x, kFuzzyReplicas), blk, 0, stream, bp,
                                               accept, dense_max);
                            hipLaunchKernelGGL(fold_background_rows_kernel, dim3(kFuzzyFoldRows), blk, 0, stream, folds.v[0].rows,
                                               folds.v[0].num_rows, folds.v[0].folded);
                        }
                        else
                        {
                            hipLaunchKernelGGL(blend_backward_fuzzy_long_views_kernel<kC>, dim3(tiles_x, kFuzzyReplicas, (unsigned)count),
                                               blk, 0, stream, views, accept, dense_max);
                            hipLaunchKernelGGL(fold_background_rows_views_kernel, dim3(kFuzzyFoldRows, (unsigned)count), blk, 0,
                                               stream, folds);
                        }
                    }
                };
                switch (C)
                {
                    case 1: launch(std::integral_constant<int, 1>{}); break;
                    case 2: launch(std::integral_constant<int, 2>{}); break;
                    case 3: launch(std::integral_constant<int, 3>{}); break;
                    default: launch(std::integral_constant<int, 4>{}); break;
                }
            }
            else
            {
                auto launch = [&](auto channels, auto bilinear) {
                    constexpr int kC         = decltype(channels)::value;
                    constexpr bool kBilinear = decltype(bilinear)::value;
                    if (one)
                        hipLaunchKernelGGL((blend_backward_kernel<kC, kBilinear>), grid, blk, 0, stream, bp);
                    else
                        hipLaunchKernelGGL((blend_backward_views_kernel<kC, kBilinear>), grid_views, blk, 0, stream, views);
                };
                auto with_channels = [&](auto bilinear) {
                    switch (C)
                    {
                        case 1: launch(std::integral_constant<int, 1>{}, bilinear); break;
                        case 2: launch(std::integral_constant<int, 2>{}, bilinear); break;
                        case 3: launch(std::integral_constant<int, 3>{}, bilinear); break;
                        default: launch(std::integral_constant<int, 4>{}, bilinear); break;
                    }
                };
                if (hits == 1)
                    with_channels(std::false_type{});
                else
                    with_channels(std::true_type{});
            }
        }
        if (N > 0)
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_GATHER);
            GatherPass gp;
            gp.vp                  = make_view_pass(a, lay, ly, first);
            gp.offsets             = ws_ptr<uint32_t>(ws, lay.offsets_base + lay.offsets_stride * first);
            gp.fragments           = ws_ptr<uint64_t>(ws, lay.fragments_base + lay.fragments_stride * first);
            gp.list_is_cut         = ws_ptr<uint8_t>(ws, lay.cut_flags_base + lay.cut_flags_stride * first);
            gp.last_key            = ws_ptr<uint64_t>(ws, lay.last_key_base + lay.last_key_stride * first);
            gp.kept                = ws_ptr<uint32_t>(ws, lay.kept_base + lay.kept_stride * first);
            gp.partial             = partial;
            gp.grad_texture        = g->grad_texture;
            gp.grad_confidence     = g->grad_confidence;
            gp.grad_points         = g->grad_points;
            gp.grad_point_count    = g->grad_point_count;
            gp.K                   = p.debug_max_list_length;
            gp.need_point_gradient = want_image_gradient ? 1 : 0;
            gp.camera_partial      = want_camera ? camera_rows : nullptr;
            gp.point_major_records = point_major_records;
            gp.view_count          = count;
            gp.dropout_stride      = (size_t)N;
            gp.flags_stride        = lay.cut_flags_stride;
            gp.last_key_stride     = lay.last_key_stride / sizeof(uint64_t);
            gp.kept_stride         = lay.kept_stride / sizeof(uint32_t);
            gp.partial_stride      = lay.lane_scratch_stride / sizeof(float4);
            gp.background_rows_stride = lay.lane_scratch_stride / sizeof(float);
            gp.camera_partial_stride  = camera_rows_bytes(N) / sizeof(double);
            gp.accumulate          = (add_to_rows || first > 0) ? 1 : 0;
            gp.background_rows       = background_rows;
            // (with the folded rows of the FUZZY_BLEND kernel that takes a wave per list, where it ran)
            gp.num_background_rows   = background_rows_count;
            gp.grad_background       = g->grad_background;
            gp.add_leak = (p.quirk_background_confidence_leak && !p.use_environment_map && hits == 1 &&
                           p.render_mode != VETRAST_RENDER_FUZZY_BLEND)
                              ? 1
                              : 0;
            gp.background_accumulate = first > 0 ? 1 : 0;
            gp.packed                = packed;
            gp.texture_raw           = a->texture;
            gp.background_raw        = a->background;
            gp.confidence_activation = p.confidence_activation;
            gp.confidence_scale      = p.confidence_scale;
            gp.texture_abs           = p.texture_abs;
            const dim3 grid(grid_for(N)), blk(kBlock);
            // cameras with distortion switched on take the variant that carries the distortion Jacobians
            auto launch = [&](auto c_tag, auto hits_tag) {
                constexpr int kC = decltype(c_tag)::value, kHits = decltype(hits_tag)::value;
                if (gp.view_count > 1)
                {
                    if (p.allow_distortion)
                        hipLaunchKernelGGL((gather_point_gradients_kernel<kC, kHits, true, true>), grid, blk, 0, stream, gp);
                    else
                        hipLaunchKernelGGL((gather_point_gradients_kernel<kC, kHits, false, true>), grid, blk, 0, stream, gp);
                }
                else if (p.allow_distortion)
                    hipLaunchKernelGGL((gather_point_gradients_kernel<kC, kHits, true>), grid, blk, 0, stream, gp);
                else
                    hipLaunchKernelGGL((gather_point_gradients_kernel<kC, kHits, false>), grid, blk, 0, stream, gp);
            };
            auto with_channels = [&](auto hits_tag) {
                switch (C)
                {
                    case 1: launch(std::integral_constant<int, 1>{}, hits_tag); break;
                    case 2: launch(std::integral_constant<int, 2>{}, hits_tag); break;
                    case 3: launch(std::integral_constant<int, 3>{}, hits_tag); break;
                    default: launch(std::integral_constant<int, 4>{}, hits_tag); break;
                }
            };
            if (hits == 1)
                with_channels(std::integral_constant<int, 1>{});
            else
                with_channels(std::integral_constant<int, 4>{});
        }
        for (int v = first; want_camera && v < last; ++v)
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_GATHER);
            hipLaunchKernelGGL(reduce_camera_kernel, dim3(1), dim3(kBlock), 0, stream,
                               camera_rows + (size_t)(v - first) * (camera_rows_bytes(N) / sizeof(double)), grid_for(N),
                               a->views[v].image_index, a->views[v].camera_index, p.K_gradient_factor, g->grad_pose,
                               g->grad_pose_count, g->grad_intrinsics, g->grad_intrinsics_count,
                               hits == 1 ? 1.f / 1024.f : 1.f, p.allow_distortion, p.distortion_gradient_factor);
        }
        for (int v = first; N == 0 && v < last; ++v)
        {
            ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_GATHER);
            hipLaunchKernelGGL(reduce_background_kernel, dim3(1), dim3(kReduceBlock), 0, stream,
                               background_rows + (size_t)(v - first) * (lay.lane_scratch_stride / sizeof(float)),
                               background_rows_count, C, g->grad_background, g->grad_confidence, 0, v > 0 ? 1 : 0,
                               p.texture_abs ? a->background : nullptr);
        }
    }
    if (g->grad_points && p.point_gradient_normalization != 0 && N > 0)
    {
        ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_POST);
        hipLaunchKernelGGL(normalize_point_gradient_kernel, dim3(grid_for(N)), dim3(kBlock), 0, stream,
                           g->grad_points, g->grad_point_count, N, p.point_gradient_normalization);
    }
    if (want_camera && p.camera_gradient_normalization)
    {
        ScopeTimer tm(ctx, stream, VETRAST_SCOPE_BACKWARD_POST);
        const int n = std::max(a->num_poses, a->num_cameras);
        hipLaunchKernelGGL(normalize_camera_gradients_kernel, dim3(grid_for(n)), dim3(kBlock), 0, stream, g->grad_pose,
                           g->grad_pose_count, a->num_poses, g->grad_intrinsics, g->grad_intrinsics_count,
                           a->num_cameras);
    }
    VET_HIP(ctx, hipGetLastError());
    return VETRAST_OK;
}

size_t vetrast_packed_descriptor_bytes(int32_t num_points)
{
    return num_points > 0 ? (size_t)num_points * 2 * sizeof(float4) : 0;
}

int vetrast_pack_descriptors(vetrast_ctx* ctx, const vetrast_pack_args* a, void* stream_)
{
    if (!ctx || !a || a->num_points < 0) return VETRAST_ERR_INVALID_ARG;
    const int C = a->params.num_texture_channels;
    if (C < 1 || C > VETRAST_MAX_CHANNELS) return VETRAST_ERR_INVALID_ARG;
    if (a->num_points == 0) return VETRAST_OK;
    if (!a->texture || !a->confidence || !a->packed) return VETRAST_ERR_INVALID_ARG;
    if (reinterpret_cast<uintptr_t>(a->packed) % (2 * sizeof(float4)) != 0) return VETRAST_ERR_INVALID_ARG;
    PackJob pack;
    pack.texture               = a->texture;
    pack.confidence            = a->confidence;
    pack.packed                = reinterpret_cast<float4*>(a->packed);
    pack.N                     = a->num_points;
    pack.C                     = C;
    pack.confidence_activation = a->params.confidence_activation;
    pack.confidence_scale      = a->params.confidence_scale;
    pack.texture_abs           = a->params.texture_abs;
    pack.visible_only          = 0;
    hipStream_t stream         = (hipStream_t)stream_;
    ScopeTimer tm(ctx, stream, VETRAST_SCOPE_PACK);
    hipLaunchKernelGGL(pack_descriptors_kernel, dim3(grid_for(a->num_points)), dim3(kBlock), 0, stream, pack);
    VET_HIP(ctx, hipGetLastError());
    return VETRAST_OK;
}

int vetrast_adam_step(vetrast_ctx* ctx, const vetrast_adam_args* a, void* stream_)
{
    if (!ctx || !a) return VETRAST_ERR_INVALID_ARG;
    if (a->n < 0 || a->step < 1) return VETRAST_ERR_INVALID_ARG;
    if (a->n == 0) return VETRAST_OK;
    if (!a->param || !a->grad || !a->exp_avg || !a->exp_avg_sq) return VETRAST_ERR_INVALID_ARG;
    // bias corrections in double as in src/lib/models/my_adam.cpp:72-73,97-100, handed to the kernel rounded once
    const double bc1 = 1.0 - std::pow(a->beta1, (double)a->step);
    const double bc2 = 1.0 - std::pow(a->beta2, (double)a->step);
    if (!(bc1 > 0.0) || !(bc2 > 0.0)) return VETRAST_ERR_INVALID_ARG;
    const float sqrt_bc2  = (float)std::sqrt(bc2);
    const float step_size = (float)(a->lr / bc1);
    hipStream_t stream    = (hipStream_t)stream_;
    const int blocks      = (int)std::min<int64_t>((a->n + kBlock - 1) / kBlock, 16384);
    hipLaunchKernelGGL(adam_step_kernel, dim3(blocks), dim3(kBlock), 0, stream, a->param, a->grad, a->exp_avg,
                       a->exp_avg_sq, (size_t)a->n, (float)a->beta1, (float)a->beta2, (float)(1.0 - a->beta1),
                       (float)(1.0 - a->beta2), sqrt_bc2, step_size, (float)a->eps, (float)a->weight_decay,
                       a->zero_grad);
    VET_HIP(ctx, hipGetLastError());
    return VETRAST_OK;
}

size_t vetrast_lift_workspace_bytes(int64_t num_cells)
{
    if (num_cells < 0) return 0;
    return lift_workspace_bytes_for((size_t)num_cells);
}

int vetrast_lift_error(vetrast_ctx* ctx, const vetrast_lift_args* a, void* stream_)
{
    if (!ctx || !a) return VETRAST_ERR_INVALID_ARG;
    bool nothing_to_do = false;
    const int st       = validate_lift(a, &nothing_to_do);
    if (st != VETRAST_OK || nothing_to_do) return st;
    if (!a->workspace || reinterpret_cast<uintptr_t>(a->workspace) % kAlign) return VETRAST_ERR_INVALID_ARG;
    if (a->workspace_bytes < vetrast_lift_workspace_bytes(a->num_cells)) return VETRAST_ERR_WORKSPACE_SMALL;
    hipStream_t stream = (hipStream_t)stream_;
    ScopeTimer tm(ctx, stream, VETRAST_SCOPE_LIFT_ERROR);
    launch_lift(a, static_cast<char*>(a->workspace), stream);
    VET_HIP(ctx, hipGetLastError());
    return VETRAST_OK;
}

int vetrast_lift_error_static(vetrast_ctx* ctx, const vetrast_lift_args* a, void* stream_)
{
    if (!ctx || !a) return VETRAST_ERR_INVALID_ARG;
    bool nothing_to_do = false;
    const int st       = validate_lift(a, &nothing_to_do);
    if (st != VETRAST_OK || nothing_to_do) return st;
    if (a->num_cells > (int64_t)VETRAST_LIFT_STATIC_MAX_CELLS) return VETRAST_ERR_TOO_LARGE;
    // the scratch pointer belongs to the context's device; kernels launched on another device's stream must not get it
    int current = -1;
    VET_HIP(ctx, hipGetDevice(&current));
    if (current != ctx->device || !ctx->lift_scratch) return VETRAST_ERR_INVALID_ARG;
    // No timing scope here: a scope takes HIP events and grows a host vector, and this entry point allocates nothing.
    launch_lift(a, ctx->lift_scratch, (hipStream_t)stream_);
    VET_HIP(ctx, hipGetLastError());
    return VETRAST_OK;
}

int vetrast_query_device_flags(vetrast_ctx* ctx, const void* workspace, const vetrast_workspace_layout* layout,
                               void* stream)
{
    if (!ctx || !workspace || !layout) return VETRAST_ERR_INVALID_ARG;
    uint32_t flags[4] = {0, 0, 0, 0};
    VET_HIP(ctx, hipStreamSynchronize((hipStream_t)stream));
    VET_HIP(ctx, hipMemcpy(flags, static_cast<const char*>(workspace) + layout->flags_base, sizeof(flags),
                           hipMemcpyDeviceToHost));
    return (flags[0] & 1u) ? VETRAST_ERR_BAD_INPUT_DATA : VETRAST_OK;
}

int vetrast_set_profiling(vetrast_ctx* ctx, int32_t enabled)
{
    if (!ctx) return VETRAST_ERR_INVALID_ARG;
    ctx->profiling = enabled ? 1 : 0;
    return VETRAST_OK;
}

static int collect_spans(vetrast_ctx* ctx)
{
    for (auto& s : ctx->spans)
    {
        VET_HIP(ctx, hipEventSynchronize(s.stop));
        float ms = 0.f;
        VET_HIP(ctx, hipEventElapsedTime(&ms, s.start, s.stop));
        ctx->acc_ms[s.scope] += ms;
        ctx->acc_launches[s.scope] += 1;
        ctx->free_events.push_back(s.start);
        ctx->free_events.push_back(s.stop);
    }
    ctx->spans.clear();
    return VETRAST_OK;
}

int vetrast_reset_scope_times(vetrast_ctx* ctx)
{
    if (!ctx) return VETRAST_ERR_INVALID_ARG;
    int st = collect_spans(ctx);
    for (int i = 0; i < VETRAST_SCOPE_COUNT_; ++i)
    {
        ctx->acc_ms[i]       = 0.f;
        ctx->acc_launches[i] = 0;
    }
    return st;
}

int vetrast_scope_times(vetrast_ctx* ctx, float* ms, int32_t* launches)
{
    if (!ctx || !ms || !launches) return VETRAST_ERR_INVALID_ARG;
    int st = collect_spans(ctx);
    for (int i = 0; i < VETRAST_SCOPE_COUNT_; ++i)
    {
        ms[i]       = ctx->acc_ms[i];
        launches[i] = ctx->acc_launches[i];
    }
    return st;
}

const char* vetrast_scope_name(int32_t scope)
{
    switch (scope)
    {
        case VETRAST_SCOPE_PREPARE: return "Build Cache";
        case VETRAST_SCOPE_PACK: return "Build Cache (descriptor interleave; part of the counting pass, no launch of its own)";
        case VETRAST_SCOPE_COUNT: return "CountingPass";
        case VETRAST_SCOPE_SCAN: return "CreateAndAllocateBuffers";
        case VETRAST_SCOPE_FILL: return "CollectionPass";
        case VETRAST_SCOPE_BUILD: return "CollectionPass (per-pixel lists) + SortingPass + BlendingPass";
        case VETRAST_SCOPE_BACKWARD_PREPARE: return "Prepare Backward";
        case VETRAST_SCOPE_BACKWARD_BLEND: return "BlendBackwards";
        case VETRAST_SCOPE_BACKWARD_GATHER: return "BlendBackwards (per-point sum)";
        case VETRAST_SCOPE_BACKWARD_POST: return "Post Process Gradient";
        case VETRAST_SCOPE_LIFT_ERROR: return "FillSceneGridWithLoss";
        default: return "?";
    }
}

const char* vetrast_status_string(int status)
{
    switch (status)
    {
        case VETRAST_OK: return "ok";
        case VETRAST_ERR_INVALID_ARG: return "invalid argument";
        case VETRAST_ERR_WORKSPACE_SMALL: return "workspace too small";
        case VETRAST_ERR_HIP: return "HIP runtime error";
        case VETRAST_ERR_UNSUPPORTED: return "feature outside the implemented blending path";
        case VETRAST_ERR_BAD_INPUT_DATA: return "device-side input check failed (non-zero distortion)";
        case VETRAST_ERR_TOO_LARGE: return "size beyond the fixed maximum of an allocation-free entry point";
        default: return "unknown status";
    }
}

int vetrast_last_hip_error(const vetrast_ctx* ctx)
{
    return ctx ? ctx->last_hip_error : 0;
}

}  // extern "C"
