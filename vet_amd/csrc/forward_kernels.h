// Forward kernels: zero fill, view preparation, descriptor interleave (+ fused preparation steps), Adam step, per-bin
// count, scan, fill. The per-bin build / sort / blend pass is in build_kernels.h.
#pragma once
#include "common.h"

namespace vetrast
{
// Plain fill kernel (used instead of hipMemsetAsync so that callers may capture the launches in a HIP graph).
__global__ void __launch_bounds__(kBlock) fill_u32_kernel(uint32_t* __restrict__ dst, size_t n, uint32_t value)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = value;
}

// One Adam step on n floats (MyAdam::step, src/lib/models/my_adam.cpp:66-101, i.e. torch's Adam without amsgrad), every
// operation rounded on its own in the order of the tensor ops there. inv_sqrt_bc2 = 1 / sqrt(1 - beta2^step) and
// step_size = lr / (1 - beta1^step) come from the host in double, rounded once.
__global__ void __launch_bounds__(kBlock) adam_step_kernel(float* __restrict__ param, float* __restrict__ grad,
                                                            float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
                                                            size_t n, float beta1, float beta2, float one_minus_beta1,
                                                            float one_minus_beta2, float sqrt_bc2, float step_size,
                                                            float eps, float weight_decay, int zero_grad)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    {
        const float p = param[i];
        float g       = grad[i];
        if (weight_decay != 0.f) g = g + weight_decay * p;            // grad.add(p, weight_decay)
        const float m = exp_avg[i] * beta1 + one_minus_beta1 * g;      // mul_(beta1).add_(grad, 1 - beta1)
        const float v = exp_avg_sq[i] * beta2 + (one_minus_beta2 * g) * g;  // mul_(beta2).addcmul_(grad, grad, 1 - beta2)
        const float denom = sqrtf(v) / sqrt_bc2 + eps;                 // (sqrt() / sqrt(bias_correction2)).add_(eps)
        exp_avg[i]    = m;
        exp_avg_sq[i] = v;
        param[i]      = p + (-step_size) * (m / denom);                // addcdiv_(exp_avg, denom, -step_size)
        if (zero_grad) grad[i] = 0.f;
    }
}

struct ViewSource
{
    int image_index, camera_index, w, h;
    float crop[5];
    float rot[4];
};

struct PrepareViewsArgs
{
    ViewSource src[16];
};

// Camera constants of one view: pose (unit quaternion + translation, double) -> 3x4 float matrix, intrinsics row -> K.
// The reference casts the SE3d to float in every thread (src/lib/rendering/RenderConstants.h:78); here the rotation
// matrix is formed once, in double, and rounded once. `distorted` reports non-zero distortion coefficients.
__device__ __forceinline__ DeviceView make_device_view(const ViewSource& s, const double* __restrict__ poses_se3,
                                                       const float* __restrict__ intrinsics, bool& distorted)
{
    const double* q = poses_se3 + 8 * (size_t)s.image_index;
    const float* in = intrinsics + 13 * (size_t)s.camera_index;
    DeviceView v;
    const double x = q[0], y = q[1], z = q[2], w = q[3];
    const double tx = 2.0 * x, ty = 2.0 * y, tz = 2.0 * z;
    const double twx = tx * w, twy = ty * w, twz = tz * w;
    const double txx = tx * x, txy = ty * x, txz = tz * x;
    const double tyy = ty * y, tyz = tz * y, tzz = tz * z;
    v.r[0] = (float)(1.0 - (tyy + tzz));
    v.r[1] = (float)(txy - twz);
    v.r[2] = (float)(txz + twy);
    v.r[3] = (float)(txy + twz);
    v.r[4] = (float)(1.0 - (txx + tzz));
    v.r[5] = (float)(tyz - twx);
    v.r[6] = (float)(txz - twy);
    v.r[7] = (float)(tyz + twx);
    v.r[8] = (float)(1.0 - (txx + tyy));
    v.t[0] = (float)q[4];
    v.t[1] = (float)q[5];
    v.t[2] = (float)q[6];
    v.fx   = in[0];
    v.fy   = in[1];
    v.cx   = in[2];
    v.cy   = in[3];
    v.s    = in[4];
    distorted = false;
    for (int j = 5; j < 13; ++j)
    {
        distorted |= (in[j] != 0.f);
        v.dist[j - 5] = in[j];
    }
    v.has_dist = distorted ? 1u : 0u;
    for (int j = 0; j < 5; ++j) v.crop[j] = s.crop[j];
    for (int j = 0; j < 4; ++j) v.rot[j] = s.rot[j];
    v.ccx = (float)(s.w / 2);
    v.ccy = (float)(s.h / 2);
    for (int j = 0; j < 3; ++j) v.pad[j] = 0.f;
    return v;
}

// One thread per view fills its camera constants; non-zero distortion coefficients raise flag bit 0 unless the caller
// has switched distortion on.
// Workgroups beyond the first zero the per-bin counters of all views (n4 uint4 elements).
__global__ void __launch_bounds__(kBlock) prepare_views_kernel(PrepareViewsArgs args, int first_view, int num_views,
                                                                const double* __restrict__ poses_se3,
                                                                const float* __restrict__ intrinsics,
                                                                DeviceView* __restrict__ views,
                                                                uint32_t* __restrict__ flags,
                                                                uint4* __restrict__ counters4, size_t n4,
                                                                const float* __restrict__ background, int channels,
                                                                int texture_abs, int allow_distortion)
{
    if (blockIdx.x > 0)
    {
        const size_t stride = (size_t)(gridDim.x - 1) * blockDim.x;
        for (size_t i = (size_t)(blockIdx.x - 1) * blockDim.x + threadIdx.x; i < n4; i += stride)
            counters4[i] = make_uint4(0u, 0u, 0u, 0u);
        return;
    }
    const int k = threadIdx.x;
    if (first_view == 0)
    {
        // the device flag word starts every call at zero
        if (k < 4) flags[k] = 0u;
        // the background as it is blended: PrepareTexture, src/lib/models/NeuralTexture.h:43-55
        if (k < VETRAST_MAX_CHANNELS)
        {
            const float bg = k < channels ? background[k] : 0.f;
            reinterpret_cast<float*>(flags)[kPreparedBackgroundOffset + k] = texture_abs ? fabsf(bg) : bg;
        }
        __syncthreads();
    }
    if (k >= num_views) return;
    bool distorted = false;
    DeviceView v = make_device_view(args.src[k], poses_se3, intrinsics, distorted);
    if (distorted && !allow_distortion)
    {
        atomicOr(flags, 1u);  // refused: the call renders the camera without distortion and says so
        v.has_dist = 0u;
    }
    views[first_view + k] = v;
}

// The viewer's confidence cut-off: the same verdict in every view of a call.
__device__ __forceinline__ bool point_is_skipped_in_all_views(const ViewPass& a, int i)
{
    if (a.viewer_only)
    {
        const int ti = a.index ? a.index[i] : i;
        float c      = a.confidence[ti];
        if (a.confidence_activation) c = sigmoid_canon(a.confidence_scale * c);
        if (c < a.stability_cutoff) return true;
    }
    return false;
}

__device__ __forceinline__ bool point_is_skipped(const ViewPass& a, int i)
{
    if (a.dropout && a.dropout[i] == 1.f) return true;  // this view's drop-out mask
    return point_is_skipped_in_all_views(a, i);
}

// ---- binning ---------------------------------------------------------------------------------------------------------
// The reference counts every (point, layer) hit with one global atomic on its pixel, fills the lists with a second one
// (CountingPrepassMulti / CollectMulti, src/lib/rendering/RenderForward.cu:806-905,1011-1096) and then sorts every
// list. MI355X retires about 26 G global atomics per second whatever their scope, return mode or address spread, and at
// the fine layers nearly every fragment has a pixel of its own, so per-pixel atomics alone would cost more than the
// rest of the forward pass. The lists are therefore built in two levels:
//   1. bin_scatter_kernel: one pass over the points. A BIN is a run of 256 / 64 / 16 / 4 consecutive pixel numbers (a
//      16x16 tile or a piece of one; the denser the layer, the smaller its bins). VET hands over clouds in Morton order
//      with 256-point blocks (src/lib/data/SceneData.cpp:105-106), so the 64 points of a wave fall into a handful of
//      bins per layer: the wave groups its hits by bin with ballots and issues one returning atomic per distinct bin,
//      which counts the bin and gives every hit its arrival rank inside it; the fragment record goes straight to
//      place `rank` of the room the bin owns (no second projection pass).
//   2. exclusive scan over the bin counts; the few records that did not fit a bin's room are filed behind it (the same
//      launch, scan_move_kernel, where a view has at most kScanMoveMax bins; overflow_move_kernel otherwise).
//   3. bin_build_kernel: one workgroup per bin counts the pixels, scans them, scatters the keys and sorts the lists, all
//      in LDS. Pixels are numbered tile by tile, so the scan of the bin counts IS the start of every bin's lists and no
//      scan over the pixels is needed.

// Per-lane grouping of equal bin numbers inside a wave: leader = lowest lane with the same bin, rank = number of
// lower lanes with the same bin, count = size of the group. Pure ballots, no memory traffic.
struct WaveGroup
{
    int leader;
    uint32_t rank, count;
};

__device__ __forceinline__ WaveGroup group_by_bin(bool has, uint32_t bin, int lane)
{
    WaveGroup g;
    g.leader = lane;
    g.rank = g.count = 0;
    uint64_t todo = __ballot(has);
    while (todo != 0ull)  // one turn per distinct bin; everything but the compare and the selects is scalar
    {
        const int first        = __ffsll((unsigned long long)todo) - 1;
        const uint32_t b_first = (uint32_t)__builtin_amdgcn_readlane((int)bin, first);
        const bool mine        = has && bin == b_first;
        const uint64_t same    = __ballot(mine);
        // number of set bits of `same` below this lane
        const uint32_t below = __builtin_amdgcn_mbcnt_hi((uint32_t)(same >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)same, 0u));
        if (mine)
        {
            g.leader = first;
            g.rank   = below;
            g.count  = (uint32_t)__popcll(same);
        }
        todo &= ~same;
    }
    return g;
}

// The same with 1..4 hits per lane for the bin. The group's slots are laid out place by place: first the first hit of
// every lane of the group in lane order, then the second hits, and so on, so that the record stores, one hit per
// lane and instruction, write runs of consecutive records. ranks holds the slot (inside the group) of the lane's
// hit at place o in bits 8 o .. 8 o + 7 (a group has at most 256 hits), total the size of the group.
struct WeightedGroup
{
    int leader;
    uint32_t ranks, total;
};

__device__ __forceinline__ WeightedGroup group_by_bin_weighted(bool has, uint32_t bin, uint32_t weight, int lane)
{
    WeightedGroup g;
    g.leader = lane;
    g.ranks = g.total = 0;
    uint64_t todo     = __ballot(has);
    while (todo != 0ull)
    {
        const int first        = __ffsll((unsigned long long)todo) - 1;
        const uint32_t b_first = (uint32_t)__builtin_amdgcn_readlane((int)bin, first);
        const bool mine        = has && bin == b_first;
        const uint64_t m0 = __ballot(mine), m1 = __ballot(mine && weight > 1u), m2 = __ballot(mine && weight > 2u),
                       m3 = __ballot(mine && weight > 3u);
        const uint32_t c0 = (uint32_t)__popcll(m0), c1 = (uint32_t)__popcll(m1), c2 = (uint32_t)__popcll(m2),
                       c3 = (uint32_t)__popcll(m3);
        auto below = [](uint64_t m) {
            return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        };
        if (mine)
        {
            g.leader = first;
            g.ranks  = below(m0) | ((c0 + below(m1)) << 8) | ((c0 + c1 + below(m2)) << 16) | ((c0 + c1 + c2 + below(m3)) << 24);
            g.total  = c0 + c1 + c2 + c3;
        }
        todo &= ~m0;
    }
    return g;
}

// Planar descriptors [C,N] + confidence [N] -> one 32-byte record per texture index, so that a fragment costs a single
// aligned gather instead of C+1 gathers from planes megabytes apart (the reference's BlendMulti reads
// d_texture.in_texture(ci, idx) per channel, src/lib/rendering/RenderForward.cu:1338-1342).
// The interleave also applies the steps VET runs on the raw tensors right before rendering, when they are switched on:
// confidence = sigmoid(scale * raw) and texture = |raw| (NeuralPointTextureImpl::PrepareConfidence / PrepareTexture,
// src/lib/models/NeuralTexture.h:38-55).
// It is a side job of the scatter pass of a call's first view (thread i also packs texture row i):
// the scatter waves spend most of their life waiting for their atomics, so the extra loads and stores ride along
// (a launch of its own on a second stream took 21 us alone and slowed the scatter pass down by 12 us beside it).
struct PackJob
{
    const float* texture;     // [C,N]
    const float* confidence;  // [N]
    float4* packed;           // [N][2], or null: nothing to pack in this launch
    int N, C;
    int confidence_activation;
    float confidence_scale;
    int texture_abs;
    int visible_only;  // pack the rows of the points that can leave a fragment in this view only (see bin_scatter_kernel)
};

// The record of texture row `slot` from its raw values.
__device__ __forceinline__ void store_packed_row(const PackJob& pack, int slot, float (&row)[4], float row_confidence)
{
    if (pack.texture_abs)
    {
#pragma unroll
        for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci) row[ci] = fabsf(row[ci]);
    }
    if (pack.confidence_activation) row_confidence = sigmoid_canon(pack.confidence_scale * row_confidence);
    pack.packed[2 * (size_t)slot]     = make_float4(row[0], row[1], row[2], row[3]);
    pack.packed[2 * (size_t)slot + 1] = make_float4(row_confidence, 0.f, 0.f, 0.f);
}

// Where the scatter pass puts a fragment record (64-bit key = depth bits << 32 | point id, pixel inside the bin).
// Every bin owns room for room_cap[layer] records; a record whose rank inside its bin is beyond that is appended to a log
// (with its bin and rank), from where overflow_move_kernel brings it to the bin's place in the compact array once the
// scan of the bin counts is known. The log is cut into segments, one per residue of the workgroup number, each with a
// cursor in a cache line of its own: appends to one cursor would queue up behind each other where many bins overflow
// (a workgroup's segment has room for every hit the workgroups of that residue can produce). Bins are sized for an expected 1024 records at most, so the log stays empty or
// short unless the cloud is far denser somewhere than on average.
// A record is 16 bytes (key low, key high, pixel in bin, 0), or, where the low key word (point id; point id << 2 |
// corner for the 2x2 splat) fits 24 bits (`compact`), 8 bytes: (key high = depth bits, key low << 8 | pixel in bin).
// Half the bytes written here and read again by the build pass.
struct ScatterTargets
{
    uint4* primary;        // the bins' rooms, LayerTable::room_base (uint2 records when compact)
    int compact;
    uint4* log;            // [kLogSegments][segment_capacity]: key low, key high, pixel in bin, bin
    uint32_t* log_rank;    // the same shape: rank of the logged record inside its bin
    uint32_t* log_cursor;  // [kLogSegments], kLogCursorStride apart: entries in every segment (this view)
    uint32_t segment_capacity;
};

// One record to its bin; `valid` lanes carry one. Called by the whole wave (uniform control flow).
__device__ __forceinline__ void store_record(const ScatterTargets& t, const LayerTable& ly, int l, bool valid, uint32_t bin,
                                             uint32_t rank, uint32_t low, uint32_t depth_bits, uint32_t in_bin, int lane)
{
    const bool over = valid && rank >= ly.room_cap[l];
    if (valid && !over)
    {
        const size_t at = room_of_bin(ly, l, bin) + rank;
        if (t.compact)
            reinterpret_cast<uint2*>(t.primary)[at] = make_uint2(depth_bits, (low << 8) | in_bin);
        else
            t.primary[at] = make_uint4(low, depth_bits, in_bin, 0u);
    }
    const uint64_t m = __ballot(over);
    if (m != 0ull)  // rare
    {
        const uint32_t segment = blockIdx.x % (uint32_t)kLogSegments;
        const int leader       = __ffsll((unsigned long long)m) - 1;
        uint32_t first         = 0;
        if (lane == leader) first = atomicAdd(t.log_cursor + segment * kLogCursorStride, (uint32_t)__popcll(m));
        first = (uint32_t)__shfl((int)first, leader, kWave);
        const uint32_t at =
            first + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
        if (over && at < t.segment_capacity)  // guard: a segment has room for every hit of its workgroups
        {
            const size_t pos = (size_t)segment * t.segment_capacity + at;
            t.log[pos]       = make_uint4(low, depth_bits, in_bin, bin);
            t.log_rank[pos]  = rank;
        }
    }
}

// The one pass over the points: projection, the bin of every hit, the hit's rank inside its bin (which also counts
// the bin) and the fragment record written to the bin's room. Counterpart of CountingPrepassMulti and CollectMulti
// (src/lib/rendering/RenderForward.cu:806-905,1011-1096), which project every point twice and draw count and rank
// from two atomic counter images.
// HITS = 1: a point lands in the pixel it rounds to (FULL_BLEND); HITS = 4: in the 2x2 pixels around it
// (BILINEAR_BLEND), each of which is a fragment of its own with its own bin; the low key word is then
// point id << 2 | corner.
// This is the part of the pass behind the projection: thread `slot` has point i, which is `visible` at p in this view.
template <int HITS>
__device__ __forceinline__ void scatter_projected(const ViewPass& a, uint32_t* __restrict__ bin_counts,
                                                  const ScatterTargets& out, const PackJob& pack, int slot, int i, bool visible,
                                                  const Projected& p)
{
    const int lane = threadIdx.x & (kWave - 1);
    float ipx = visible ? p.ipx : 0.f, ipy = visible ? p.ipy : 0.f, radius = visible ? p.radius : 0.f;
    const uint32_t depth_bits = __float_as_uint(p.z);
    // A position further outside the image than the reach of the coarsest layer's border pixels hits no pixel of any
    // layer (layer l halves the coordinates l times, exactly; its pixel 0 reaches down to -2^l in layer-0 units with the
    // 2x2 splat, its last pixel not beyond the image size plus 2^l). A crop leaves most of the cloud out there: where
    // that is so for a whole wave, the wave skips the layers altogether.
    const float reach = (float)(1 << (a.ly.L - 1)) + 1.f;
    const bool inside = visible && ipx >= -reach && ipx <= (float)a.ly.w[0] + reach && ipy >= -reach &&
                        ipy <= (float)a.ly.h[0] + reach;
    const bool any_inside = __ballot(inside) != 0ull;
    // side job: texture row `slot`, asked for here and stored last. Only fragments ever read a row, so a call with one
    // view, no texture index and no processing order (row, point and thread then are the same number) leaves out the
    // rows of the points outside the view: half of the cloud for a full frame, most of it for a crop.
    const bool packs = pack.packed != nullptr && slot < pack.N && (!pack.visible_only || inside);
    float row[4] = {0.f, 0.f, 0.f, 0.f}, row_confidence = 0.f;
    if (packs)
    {
#pragma unroll
        for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci)
            if (ci < pack.C) row[ci] = pack.texture[(size_t)ci * pack.N + slot];
        row_confidence = pack.confidence[slot];
    }
    bool dropped = !inside;  // also from the layer on at which the splat radius falls under the threshold
    if constexpr (HITS == 1)
    {
        // Layer by layer: group the wave's hits by bin and issue the group's atomic right away. The atomics of a wave
        // are independent and their results are only looked at after the last one has been issued, so the wave waits
        // once. Kept per layer: the atomic's result, the bin, and
        // who = leader lane | rank << 8 | pixel in bin << 16 | has << 31.
        uint32_t base[VETRAST_MAX_LAYERS], who[VETRAST_MAX_LAYERS], bins[VETRAST_MAX_LAYERS];
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
        {
            base[l] = 0, who[l] = 0, bins[l] = 0;
            if (l >= a.ly.L || !any_inside) continue;
            if (a.drop_by_radius && radius < a.radius_threshold) dropped = true;
            uint32_t tile = 0, in_tile = 0, bin = 0, in_bin = 0;
            const bool has = !dropped && layer_hit<HITS>(a.ly, l, ipx, ipy, 0, tile, in_tile);
            if (has) bin_of_pixel(a.ly, l, tile, in_tile, bin, in_bin);
            const WaveGroup g = group_by_bin(has, bin, lane);
            who[l]            = (uint32_t)g.leader | (g.rank << 8) | (in_bin << 16) | (has ? 0x80000000u : 0u);
            bins[l]           = bin;
            if (has && g.leader == lane) base[l] = atomicAdd(&bin_counts[bin], g.count);
        }
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
        {
            if (l >= a.ly.L || !any_inside) continue;
            const uint32_t group_base = (uint32_t)__shfl((int)base[l], (int)(who[l] & 0xFF), kWave);
            store_record(out, a.ly, l, (who[l] & 0x80000000u) != 0u, bins[l], group_base + ((who[l] >> 8) & 0xFFu), (uint32_t)i,
                         depth_bits, (who[l] >> 16) & 0xFFu, lane);
        }
    }
    else
    {
        // The blend and its backward pass form a fragment's bilinear weight from the point's image position; they
        // read it from here (8 bytes) instead of projecting the point again for every one of its fragments.
        if (inside) a.projected[i] = make_float2(p.ipx, p.ipy);
        // The four pixels of a point mostly lie in one bin or two. Per layer the hits of a lane are therefore taken
        // bin by bin: in every turn a lane brings all its remaining hits that share the bin of its first remaining
        // hit, as one entry of that weight, so a layer takes as many grouping turns as the lane with the most
        // distinct bins has (1 or 2 as a rule, never more than 4) instead of 4, and one atomic per bin and turn.
        // The results of a layer's atomics are looked at after those of the next layer have been issued.
        // Kept per layer and turn: the atomic's result, the leader lane, the packed ranks and the bin; per layer,
        // 5 bits per hit: valid | turn << 1 | place among the lane's hits of that turn << 3, and the four pixels in bin.
        constexpr int kTurns = HITS;
        uint32_t base[VETRAST_MAX_LAYERS][kTurns], leader[VETRAST_MAX_LAYERS][kTurns], ranks[VETRAST_MAX_LAYERS][kTurns],
            bins[VETRAST_MAX_LAYERS][kTurns], code[VETRAST_MAX_LAYERS], in_bins[VETRAST_MAX_LAYERS];
        auto store_layer = [&](int l) {
            uint32_t start[kTurns];  // first slot of the group this lane's hits of every turn belong to
#pragma unroll
            for (int t = 0; t < kTurns; ++t) start[t] = (uint32_t)__shfl((int)base[l][t], (int)leader[l][t], kWave);
#pragma unroll
            for (int h = 0; h < HITS; ++h)
            {
                const uint32_t c = code[l] >> (5 * h);
                const uint32_t t = (c >> 1) & 3u, place = (c >> 3) & 3u;
                const uint32_t s = t == 0 ? start[0] : t == 1 ? start[1] : t == 2 ? start[2] : start[3];
                const uint32_t r = t == 0 ? ranks[l][0] : t == 1 ? ranks[l][1] : t == 2 ? ranks[l][2] : ranks[l][3];
                const uint32_t b = t == 0 ? bins[l][0] : t == 1 ? bins[l][1] : t == 2 ? bins[l][2] : bins[l][3];
                store_record(out, a.ly, l, (c & 1u) != 0u, b, s + ((r >> (8u * place)) & 0xFFu), ((uint32_t)i << 2) | (uint32_t)h,
                             depth_bits, (in_bins[l] >> (8 * h)) & 0xFFu, lane);
            }
        };
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
        {
            code[l] = 0, in_bins[l] = 0;
#pragma unroll
            for (int t = 0; t < kTurns; ++t) base[l][t] = 0, leader[l][t] = 0, ranks[l][t] = 0, bins[l][t] = 0;
            if (l < a.ly.L && any_inside)
            {
                if (a.drop_by_radius && radius < a.radius_threshold) dropped = true;
                uint32_t bin[HITS];
                uint32_t left = 0;  // hits not yet counted, one bit each
#pragma unroll
                for (int h = 0; h < HITS; ++h)
                {
                    uint32_t tile = 0, in_tile = 0, in_bin = 0;
                    bin[h]         = 0;
                    const bool has = !dropped && layer_hit<HITS>(a.ly, l, ipx, ipy, h, tile, in_tile);
                    if (has)
                    {
                        bin_of_pixel(a.ly, l, tile, in_tile, bin[h], in_bin);
                        left |= 1u << h;
                        in_bins[l] |= in_bin << (8 * h);
                    }
                }
#pragma unroll
                for (int t = 0; t < kTurns; ++t)
                {
                    if (__ballot(left != 0u) == 0ull) break;  // the same for the whole wave
                    uint32_t key = 0;
#pragma unroll
                    for (int h = HITS - 1; h >= 0; --h)
                        if (left & (1u << h)) key = bin[h];  // bin of the first remaining hit
                    uint32_t weight = 0;
#pragma unroll
                    for (int h = 0; h < HITS; ++h)
                        if ((left & (1u << h)) && bin[h] == key)
                        {
                            code[l] |= (1u | ((uint32_t)t << 1) | (weight << 3)) << (5 * h);
                            ++weight;
                            left &= ~(1u << h);
                        }
                    const bool has        = weight != 0u;
                    const WeightedGroup g = group_by_bin_weighted(has, key, weight, lane);
                    leader[l][t]          = (uint32_t)g.leader;
                    ranks[l][t]           = g.ranks;
                    bins[l][t]            = key;
                    if (has && g.leader == lane) base[l][t] = atomicAdd(&bin_counts[key], g.total);
                }
            }
            if (l >= 1 && l - 1 < a.ly.L && any_inside) store_layer(l - 1);
        }
        if (VETRAST_MAX_LAYERS - 1 < a.ly.L && any_inside) store_layer(VETRAST_MAX_LAYERS - 1);
    }
    if (packs) store_packed_row(pack, slot, row, row_confidence);
}

// The pass for one view: fetch, projection, and the above.
template <int HITS>
__device__ __forceinline__ void bin_scatter(const ViewPass& a, uint32_t* __restrict__ bin_counts,
                                            const ScatterTargets& out, const PackJob& pack)
{
    const int slot = blockIdx.x * blockDim.x + threadIdx.x;
    // the point this thread takes: the caller's processing order, if there is one (neighbours in a wave should be
    // neighbours in space; ids in the records are the caller's either way)
    const int i = (a.point_order != nullptr && slot < a.N) ? a.point_order[slot] : slot;
    Projected p;
    p.ipx = p.ipy = p.z = p.radius = 0.f;
    const bool visible = (uint32_t)i < (uint32_t)a.N && !point_is_skipped(a, i) && project_point(*a.view, a.position[i], p);
    scatter_projected<HITS>(a, bin_counts, out, pack, slot, i, visible, p);
}

template <int HITS>
__global__ void __launch_bounds__(kBlock) bin_scatter_kernel(ViewPass a, uint32_t* __restrict__ bin_counts,
                                                              ScatterTargets out, PackJob pack)
{
    bin_scatter<HITS>(a, bin_counts, out, pack);
}

struct ScatterArgs
{
    ViewPass view;
    uint32_t* bin_counts;
    ScatterTargets out;
    PackJob pack;
};

// The views of a round, one per blockIdx.y. (One pass over the points for all views of the round, each thread taking
// its point through one view after the other, reads the point arrays once instead of once per view; measured on four
// training crops it is slower by a fifth to a half, also with the fetch shared and only the projection repeated: the
// pass waits for its atomics, not for memory, and more, shorter threads hide more of that. Workgroups of the views
// taking turns, instead of all of one view before those of the next, is slower as well, by a tenth for crops and by
// half for full frames.)
template <int HITS>
__global__ void __launch_bounds__(kBlock) bin_scatter_views_kernel(PerView<ScatterArgs> views)
{
    const ScatterArgs& v = views.v[blockIdx.y];
    bin_scatter<HITS>(v.view, v.bin_counts, v.out, v.pack);
}

// The interleave as a launch of its own, for a caller that keeps the records across calls while texture and confidence
// stay as they are (vetrast_pack_descriptors): every row, whatever a view sees.
__global__ void __launch_bounds__(kBlock) pack_descriptors_kernel(PackJob pack)
{
    const int slot = blockIdx.x * blockDim.x + threadIdx.x;
    if (slot >= pack.N) return;
    float row[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci)
        if (ci < pack.C) row[ci] = pack.texture[(size_t)ci * pack.N + slot];
    store_packed_row(pack, slot, row, pack.confidence[slot]);
}

// Brings the logged records (rank beyond the bin's own room) to the bin's place in the compact array:
// binned[bin_offsets[bin] + rank]. Runs after the scan of the bin counts; the log is empty as a rule.
__device__ __forceinline__ void overflow_move(const ScatterTargets& in, const uint32_t* __restrict__ bin_offsets,
                                              uint4* __restrict__ binned, uint32_t capacity)
{
    for (uint32_t segment = blockIdx.x; segment < (uint32_t)kLogSegments; segment += gridDim.x)
    {
        const uint32_t entries = min(in.log_cursor[segment * kLogCursorStride], in.segment_capacity);
        const size_t first     = (size_t)segment * in.segment_capacity;
        for (uint32_t e = threadIdx.x; e < entries; e += blockDim.x)
        {
            const uint4 rec    = in.log[first + e];
            const uint32_t pos = bin_offsets[rec.w] + in.log_rank[first + e];
            if (pos >= capacity) continue;  // guard: never true
            if (in.compact)
                reinterpret_cast<uint2*>(binned)[pos] = make_uint2(rec.y, (rec.x << 8) | rec.z);
            else
                binned[pos] = make_uint4(rec.x, rec.y, rec.z, 0u);
        }
    }
}

__global__ void __launch_bounds__(kBlock) overflow_move_kernel(ScatterTargets in, const uint32_t* __restrict__ bin_offsets,
                                                                uint4* __restrict__ binned, uint32_t capacity)
{
    overflow_move(in, bin_offsets, binned, capacity);
}

// What the scan and move kernels of one view work on.
struct ScanArgs
{
    uint32_t* bin_counts;     // the counts; the scan-and-move kernel leaves its result `scanned_behind` words behind
    uint32_t scanned_behind;  // them, the two-launch scan in place
    uint32_t n;               // counts (scan and move in one launch)
    uint32_t* partials;       // one word per 4096 counts (scan in two launches)
    ScatterTargets in;
    uint4* binned;
    uint32_t capacity;
};

__global__ void __launch_bounds__(kBlock) overflow_move_views_kernel(PerView<ScanArgs> views)
{
    const ScanArgs& v = views.v[blockIdx.y];
    overflow_move(v.in, v.bin_counts, v.binned, v.capacity);
}

// ---- exclusive scan of the per-tile counts, in place, in two launches --------------------------------------------
// Launch 1: one partial sum per 4096 counts. Launch 2: every workgroup adds up the partials in front of it (a few
// hundred values, cache resident), then scans its own 4096 counts. No workgroup waits for another one.
// Counterpart of thrust::exclusive_scan + the two .item<int>() read-backs (src/lib/rendering/PointRenderer.cu:799-813);
// the total lands at counts[T] because the array is zero padded behind the T tile counts.
__device__ __forceinline__ uint32_t block_reduce_sum(uint32_t v, uint32_t* lds4)
{
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds4[wave] = v;
    __syncthreads();
    const uint32_t total = lds4[0] + lds4[1] + lds4[2] + lds4[3];
    __syncthreads();
    return total;
}

__device__ __forceinline__ void scan_partials(const uint4* __restrict__ counts4, uint32_t* __restrict__ partials)
{
    __shared__ uint32_t lds4[4];
    const uint4* src = counts4 + (size_t)blockIdx.x * (kScanPerBlock / 4);
    uint32_t sum     = 0;
#pragma unroll
    for (int k = 0; k < kScanPerThread / 4; ++k)
    {
        const uint4 v = src[k * kBlock + threadIdx.x];
        sum += (v.x + v.y) + (v.z + v.w);
    }
    const uint32_t total = block_reduce_sum(sum, lds4);
    if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

__global__ void __launch_bounds__(kBlock) scan_partials_kernel(const uint4* __restrict__ counts4,
                                                                uint32_t* __restrict__ partials)
{
    scan_partials(counts4, partials);
}

__global__ void __launch_bounds__(kBlock) scan_partials_views_kernel(PerView<ScanArgs> views)
{
    const ScanArgs& v = views.v[blockIdx.y];
    scan_partials(reinterpret_cast<const uint4*>(v.bin_counts), v.partials);
}

__device__ __forceinline__ void scan_apply(uint4* __restrict__ counts4, const uint32_t* __restrict__ partials)
{
    __shared__ uint32_t lds4[4];
    __shared__ uint32_t wave_tot[4];
    uint32_t before = 0;
    for (int k = threadIdx.x; k < (int)blockIdx.x; k += kBlock) before += partials[k];
    const uint32_t block_base = block_reduce_sum(before, lds4);

    // thread t owns the 16 consecutive counts [16 t, 16 t + 16) of this workgroup's 4096
    uint4* mine = counts4 + (size_t)blockIdx.x * (kScanPerBlock / 4) + threadIdx.x * (kScanPerThread / 4);
    uint4 v[kScanPerThread / 4];
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kScanPerThread / 4; ++k)
    {
        v[k] = mine[k];
        sum += (v[k].x + v[k].y) + (v[k].z + v[k].w);
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint32_t incl = wave_inclusive_scan(sum, lane);
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    uint32_t run = block_base + (incl - sum);
    for (int k = 0; k < wave; ++k) run += wave_tot[k];
#pragma unroll
    for (int k = 0; k < kScanPerThread / 4; ++k)
    {
        uint4 o;
        o.x = run;
        run += v[k].x;
        o.y = run;
        run += v[k].y;
        o.z = run;
        run += v[k].z;
        o.w = run;
        run += v[k].w;
        mine[k] = o;
    }
}

__global__ void __launch_bounds__(kBlock) scan_apply_kernel(uint4* __restrict__ counts4,
                                                             const uint32_t* __restrict__ partials)
{
    scan_apply(counts4, partials);
}

__global__ void __launch_bounds__(kBlock) scan_apply_views_kernel(PerView<ScanArgs> views)
{
    const ScanArgs& v = views.v[blockIdx.y];
    scan_apply(reinterpret_cast<uint4*>(v.bin_counts), v.partials);
}

// Scan and move in one launch, for up to kScanMoveMax counts: one workgroup per segment of the overflow log. Every
// workgroup whose segment holds entries scans the bin counts into LDS for itself and files its entries with them;
// workgroup 0 scans in any case and writes the result to `offsets` (the counts stay as they are, so that the other
// workgroups may read them meanwhile). As a rule the log is empty: 255 workgroups leave at once and the launch is the
// scan alone, where the two kernels cost a launch (and a dependency on the one before) each.
constexpr int kScanMoveMax = 60 * kBlock;  // 61 440 bytes of LDS

__device__ __forceinline__ void scan_move(const uint4* __restrict__ counts4, uint32_t n, uint4* __restrict__ offsets4,
                                          const ScatterTargets& in, uint4* __restrict__ binned, uint32_t capacity)
{
    __shared__ uint32_t s_off[kScanMoveMax];
    __shared__ uint32_t wave_tot[kBlock / kWave];
    const uint32_t segment = blockIdx.x;
    // (workgroup 0 scans whatever its segment holds: it asks for its cursor and for the counts at once)
    const uint32_t entries = min(in.log_cursor[segment * kLogCursorStride], in.segment_capacity);
    if (segment != 0u && entries == 0u) return;
    constexpr int kPer = kScanMoveMax / kBlock;  // 60 consecutive counts per thread, as 15 16-byte loads
    const uint4* src   = counts4 + threadIdx.x * (kPer / 4);
    uint4 v[kPer / 4];
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kPer / 4; ++k)
    {
        // (the array is zero padded to a multiple of 4096 counts, so whole loads never leave it)
        v[k] = (uint32_t)threadIdx.x * kPer + 4 * k < n ? src[k] : make_uint4(0u, 0u, 0u, 0u);
        sum += (v[k].x + v[k].y) + (v[k].z + v[k].w);
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint32_t incl = wave_inclusive_scan(sum, lane);
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    uint32_t run = incl - sum;
    for (int k = 0; k < wave; ++k) run += wave_tot[k];
    uint4* dst = offsets4 + threadIdx.x * (kPer / 4);
#pragma unroll
    for (int k = 0; k < kPer / 4; ++k)
    {
        uint4 o;
        o.x = run;
        run += v[k].x;
        o.y = run;
        run += v[k].y;
        o.z = run;
        run += v[k].z;
        o.w = run;
        run += v[k].w;
        if (segment == 0u && (uint32_t)threadIdx.x * kPer + 4 * k < n) dst[k] = o;
        if (entries != 0u) reinterpret_cast<uint4*>(s_off)[threadIdx.x * (kPer / 4) + k] = o;
    }
    if (entries == 0u) return;
    __syncthreads();
    const size_t first = (size_t)segment * in.segment_capacity;
    for (uint32_t e = threadIdx.x; e < entries; e += blockDim.x)
    {
        const uint4 rec    = in.log[first + e];
        const uint32_t pos = (rec.w < (uint32_t)kScanMoveMax ? s_off[rec.w] : capacity) + in.log_rank[first + e];
        if (pos >= capacity) continue;  // guard: never true
        if (in.compact)
            reinterpret_cast<uint2*>(binned)[pos] = make_uint2(rec.y, (rec.x << 8) | rec.z);
        else
            binned[pos] = make_uint4(rec.x, rec.y, rec.z, 0u);
    }
}

__global__ void __launch_bounds__(kBlock) scan_move_kernel(const uint4* __restrict__ counts4, uint32_t n,
                                                            uint4* __restrict__ offsets4, ScatterTargets in,
                                                            uint4* __restrict__ binned, uint32_t capacity)
{
    scan_move(counts4, n, offsets4, in, binned, capacity);
}

__global__ void __launch_bounds__(kBlock) scan_move_views_kernel(PerView<ScanArgs> views)
{
    const ScanArgs& v = views.v[blockIdx.y];
    scan_move(reinterpret_cast<const uint4*>(v.bin_counts), v.n,
              reinterpret_cast<uint4*>(v.bin_counts + v.scanned_behind), v.in, v.binned, v.capacity);
}

// Front-to-back blend of one pixel's sorted list read from memory: out += (T*c)*t, T = (1-c)*T, in exactly this order
// (BlendMulti, src/lib/rendering/RenderForward.cu:1303-1357). The list is walked in chunks of kBlendChunk fragments: all
// keys of a chunk are loaded first, then all descriptor records, and only then the (strictly sequential) arithmetic
// runs, so a thread keeps several gathers in flight instead of one dependent load chain per fragment.
template <int C>
__device__ __forceinline__ void blend_list_from_memory(const uint64_t* list, uint32_t n, const int32_t* index,
                                                       const float4* packed, int N, float* transmittance, float& T,
                                                       float (&color)[C])
{
    for (uint32_t base = 0; base < n; base += kBlendChunk)
    {
        int ti[kBlendChunk];
        float4 t4[kBlendChunk];
        float c[kBlendChunk];
#pragma unroll
        for (int u = 0; u < kBlendChunk; ++u)
        {
            ti[u] = -1;
            if (base + u < n)
            {
                const int id = (int)(uint32_t)list[base + u];
                // an id or texture index out of range cannot come from a list the scatter pass wrote; such a fragment is
                // skipped instead of gathered (the reference asserts on the texture index, RenderForward.cu:1335-1336)
                if ((uint32_t)id < (uint32_t)N) ti[u] = index ? index[id] : id;
                if ((uint32_t)ti[u] >= (uint32_t)N) ti[u] = -1;
            }
        }
#pragma unroll
        for (int u = 0; u < kBlendChunk; ++u)
        {
            if (ti[u] >= 0)
            {
                t4[u] = packed[2 * (size_t)ti[u]];
                c[u]  = packed[2 * (size_t)ti[u] + 1].x;
            }
        }
#pragma unroll
        for (int u = 0; u < kBlendChunk; ++u)
        {
            if (ti[u] >= 0)
            {
                if (transmittance) transmittance[base + u] = T;
                const float t[4] = {t4[u].x, t4[u].y, t4[u].z, t4[u].w};
                const float Tc   = T * c[u];
#pragma unroll
                for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                T = (1.f - c[u]) * T;
            }
        }
    }
}

}  // namespace vetrast
