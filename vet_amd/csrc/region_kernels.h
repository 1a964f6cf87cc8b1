// Region-major path of FULL_BLEND: one record per point and screen region instead of one per point and layer.
//
// The layers of the pyramid show the same part of the scene at 1, 1/2, 1/4 ... of the resolution, so the fragments a
// point leaves in the layers lie over each other on the screen. A REGION is a square of 16x16 pixels of layer 0 together
// with the 8x8, 4x4, 2x2 and 1 pixels of the coarser layers over the same area (pixel x of layer l belongs to region
// column x >> (4 - l)). The pass over the points writes ONE 32-byte record per point and region the point touches: its
// pixel in every layer, depth, id, and the point's confidence and descriptor, read with plain coalesced loads. Because
// every layer rounds the halved position on its own (src/lib/rendering/RenderForward.cu:856,888) the pixels of a point
// are not nested, so a point near a region border can touch two regions (up to four at a corner): 1.4 records per
// visible point on a 1080p frame. One workgroup per region then builds, sorts and blends the lists of all its pixels of
// all layers from records that sit in one place (no gather from a descriptor table per fragment), and the backward pass
// adds up the gradient of a record over all its layers in LDS and writes ONE row per record.
// Counterparts in the reference: CountingPrepassMulti / CollectMulti (src/lib/rendering/RenderForward.cu:806-905,
// 1011-1096), SortMulti (:1277-1300), BlendMulti (:1303-1357), BlendBackwards2 (src/lib/rendering/RenderBackward.cu:
// 1083-1513).
//
// Every region owns room for kRegionRoom records. A region that holds more (a surface seen edge-on puts thousands of
// points into a few pixels) is a HEAVY region: its later records go to a log, and it is built from global memory with
// (depth, id) keys and descriptors read from the caller's tensors, layer by layer as the bins of the per-layer path
// are. The host only takes this path where regions are expected to hold a few hundred records.
#pragma once
#include "backward_kernels.h"
#include "build_kernels.h"
#include "common.h"
#include "forward_kernels.h"
#include "sort_kernels.h"

namespace vetrast
{
constexpr int kRegionLog       = 4;
constexpr int kRegion          = 1 << kRegionLog;  // pixels of layer 0 along a region's side
constexpr int kRegionPixelsMax = 341;              // 256 + 64 + 16 + 4 + 1
constexpr int kRegionPixelsPad = 352;              // counters in LDS (a multiple of 32 above kRegionPixelsMax)
constexpr int kRegionRoom      = 1024;             // records a region has room for (and builds in LDS)
constexpr int kRegionKeys      = 1024;             // list places of a region built in LDS in one go
constexpr int kRegionIdBits    = 27;               // the layer mask of a record sits above the point id
constexpr uint32_t kRegionIdMask = (1u << kRegionIdBits) - 1u;
constexpr int kRegionCounterWords = 16;            // per view: [0] list places handed out to heavy regions

// The region kernels are launched three times over (grid.y): the workgroups of plane 0 take the regions with the most
// records, those of plane 2 the ordinary ones, and a workgroup whose region belongs to another plane leaves at once.
// A region's work grows with its records, a few regions hold ten times the median, and the hardware starts workgroups
// in grid order: so the long ones start first and the many short ones fill in behind them, instead of a long one
// starting last and the whole chip waiting for it.
constexpr int kRegionPlanes = 3;
__device__ __forceinline__ uint32_t region_plane(uint32_t records)
{
    return records > 640u ? 0u : (records > 256u ? 1u : 2u);
}

struct RegionTable
{
    int L;
    int w[VETRAST_MAX_LAYERS], h[VETRAST_MAX_LAYERS];
    uint32_t regions_x, regions;
    uint32_t ppr;                            // pixels of a region over all layers
    uint32_t first[VETRAST_MAX_LAYERS + 1];  // number (inside the region) of the first pixel of every layer; [L] = ppr
};

// Bits of a record's pixel word that hold the pixel of layer l: 8, 6, 4, 2 and 0 bits from bit 0, 8, 14, 18, 20 on.
__host__ __device__ __forceinline__ int region_code_shift(int l) { return l * (9 - l); }
__host__ __device__ __forceinline__ uint32_t region_code_mask(int l) { return (1u << (2 * (kRegionLog - l))) - 1u; }

// Record of a point in a region, two 16-byte halves:
//   a = (pixel of every layer the point hits inside this region, depth bits, point id | layer mask << 27, confidence)
//   t = descriptor (4 floats, zero padded)
// A logged record (heavy regions only) is the first three words of `a` and the region.

struct RegionTargets
{
    uint32_t* region_count;  // [regions] records per region (this view)
    uint4* rooms;            // [regions][kRegionRoom][2] (this view)
    uint4* log;              // [kLogSegments][segment_capacity]
    uint32_t* log_cursor;    // [kLogSegments], kLogCursorStride apart (this view)
    uint32_t segment_capacity;
    const float* texture;     // [C,N]
    const float* confidence;  // [N]
    int C;
    int texture_abs;
};

// The one pass over the points. Projection and the per-layer pixel as in bin_scatter_kernel; the layers a point hits
// are then grouped by region (one turn per distinct region of a lane, at most four), the wave groups the lanes of a
// turn by region and draws the ranks with one atomic per distinct region.
__global__ void __launch_bounds__(kBlock) region_scatter_kernel(ViewPass a, RegionTable rt, RegionTargets out)
{
    const int slot = blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = threadIdx.x & (kWave - 1);
    const int i    = (a.point_order != nullptr && slot < a.N) ? a.point_order[slot] : slot;
    Projected p;
    p.ipx = p.ipy = p.z = p.radius = 0.f;
    const bool visible = (uint32_t)i < (uint32_t)a.N && !point_is_skipped(a, i) && project_point(*a.view, a.position[i], p);
    float ipx = visible ? p.ipx : 0.f, ipy = visible ? p.ipy : 0.f, radius = visible ? p.radius : 0.f;
    const uint32_t depth_bits = __float_as_uint(p.z);
    const float reach = (float)(1 << (rt.L - 1)) + 1.f;  // see bin_scatter_kernel
    const bool inside = visible && ipx >= -reach && ipx <= (float)rt.w[0] + reach && ipy >= -reach &&
                        ipy <= (float)rt.h[0] + reach;
    if (__ballot(inside) == 0ull) return;  // the whole wave lies outside the image (most of the cloud, for a crop)
    // the point's descriptor row and confidence, asked for now and needed when the records are stored
    float row[4] = {0.f, 0.f, 0.f, 0.f}, conf = 0.f;
    if (inside)
    {
        const int ti = a.index ? a.index[i] : i;
        if ((uint32_t)ti < (uint32_t)a.N)  // a row out of range blends as fully transparent
        {
#pragma unroll
            for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci)
                if (ci < out.C) row[ci] = out.texture[(size_t)ci * a.N + ti];
            conf = out.confidence[ti];
        }
    }
    uint32_t reg[VETRAST_MAX_LAYERS], loc[VETRAST_MAX_LAYERS];
    uint32_t left = 0;  // layers the point hits, not yet filed under a region
    bool dropped  = !inside;
#pragma unroll
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
    {
        reg[l] = 0, loc[l] = 0;
        if (l >= rt.L) continue;
        if (a.drop_by_radius && radius < a.radius_threshold) dropped = true;
        const float fx = rintf(ipx), fy = rintf(ipy);
        if (dropped || !(fx >= 0.f && fx < (float)rt.w[l] && fy >= 0.f && fy < (float)rt.h[l])) continue;
        const uint32_t x = (uint32_t)(int)fx, y = (uint32_t)(int)fy;
        const int sl     = kRegionLog - l;
        reg[l]           = (y >> sl) * rt.regions_x + (x >> sl);
        loc[l]           = ((y & ((1u << sl) - 1u)) << sl) | (x & ((1u << sl) - 1u));
        left |= 1u << l;
    }
    constexpr int kTurns = 4;  // a point touches at most 2 x 2 regions
    uint32_t t_base[kTurns], t_who[kTurns], t_reg[kTurns], t_code[kTurns];  // who = leader | rank << 8 | mask << 24
    bool done = false;
#pragma unroll
    for (int t = 0; t < kTurns; ++t)
    {
        t_base[t] = 0, t_who[t] = 0, t_reg[t] = 0, t_code[t] = 0;
        if (!done && __ballot(left != 0u) == 0ull) done = true;  // the same for the whole wave
        if (done) continue;
        uint32_t key = 0;
#pragma unroll
        for (int l = VETRAST_MAX_LAYERS - 1; l >= 0; --l)
            if (left & (1u << l)) key = reg[l];  // region of the finest remaining layer
        uint32_t mask = 0, code = 0;
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
            if ((left & (1u << l)) && reg[l] == key)
            {
                mask |= 1u << l;
                code |= loc[l] << region_code_shift(l);
            }
        left &= ~mask;
        const bool has    = mask != 0u;
        const WaveGroup g = group_by_bin(has, key, lane);
        t_who[t]          = (uint32_t)g.leader | (g.rank << 8) | (mask << 24);
        t_reg[t]          = key;
        t_code[t]         = code;
        if (has && g.leader == lane) t_base[t] = atomicAdd(&out.region_count[key], g.count);
    }
    if (out.texture_abs)
    {
#pragma unroll
        for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci) row[ci] = fabsf(row[ci]);
    }
    if (a.confidence_activation) conf = sigmoid_canon(a.confidence_scale * conf);
#pragma unroll
    for (int t = 0; t < kTurns; ++t)
    {
        if (__ballot(t_who[t] >> 24) == 0ull) continue;
        const uint32_t mask = t_who[t] >> 24;
        const uint32_t rank = (uint32_t)__shfl((int)t_base[t], (int)(t_who[t] & 0xFFu), kWave) + ((t_who[t] >> 8) & 0xFFu);
        const uint32_t idm  = (uint32_t)i | (mask << kRegionIdBits);
        const bool valid    = mask != 0u;
        const bool over     = valid && rank >= (uint32_t)kRegionRoom;
        if (valid && !over)
        {
            uint4* rec = out.rooms + 2 * ((size_t)t_reg[t] * kRegionRoom + rank);
            rec[0]     = make_uint4(t_code[t], depth_bits, idm, __float_as_uint(conf));
            rec[1]     = make_uint4(__float_as_uint(row[0]), __float_as_uint(row[1]), __float_as_uint(row[2]),
                                    __float_as_uint(row[3]));
        }
        const uint64_t m = __ballot(over);
        if (m != 0ull)  // the region is a heavy one
        {
            const uint32_t segment = blockIdx.x % (uint32_t)kLogSegments;
            const int leader       = __ffsll((unsigned long long)m) - 1;
            uint32_t first         = 0;
            if (lane == leader) first = atomicAdd(out.log_cursor + segment * kLogCursorStride, (uint32_t)__popcll(m));
            first = (uint32_t)__shfl((int)first, leader, kWave);
            const uint32_t at =
                first + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
            if (over && at < out.segment_capacity)  // guard: a segment has room for every record of its workgroups
                out.log[(size_t)segment * out.segment_capacity + at] = make_uint4(t_code[t], depth_bits, idm, t_reg[t]);
        }
    }
}

// Order of the keys (depth bits << 32 | slot of the record in its region's room): by depth, then by the point id of the
// record, which is looked up in the room where two depths are equal (rare). The result is the order of the
// (depth bits, point id) keys the per-layer path sorts.
struct RegionLess
{
    const uint4* room;  // the region's records
    __device__ __forceinline__ bool operator()(uint64_t x, uint64_t y) const
    {
        bool lt           = x < y;
        const uint32_t dx = (uint32_t)(x >> 32), dy = (uint32_t)(y >> 32);
        const bool tie    = dx == dy && dx != 0xFFFFFFFFu && (uint32_t)x != (uint32_t)y;
        if (__ballot(tie) != 0ull)
        {
            if (tie)
                lt = (room[2 * (size_t)((uint32_t)x & 0xFFFFu)].z & kRegionIdMask) <
                     (room[2 * (size_t)((uint32_t)y & 0xFFFFu)].z & kRegionIdMask);
        }
        return lt;
    }
};

struct RegionPass
{
    RegionTable rt;
    const uint32_t* region_count;
    const uint4* rooms;
    const uint4* log;
    const uint32_t* log_cursor;
    uint32_t segment_capacity;
    uint32_t* counters;    // kRegionCounterWords words of this view
    uint2* region_info;    // [regions]: heavy regions: first list place of the region in list_key / heavy_T; list places
    uint2* pixel_info;     // [regions * ppr]: (start inside the region's places | count << 16), final transmittance
    uint2* heavy_pixel;    // [regions * ppr]: (start inside the region's places, count) of the pixels of heavy regions
    // A region built in LDS owns list_places places at [region * list_places, ...) of list_slot and list_T (one place
    // per record and layer at most): a cursor shared by all regions would be one address for thousands of atomics,
    // which the memory system retires one after the other.
    uint16_t* list_slot;   // per list place: the record's slot in the region's room
    float* list_T;         // per blended list place: transmittance in front of the fragment; null without a backward pass
    uint32_t list_places;  // L * kRegionRoom
    // heavy regions draw their places from one cursor (there are few of them)
    uint64_t* list_key;    // per list place of a heavy region: depth bits << 32 | point id
    float* heavy_T;        // the same places: transmittance in front of the fragment; null without a backward pass
    uint32_t list_capacity;
    // descriptors as the caller holds them (heavy regions)
    const float* texture;
    const float* confidence;
    const int32_t* index;
    int N, C;
    int confidence_activation;
    float confidence_scale;
    int texture_abs;
    const float* background;  // as it is blended
    float* out[VETRAST_MAX_LAYERS];
    float* out_mask[VETRAST_MAX_LAYERS];
    float* out_weight[VETRAST_MAX_LAYERS];
    int K;
    int use_environment_map;
    float mask_value;
};

// Confidence and descriptor of point `id` as the scatter pass puts them into a record.
template <class P>
__device__ __forceinline__ void region_fetch_descriptor(const P& a, int id, float4& t4, float& conf)
{
    t4   = make_float4(0.f, 0.f, 0.f, 0.f);
    conf = 0.f;
    int ti = -1;
    if ((uint32_t)id < (uint32_t)a.N) ti = a.index ? a.index[id] : id;
    if ((uint32_t)ti >= (uint32_t)a.N) return;
    float row[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci)
        if (ci < a.C) row[ci] = a.texture[(size_t)ci * a.N + ti];
    conf = a.confidence[ti];
    if (a.texture_abs)
    {
#pragma unroll
        for (int ci = 0; ci < VETRAST_MAX_CHANNELS; ++ci) row[ci] = fabsf(row[ci]);
    }
    if (a.confidence_activation) conf = sigmoid_canon(a.confidence_scale * conf);
    t4 = make_float4(row[0], row[1], row[2], row[3]);
}

// Layer of pixel number `px` of a region.
__device__ __forceinline__ int region_layer_of(const RegionTable& rt, uint32_t px)
{
    int l = 0;
#pragma unroll
    for (int k = 1; k < VETRAST_MAX_LAYERS; ++k)
        if (k < rt.L && px >= rt.first[k]) l = k;
    return l;
}

// Exclusive scan of the kRegionPixelsPad counters of a region by the whole workgroup (two counters per thread);
// returns the total. s_start[kRegionPixelsPad] is set to the total as well.
__device__ __forceinline__ uint32_t region_scan(const uint32_t* s_cnt, uint32_t* s_start, uint32_t* s_wave_tot, int tid)
{
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    uint32_t c0 = 0, c1 = 0;
    if (2 * tid + 1 < kRegionPixelsPad)
    {
        c0 = s_cnt[2 * tid];
        c1 = s_cnt[2 * tid + 1];
    }
    const uint32_t v    = c0 + c1;
    const uint32_t incl = wave_inclusive_scan(v, lane);
    if (lane == kWave - 1) s_wave_tot[wave] = incl;
    __syncthreads();
    uint32_t start = incl - v;
    for (int k = 0; k < wave; ++k) start += s_wave_tot[k];
    if (2 * tid + 1 < kRegionPixelsPad)
    {
        s_start[2 * tid]     = start;
        s_start[2 * tid + 1] = start + c0;
    }
    const uint32_t total = (s_wave_tot[0] + s_wave_tot[1]) + (s_wave_tot[2] + s_wave_tot[3]);
    if (tid == 0) s_start[kRegionPixelsPad] = total;
    __syncthreads();
    return total;
}

// ---- forward: per-pixel lists (count, scan, placement, sort), blend, outputs ------------------------------------------
//
// A workgroup's life is a chain of memory round trips and barriers, which the chip hides only with many workgroups in
// flight, and a region's work grows with its records while a few regions hold ten times the median. So:
//   * an ordinary region (at most kStage records) is built by ONE workgroup, all layers in one go: a thread holds one
//     record in registers from the first load to the placement, the region's descriptors sit in an LDS table indexed by
//     the record's slot, and the blend walks a pixel's list without any gather or barrier;
//   * a big region (up to kRegionRoom records) is built by one workgroup PER LAYER, as a bin of the per-layer path is:
//     four times the workgroups in flight for the regions whose chains are the longest;
//   * a heavy region (more records than its room) by one workgroup from global memory.
// The kernel is launched L + 1 times over (grid.y): planes 0 .. L-1 are the layers of the big regions (plane 0 also
// takes the heavy ones), plane L the ordinary regions; a workgroup whose region belongs elsewhere leaves at once. The
// hardware starts workgroups in grid order, so the long chains start first and the many short ones fill in behind them.
// Registers (64) and LDS (under 20 KB) are kept to what lets eight workgroups share a compute unit.
struct RegionShared
{
    uint32_t cnt[kRegionPixelsPad];
    uint32_t start[kRegionPixelsPad + 1];
    uint32_t wave_tot[kBlock / kWave];
    uint32_t misc[4];
    uint8_t src_lane[kBlock / kWave][kWave];
    uint64_t block_sorted[kBlock / kWave];
    uint64_t keys[kRegionKeys];
    uint16_t pix[kRegionKeys];   // pixel of every list place (heavy regions: places handed out per pixel, as uint32)
    float4 stage_t[kStage];      // descriptors: of the region's records by slot, or of a stretch of blended fragments
    float stage_c[kStage];       // confidences, likewise
};
static_assert(kRegionKeys >= kBuildCap, "block_sort_in_lds sorts through the key array");
static_assert(kRegionPixelsPad * sizeof(uint32_t) <= kRegionKeys * sizeof(uint16_t), "a heavy region's cursors borrow the pixel array");
static_assert((kLogSegments + 1) * sizeof(uint32_t) <= sizeof(float4) * kStage, "the log's segment starts borrow the stage");

__device__ __forceinline__ bool region_is_small(uint32_t records, int L)
{
    return records <= (uint32_t)kStage && records * (uint32_t)L <= (uint32_t)kRegionKeys;
}

// Blend step of one fragment: out += (T * c) * t, T = (1 - c) * T (BlendMulti, src/lib/rendering/RenderForward.cu:1343-1346).
template <int C>
__device__ __forceinline__ void region_blend_step(float4 t4, float cf, float& T, float (&color)[C])
{
    const float t[4] = {t4.x, t4.y, t4.z, t4.w};
    const float Tc   = T * cf;
#pragma unroll
    for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
    T = (1.f - cf) * T;
}

// Stores what the forward pass leaves for a pixel: the blended features (background included), mask and weight images,
// and the pixel's list bounds and final transmittance.
template <int C>
__device__ __forceinline__ void region_store_pixel(const RegionPass& a, uint32_t region, int l, uint32_t loc, float T,
                                                   const float (&color)[C], uint32_t start, uint32_t cnt, bool heavy)
{
    const RegionTable& rt = a.rt;
    const uint32_t ry = region / rt.regions_x, rx = region - ry * rt.regions_x;
    const int sl = kRegionLog - l;
    const int x = (int)((rx << sl) + (loc & ((1u << sl) - 1u))), y = (int)((ry << sl) + (loc >> sl));
    const size_t q = (size_t)region * rt.ppr + rt.first[l] + loc;
    float Tf = 1.f;
    if (x < rt.w[l] && y < rt.h[l])
    {
        const size_t plane   = (size_t)rt.w[l] * rt.h[l];
        const uint32_t local = (uint32_t)y * (uint32_t)rt.w[l] + (uint32_t)x;
        Tf                   = T;
#pragma unroll
        for (int ci = 0; ci < C; ++ci)
        {
            float v = color[ci];
            if (!a.use_environment_map) v = (Tf * 1.f) * a.background[ci] + v;
            a.out[l][ci * plane + local] = v;
        }
        if (a.out_mask[l]) a.out_mask[l][local] = (Tf == 0.f) ? a.mask_value : 1.f;
        if (a.out_weight[l]) a.out_weight[l][local] = Tf;
    }
    if (heavy)
    {
        a.heavy_pixel[q] = make_uint2(start, cnt);
        a.pixel_info[q]  = make_uint2(0u, __float_as_uint(Tf));
    }
    else
        a.pixel_info[q] = make_uint2(start | (cnt << 16), __float_as_uint(Tf));
}

// An ordinary region: n <= kStage records, one per thread; `ra`, `rt4` are the two halves of thread tid's record (asked
// for before n was known: whatever lies in the room behind the n-th record is ignored).
template <int C>
__device__ __forceinline__ void region_forward_small(const RegionPass& a, RegionShared& s, uint32_t region, uint32_t n,
                                                     uint4 ra, uint4 rt4)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const RegionTable& rt = a.rt;
    const uint4* room     = a.rooms + 2 * (size_t)region * kRegionRoom;
    const bool mine       = (uint32_t)tid < n;
    const uint32_t mask   = mine ? ra.z >> kRegionIdBits : 0u;
    // count per pixel; the LDS atomic also hands the record its rank inside the pixel (10 bits per layer)
    uint64_t ranks = 0ull;
#pragma unroll
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
        if (mask & (1u << l))
        {
            const uint32_t px = rt.first[l] + ((ra.x >> region_code_shift(l)) & region_code_mask(l));
            ranks |= (uint64_t)atomicAdd(&s.cnt[px], 1u) << (10 * l);
        }
    if (mine)
    {
        s.stage_t[tid] = make_float4(__uint_as_float(rt4.x), __uint_as_float(rt4.y), __uint_as_float(rt4.z), __uint_as_float(rt4.w));
        s.stage_c[tid] = __uint_as_float(ra.w);
    }
    __syncthreads();
    const uint32_t n_keys = region_scan(s.cnt, s.start, s.wave_tot, tid);
    if (tid == 0) a.region_info[region] = make_uint2(0u, n_keys);
#pragma unroll
    for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
        if (mask & (1u << l))
        {
            const uint32_t px    = rt.first[l] + ((ra.x >> region_code_shift(l)) & region_code_mask(l));
            const uint32_t place = s.start[px] + (uint32_t)((ranks >> (10 * l)) & 0x3FFu);
            s.keys[place]        = ((uint64_t)ra.y << 32) | (uint32_t)tid;
            s.pix[place]         = (uint16_t)px;
        }
    __syncthreads();
    // A thread owns pixel tid of layer 0 and pixel `lane` of layer 1 + wave (the 64, 16, 4 and 1 pixels of layers 1 to
    // 4): the lists of a wave's second round are about equally long, so the wave runs sorting networks of one or two
    // sizes, each filled with lists, and its threads walk about as many fragments each.
    static_assert(VETRAST_MAX_LAYERS - 1 <= kBlock / kWave, "one wave per coarse layer");
    constexpr int kOwned = 2;
    uint32_t own_px[kOwned], own_start[kOwned], own_cnt[kOwned];
    own_px[0] = (uint32_t)tid;
    own_px[1] = rt.ppr;
    if (1 + wave < rt.L && (uint32_t)lane < rt.first[2 + wave] - rt.first[1 + wave]) own_px[1] = rt.first[1 + wave] + (uint32_t)lane;
    const RegionLess less{room};
#pragma unroll
    for (int o = 0; o < kOwned; ++o)
    {
        own_start[o] = own_cnt[o] = 0u;
        if (own_px[o] < rt.ppr)
        {
            own_start[o] = s.start[own_px[o]];
            own_cnt[o]   = s.cnt[own_px[o]];
        }
        if (__ballot(own_cnt[o] > 1u) != 0ull)
            sort_wave_lists(s.keys, s.src_lane[wave], own_start[o], own_cnt[o], lane, a.K, 0u, less);
    }
    __syncthreads();
    const size_t list_base = (size_t)region * a.list_places;
    for (uint32_t r = tid; r < n_keys; r += kBlock) a.list_slot[list_base + r] = (uint16_t)(uint32_t)s.keys[r];
    // blend: a pixel's places are read and written by its own thread only; the depth half of a key makes room for the
    // transmittance in front of the fragment
    float* s_T            = reinterpret_cast<float*>(s.keys);
    const uint32_t* s_low = reinterpret_cast<const uint32_t*>(s.keys);
#pragma unroll
    for (int o = 0; o < kOwned; ++o)
    {
        if (own_px[o] >= rt.ppr) continue;
        float T = 1.f, color[C];
#pragma unroll
        for (int ci = 0; ci < C; ++ci) color[ci] = 0.f;
        const uint32_t keep = a.K > 0 ? min(own_cnt[o], (uint32_t)a.K) : own_cnt[o];
        for (uint32_t q = own_start[o]; q < own_start[o] + keep; ++q)
        {
            const uint32_t slot = s_low[2 * q] & 0xFFFFu;
            s_T[2 * q + 1]      = T;
            region_blend_step<C>(s.stage_t[slot], s.stage_c[slot], T, color);
        }
        const int l = o == 0 ? 0 : 1 + wave;
        region_store_pixel<C>(a, region, l, own_px[o] - rt.first[l], T, color, own_start[o], own_cnt[o], false);
    }
    if (a.list_T)
    {
        __syncthreads();
        for (uint32_t r = tid; r < n_keys; r += kBlock)
        {
            const uint32_t px  = s.pix[r];
            const uint32_t len = a.K > 0 ? min(s.cnt[px], (uint32_t)a.K) : s.cnt[px];
            if (r - s.start[px] < len) a.list_T[list_base + r] = s_T[2 * r + 1];
        }
    }
}

// One layer of a big region (more than kStage and at most kRegionRoom records): a thread holds up to four records and
// owns one pixel; the blended fragments' descriptors are gathered from the region's room (which the L2 holds) into the
// stage, a stretch of kStage blended fragments at a time.
template <int C>
__device__ __forceinline__ void region_forward_layer(const RegionPass& a, RegionShared& s, uint32_t region, uint32_t n, int l)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const RegionTable& rt = a.rt;
    const uint4* room     = a.rooms + 2 * (size_t)region * kRegionRoom;
    const uint32_t npx    = rt.first[l + 1] - rt.first[l];  // 256, 64, 16, 4 or 1
    constexpr int kPerThread = kRegionRoom / kBlock;
    uint32_t where[kPerThread], depth[kPerThread];  // pixel | rank << 8 | valid << 31
#pragma unroll
    for (int k = 0; k < kPerThread; ++k)
    {
        where[k] = depth[k] = 0u;
        const uint32_t r = (uint32_t)(k * kBlock + tid);
        if (r < n)
        {
            const uint4 ra = room[2 * (size_t)r];
            if ((ra.z >> kRegionIdBits) & (1u << l))
            {
                const uint32_t px = (ra.x >> region_code_shift(l)) & region_code_mask(l);
                where[k]          = px | (atomicAdd(&s.cnt[px], 1u) << 8) | 0x80000000u;
                depth[k]          = ra.y;
            }
        }
    }
    __syncthreads();
    // scan of the layer's (at most kBlock) pixel counts, one per thread
    const uint32_t cnt  = (uint32_t)tid < npx ? s.cnt[tid] : 0u;
    uint32_t incl       = wave_inclusive_scan(cnt, lane);
    if (lane == kWave - 1) s.wave_tot[wave] = incl;
    __syncthreads();
    uint32_t start = incl - cnt;
    for (int k = 0; k < wave; ++k) start += s.wave_tot[k];
    const uint32_t n_keys = (s.wave_tot[0] + s.wave_tot[1]) + (s.wave_tot[2] + s.wave_tot[3]);
    s.start[tid] = start;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kPerThread; ++k)
        if (where[k] & 0x80000000u)
        {
            const uint32_t px    = where[k] & 0xFFu;
            const uint32_t place = s.start[px] + ((where[k] >> 8) & 0x7FFFFFu);
            s.keys[place]        = ((uint64_t)depth[k] << 32) | (uint32_t)(k * kBlock + tid);
            s.pix[place]         = (uint16_t)px;
        }
    __syncthreads();
    {
        // a wave sorts 64 of the layer's 256 pixels, or every fourth pixel of a coarser layer (whose few lists are long)
        const uint32_t px = npx >= (uint32_t)kBlock ? (uint32_t)tid : 4u * lane + wave;
        uint32_t off = 0, len = 0;
        if (px < npx)
        {
            off = s.start[px];
            len = s.cnt[px];
        }
        const RegionLess less{room};
        if (__ballot(len > 1u) != 0ull) sort_wave_lists(s.keys, s.src_lane[wave], off, len, lane, a.K, 0u, less);
    }
    __syncthreads();
    // the layer's list places: kRegionRoom places from place l * kRegionRoom of the region's stretch on
    const uint32_t layer_base = (uint32_t)l * kRegionRoom;
    const size_t list_base    = (size_t)region * a.list_places + layer_base;
    for (uint32_t r = tid; r < n_keys; r += kBlock) a.list_slot[list_base + r] = (uint16_t)(uint32_t)s.keys[r];
    // the blended fragments of all pixels, numbered pixel after pixel: kstart[px] = blended fragments in front of pixel px
    const uint32_t keep = a.K > 0 ? min(cnt, (uint32_t)a.K) : cnt;
    incl                = wave_inclusive_scan(keep, lane);
    __syncthreads();  // (the scan totals of the counts have been read)
    if (lane == kWave - 1) s.wave_tot[wave] = incl;
    __syncthreads();
    uint32_t kstart = incl - keep;
    for (int k = 0; k < wave; ++k) kstart += s.wave_tot[k];
    const uint32_t n_kept = (s.wave_tot[0] + s.wave_tot[1]) + (s.wave_tot[2] + s.wave_tot[3]);
    uint32_t* s_kstart    = s.cnt;  // the counts live on in their owners' registers
    s_kstart[tid]         = kstart;
    if (tid == 0) s_kstart[kBlock] = n_kept;
    __syncthreads();
    float* s_T            = reinterpret_cast<float*>(s.keys);
    const uint32_t* s_low = reinterpret_cast<const uint32_t*>(s.keys);
    float T = 1.f, color[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) color[ci] = 0.f;
    for (uint32_t base = 0; base < n_kept; base += kStage)
    {
        const uint32_t i = base + tid;
        if (i < n_kept)
        {
            uint32_t lo = 0, hi = (uint32_t)kBlock;  // s_kstart[lo] <= i < s_kstart[hi]
            while (hi - lo > 1u)
            {
                const uint32_t mid = (lo + hi) >> 1;
                if (s_kstart[mid] <= i)
                    lo = mid;
                else
                    hi = mid;
            }
            const uint32_t place = s.start[lo] + (i - s_kstart[lo]);
            const uint32_t slot  = s_low[2 * place] & 0xFFFFu;
            const uint4 ra       = room[2 * (size_t)slot];
            const uint4 rt4      = room[2 * (size_t)slot + 1];
            s.stage_t[tid] = make_float4(__uint_as_float(rt4.x), __uint_as_float(rt4.y), __uint_as_float(rt4.z), __uint_as_float(rt4.w));
            s.stage_c[tid] = __uint_as_float(ra.w);
        }
        __syncthreads();
        const uint32_t lo = max(kstart, base), hi = min(kstart + keep, base + (uint32_t)kStage);
        for (uint32_t i2 = lo; i2 < hi; ++i2)
        {
            s_T[2 * (start + (i2 - kstart)) + 1] = T;
            region_blend_step<C>(s.stage_t[i2 - base], s.stage_c[i2 - base], T, color);
        }
        __syncthreads();
    }
    if ((uint32_t)tid < npx) region_store_pixel<C>(a, region, l, (uint32_t)tid, T, color, layer_base + start, cnt, false);
    if (a.list_T)
        for (uint32_t r = tid; r < n_keys; r += kBlock)
        {
            const uint32_t px = s.pix[r];
            if (r - s.start[px] < s_kstart[px + 1] - s_kstart[px]) a.list_T[list_base + r] = s_T[2 * r + 1];
        }
}

// A heavy region: lists of (depth, id) keys in global memory, sorted there, as a streamed bin of bin_build_kernel;
// descriptors from the caller's tensors.
template <int C>
__device__ __forceinline__ void region_forward_heavy(const RegionPass& a, RegionShared& s, uint32_t region)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const RegionTable& rt = a.rt;
    const uint4* room     = a.rooms + 2 * (size_t)region * kRegionRoom;
    uint32_t* s_cur       = reinterpret_cast<uint32_t*>(s.pix);       // places handed out per pixel
    uint32_t* s_log_start = reinterpret_cast<uint32_t*>(s.stage_t);   // entries of the log in front of every segment
    for (int p = tid; p < kRegionPixelsPad; p += kBlock) s_cur[p] = 0u;
    static_assert(kLogSegments == kBlock, "one thread per log segment");
    uint32_t log_total;
    {
        const uint32_t mine = min(a.log_cursor[tid * kLogCursorStride], a.segment_capacity);
        const uint32_t incl = wave_inclusive_scan(mine, lane);
        if (lane == kWave - 1) s.wave_tot[wave] = incl;
        __syncthreads();
        uint32_t before = incl - mine;
        for (int k = 0; k < wave; ++k) before += s.wave_tot[k];
        s_log_start[tid] = before;
        log_total        = (s.wave_tot[0] + s.wave_tot[1]) + (s.wave_tot[2] + s.wave_tot[3]);
        if (tid == 0) s_log_start[kLogSegments] = log_total;
    }
    __syncthreads();
    // entry e of the log (its segments taken as one run): the segment is the last one that starts at or in front of e
    auto log_entry = [&](uint32_t e) {
        uint32_t lo = 0, hi = (uint32_t)kLogSegments;
        while (hi - lo > 1u)
        {
            const uint32_t mid = (lo + hi) >> 1;
            if (s_log_start[mid] <= e)
                lo = mid;
            else
                hi = mid;
        }
        return a.log[(size_t)lo * a.segment_capacity + (e - s_log_start[lo])];
    };
    // all records of the region: those in its room, and the entries of the log that belong to it
    auto for_each_record = [&](auto&& f) {
        for (uint32_t r = tid; r < (uint32_t)kRegionRoom; r += kBlock)
        {
            const uint4 rec = room[2 * (size_t)r];
            f(rec.x, rec.y, rec.z);
        }
        for (uint32_t e0 = 0; e0 < log_total; e0 += 4 * kBlock)
        {
            uint4 rec[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const uint32_t e = e0 + u * kBlock + tid;
                rec[u]           = e < log_total ? log_entry(e) : make_uint4(0u, 0u, 0u, 0xFFFFFFFFu);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (rec[u].w == region) f(rec[u].x, rec[u].y, rec[u].z);
        }
    };
    for_each_record([&](uint32_t pixels, uint32_t, uint32_t idm) {
        const uint32_t m = idm >> kRegionIdBits;
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
            if (m & (1u << l)) atomicAdd(&s.cnt[rt.first[l] + ((pixels >> region_code_shift(l)) & region_code_mask(l))], 1u);
    });
    __syncthreads();
    const uint32_t n_keys = region_scan(s.cnt, s.start, s.wave_tot, tid);
    if (tid == 0)
    {
        // the region's list places in the view's key array: heavy regions are few, so one cursor does
        uint32_t base = atomicAdd(&a.counters[0], n_keys);
        if (base > a.list_capacity - n_keys) base = 0u;  // guard: the places of a view are bounded by its capacity
        s.misc[0]             = base;
        a.region_info[region] = make_uint2(base, n_keys);
    }
    __syncthreads();
    const uint32_t list_base = s.misc[0];
    uint64_t* list           = a.list_key + list_base;
    for_each_record([&](uint32_t pixels, uint32_t depth_bits, uint32_t idm) {
        const uint32_t m = idm >> kRegionIdBits;
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
            if (m & (1u << l))
            {
                const uint32_t px   = rt.first[l] + ((pixels >> region_code_shift(l)) & region_code_mask(l));
                const uint32_t rank = atomicAdd(&s_cur[px], 1u);
                list[s.start[px] + rank] = ((uint64_t)depth_bits << 32) | (idm & kRegionIdMask);
            }
    });
    __threadfence_block();
    __syncthreads();
    // Every list is sorted in full, whatever the cut: the backward pass walks the fragments behind the cut as well (it
    // owes each of them a row of zeros), so a list has to stay a permutation of its fragments, which the selection of
    // the K nearest does not leave behind.
    for (uint32_t j0 = 0; j0 < rt.ppr; j0 += kBlock)
    {
        const uint32_t px = j0 + 4u * lane + wave;
        uint32_t off = 0, len = 0;
        if (px < rt.ppr)
        {
            off = s.start[px];
            len = s.cnt[px];
        }
        sort_wave_lists(list, s.src_lane[wave], off, len, lane, /*K=*/0, /*skip_longer=*/(uint32_t)kBuildCap);
    }
    __threadfence_block();
    __syncthreads();
    // lists too long for a wave's registers: by the whole workgroup through the key array in LDS, one after the other
    for (uint32_t j0 = 0; j0 < rt.ppr; j0 += kBlock)
    {
        const uint32_t px = j0 + tid;
        const bool mine   = px < rt.ppr && s.cnt[px] > kRegisterSortKeys && s.cnt[px] <= (uint32_t)kBuildCap;
        const uint64_t wave_mask = __ballot(mine);
        if (lane == 0) s.block_sorted[wave] = wave_mask;
        __syncthreads();
        for (int w = 0; w < kBlock / kWave; ++w)
        {
            uint64_t todo = s.block_sorted[w];
            while (todo != 0ull)
            {
                const uint32_t p = j0 + w * kWave + (__ffsll((unsigned long long)todo) - 1);
                todo &= todo - 1ull;
                block_sort_in_lds(list + s.start[p], s.cnt[p], s.keys, tid);
            }
        }
        __syncthreads();
    }
    __threadfence_block();
    __syncthreads();
    // blend through the stage: all threads fetch the descriptors of a stretch of list places, then the thread of a pixel
    // walks its fragments of that stretch. A thread owns pixel tid and pixel kBlock + tid.
    constexpr int kOwned = 2;
    uint32_t start[kOwned], keep[kOwned];
    float T[kOwned], color[kOwned][C];
#pragma unroll
    for (int o = 0; o < kOwned; ++o)
    {
        const uint32_t px = (uint32_t)(o * kBlock + tid);
        start[o] = keep[o] = 0u;
        T[o] = 1.f;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) color[o][ci] = 0.f;
        if (px < rt.ppr)
        {
            start[o] = s.start[px];
            keep[o]  = a.K > 0 ? min(s.cnt[px], (uint32_t)a.K) : s.cnt[px];
        }
    }
    for (uint32_t base = 0; base < n_keys; base += kStage)
    {
        const uint32_t r = base + tid;
        if (r < n_keys)
        {
            uint32_t lo = 0, hi = rt.ppr;  // pixel of place r: s.start[lo] <= r < s.start[hi]
            while (hi - lo > 1u)
            {
                const uint32_t mid = (lo + hi) >> 1;
                if (s.start[mid] <= r)
                    lo = mid;
                else
                    hi = mid;
            }
            const uint32_t len = a.K > 0 ? min(s.cnt[lo], (uint32_t)a.K) : s.cnt[lo];
            if (r - s.start[lo] < len)
            {
                float4 t4;
                float cf;
                region_fetch_descriptor(a, (int)(uint32_t)list[r], t4, cf);
                s.stage_t[tid] = t4;
                s.stage_c[tid] = cf;
            }
        }
        __syncthreads();
#pragma unroll
        for (int o = 0; o < kOwned; ++o)
        {
            const uint32_t lo = max(start[o], base), hi = min(start[o] + keep[o], base + (uint32_t)kStage);
            for (uint32_t q = lo; q < hi; ++q)
            {
                if (a.heavy_T) a.heavy_T[list_base + q] = T[o];
                region_blend_step<C>(s.stage_t[q - base], s.stage_c[q - base], T[o], color[o]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int o = 0; o < kOwned; ++o)
    {
        const uint32_t px = (uint32_t)(o * kBlock + tid);
        if (px >= rt.ppr) continue;
        const int l = region_layer_of(rt, px);
        region_store_pixel<C>(a, region, l, px - rt.first[l], T[o], color[o], s.start[px], s.cnt[px], true);
    }
}

template <int C>
__global__ void __launch_bounds__(kBlock) region_forward_kernel(RegionPass a)
{
    __shared__ RegionShared s;
    const int tid         = threadIdx.x;
    const uint32_t region = blockIdx.x;
    const int plane       = (int)blockIdx.y;  // 0 .. L-1: a layer of a big region; L: an ordinary region
    const int L           = a.rt.L;
    const uint4* room     = a.rooms + 2 * (size_t)region * kRegionRoom;
    // thread tid's record, asked for together with the region's record count
    uint4 ra = make_uint4(0u, 0u, 0u, 0u), rt4 = ra;
    if (plane == L)
    {
        ra  = room[2 * (size_t)tid];
        rt4 = room[2 * (size_t)tid + 1];
    }
    const uint32_t n_all = (uint32_t)__builtin_amdgcn_readfirstlane((int)a.region_count[region]);
    const bool small = region_is_small(n_all, L), heavy = n_all > (uint32_t)kRegionRoom;
    if (plane == L ? !small : (small || (heavy && plane != 0))) return;
    for (int p = tid; p < kRegionPixelsPad; p += kBlock) s.cnt[p] = 0u;
    __syncthreads();
    if (plane == L)
        region_forward_small<C>(a, s, region, n_all, ra, rt4);
    else if (heavy)
        region_forward_heavy<C>(a, s, region);
    else
    {
        if (tid == 0 && plane == 0) a.region_info[region] = make_uint2(0u, 0u);
        region_forward_layer<C>(a, s, region, n_all, plane);
    }
}

struct RegionBackwardPass
{
    RegionTable rt;
    const uint32_t* region_count;
    const uint4* rooms;
    const uint2* region_info;
    const uint2* pixel_info;
    const uint2* heavy_pixel;
    const uint16_t* list_slot;
    const float* list_T;
    uint32_t list_places;
    const uint64_t* list_key;
    const float* heavy_T;
    const float* texture;
    const float* confidence;
    const int32_t* index;
    int N, C;
    int confidence_activation;
    float confidence_scale;
    int texture_abs;
    const float* background;
    const float* grad_out[VETRAST_MAX_LAYERS];
    const float* out[VETRAST_MAX_LAYERS];
    float4* partial;            // [L][N][2]: (d tex0..3), (d conf, d image x, d image y in pixels of layer 0, fragments with a position gradient)
    float* background_partial;  // [regions][kBackgroundRow]
    int K;
    int use_environment_map;
    int need_point_gradient;
    int quirk_background_confidence_leak;
    ClearJob clear;
};

// LDS of one wave of the backward kernel: what blend_backward_kernel keeps per pixel lane, and the item table.
struct RegionWaveShared
{
    uint32_t off[kWave];
    uint32_t base[kWave];
    float carry[kWave];
    float4 g[kWave];
    float4 ax[kWave];
    float4 ay[kWave];
    float2 bxy[kWave];
    uint8_t point[kWave];
    uint8_t item[kWaveItems];
};

// One layer of one region by one wave: the per-pixel part and the dense fragment rounds of blend_backward_kernel (see
// there for the arithmetic) on the pixels wave * per_wave + lane of the layer. Where the gradient of a fragment goes:
//   kRowsInLds     the row of its record in LDS (s_lo / s_hi / s_n, indexed by slot): a record has at most one fragment
//                  per layer and the layers are taken one after the other, so plain adds do;
//   kRowsInMemory  the same row at its final place, partial[first layer of the record][point], added to through the L2
//                  (regions with more records than the LDS rows hold; the kernel has cleared the rows before);
//   kRowsPerLayer  heavy regions: stored at partial[layer][point], and so is a row of zeros for every fragment behind
//                  the cut.
constexpr int kRowsInLds = 0, kRowsInMemory = 1, kRowsPerLayer = 2;
template <int C, int ROWS>
__device__ __forceinline__ void region_backward_layer(const RegionBackwardPass& a, uint32_t region, int l,
                                                      size_t list_base, RegionWaveShared& s, float4* s_lo, float* s_hi,
                                                      uint8_t* s_n, float (&bg_grad)[C], float& leak, int lane, int wave)
{
    const RegionTable& rt = a.rt;
    const int sl          = kRegionLog - l;
    const uint32_t npx    = 1u << (2 * sl);
    const uint32_t per_wave = (npx + 3u) / 4u;
    const uint32_t j        = (uint32_t)wave * per_wave + (uint32_t)lane;
    const bool has_px       = (uint32_t)lane < per_wave && j < npx;
    const uint32_t ry = region / rt.regions_x, rx = region - ry * rt.regions_x;
    const int x = (int)((rx << sl) + (j & ((1u << sl) - 1u))), y = (int)((ry << sl) + (j >> sl));
    const int lw = rt.w[l], lh = rt.h[l];
    constexpr bool HEAVY = ROWS == kRowsPerLayer;
    const bool active = has_px && x < lw && y < lh;
    const uint4* room = a.rooms + 2 * (size_t)region * kRegionRoom;
    const float layer_scale = __uint_as_float((uint32_t)(127 - l) << 23);  // 0.5^l
    uint32_t n = 0, count = 0, off = 0;  // off: the pixel's first list place, inside the region's places
    s.off[lane]   = 0u;
    s.carry[lane] = 0.f;
    s.point[lane] = 0;
    s.g[lane]     = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active)
    {
        const size_t plane   = (size_t)lw * lh;
        const uint32_t local = (uint32_t)y * (uint32_t)lw + (uint32_t)x;
        const float* G       = a.grad_out[l];
        float g[4]           = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ci = 0; ci < C; ++ci) g[ci] = G[ci * plane + local];
        const size_t q   = (size_t)region * rt.ppr + rt.first[l] + j;
        const uint2 info = a.pixel_info[q];
        if constexpr (HEAVY)
        {
            const uint2 hp = a.heavy_pixel[q];
            off            = hp.x;
            count          = hp.y;
        }
        else
        {
            off   = info.x & 0xFFFFu;
            count = info.x >> 16;
        }
        n = a.K > 0 ? min(count, (uint32_t)a.K) : count;
        float S        = 0.f;
        const float Tn = a.use_environment_map ? 0.f : __uint_as_float(info.y);
        if (!a.use_environment_map)
        {
            float dot = 0.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                const float bgc = a.background[ci];
                bg_grad[ci] += (Tn * 1.f) * g[ci];
                dot += bgc * g[ci];
                S += ((g[ci] * bgc) * Tn) * 1.f;
            }
            if (a.quirk_background_confidence_leak) leak += dot * Tn;
        }
        const bool inner    = interior_pixel(x, y, lw, lh);
        const bool do_point = a.need_point_gradient && n > 0 && inner;
        s.off[lane]   = off;
        s.carry[lane] = S;
        s.g[lane]     = make_float4(g[0], g[1], g[2], g[3]);
        s.point[lane] = do_point ? 1 : 0;
        if (do_point)
        {
            const float* I = a.out[l];
            float ax[4] = {0.f, 0.f, 0.f, 0.f}, ay[4] = {0.f, 0.f, 0.f, 0.f};
            float bx = 0.f, by = 0.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                const float* Ic = I + ci * plane + local;
                const float* Gc = G + ci * plane + local;
                const float Ix0 = Ic[-1], Ix1 = Ic[1], Iy0 = Ic[-lw], Iy1 = Ic[lw];
                const float Gx0 = Gc[-1], Gx1 = Gc[1], Gy0 = Gc[-lw], Gy1 = Gc[lw];
                ax[ci] = 0.5f * (Gx1 - Gx0);
                ay[ci] = 0.5f * (Gy1 - Gy0);
                bx += 0.5f * (Ix0 * Gx0 - Ix1 * Gx1);
                by += 0.5f * (Iy0 * Gy0 - Iy1 * Gy1);
            }
            s.ax[lane]  = make_float4(ax[0], ax[1], ax[2], ax[3]);
            s.ay[lane]  = make_float4(ay[0], ay[1], ay[2], ay[3]);
            s.bxy[lane] = make_float2(bx, by);
        }
    }
    float4* partial_l = a.partial + 2 * (size_t)l * a.N;

    uint32_t max_n = n;
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) max_n = max(max_n, (uint32_t)__shfl_xor((int)max_n, d, kWave));
    for (uint32_t top = (max_n + kWindow - 1) / kWindow * kWindow; top > 0;)
    {
        uint32_t width = kWindow;
        if (top >= 4u * kWindow && __popcll(__ballot(n + 4u * kWindow > top)) <= kWave / 4)
        {
            width = 4u * kWindow;
            if (top >= 16u * kWindow && __popcll(__ballot(n + 16u * kWindow > top)) <= kWave / 16) width = 16u * kWindow;
        }
        top -= width;
        const uint32_t jw    = top;
        const uint32_t nw    = (n > jw) ? min(n - jw, width) : 0u;
        const uint32_t incl  = wave_inclusive_scan(nw, lane);
        const uint32_t base  = incl - nw;
        const uint32_t total = __shfl(incl, kWave - 1, kWave);
        s.base[lane]         = base;
        for (uint32_t jj = 0; jj < nw; ++jj) s.item[base + jj] = (uint8_t)lane;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        for (int k0 = (int)((total - 1) / kWave) * kWave; total > 0 && k0 >= 0; k0 -= kWave)
        {
            const uint32_t k = (uint32_t)k0 + lane;
            const bool valid = k < total;
            const int p      = valid ? (int)s.item[k] : -1;
            float xsum = 0.f, T = 0.f, c = 0.f, dot = 0.f;
            float t[4] = {0.f, 0.f, 0.f, 0.f};
            float4 g4  = make_float4(0.f, 0.f, 0.f, 0.f);
            int target = -1;  // slot of the record, or the point id in a heavy region
            float4* row = nullptr;  // kRowsInMemory: the record's row
            bool give  = false;
            if (valid)
            {
                const size_t pos = list_base + s.off[p] + jw + (k - s.base[p]);
                T                = HEAVY ? a.heavy_T[pos] : a.list_T[pos];
                g4               = s.g[p];
                float4 t4;
                if constexpr (HEAVY)
                {
                    target = (int)(uint32_t)a.list_key[pos];
                    region_fetch_descriptor(a, target, t4, c);
                    give = (uint32_t)target < (uint32_t)a.N;
                }
                else
                {
                    target          = (int)a.list_slot[pos];
                    const uint4 ra  = room[2 * (size_t)target];
                    const uint4 rt4 = room[2 * (size_t)target + 1];
                    c               = __uint_as_float(ra.w);
                    t4 = make_float4(__uint_as_float(rt4.x), __uint_as_float(rt4.y), __uint_as_float(rt4.z), __uint_as_float(rt4.w));
                    give = true;
                    if constexpr (ROWS == kRowsInMemory)
                    {
                        const uint32_t id = ra.z & kRegionIdMask;
                        const int fl      = __ffs((int)(ra.z >> kRegionIdBits)) - 1;
                        give              = fl >= 0 && id < (uint32_t)a.N;  // guard: always true for records of the scatter pass
                        row               = a.partial + 2 * ((size_t)(give ? fl : 0) * a.N + (give ? id : 0u));
                    }
                }
                t[0] = t4.x, t[1] = t4.y, t[2] = t4.z, t[3] = t4.w;
                const float g[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
                for (int ci = 0; ci < C; ++ci)
                {
                    dot += t[ci] * g[ci];
                    xsum += ((g[ci] * t[ci]) * T) * c;
                }
            }
            const int pp         = __shfl_up(p, 1, kWave);
            const bool head      = lane == 0 || pp != p;
            const uint64_t heads = __ballot(head);
            const uint64_t above = lane == kWave - 1 ? 0ull : heads >> (lane + 1);
            const int last       = above != 0ull ? lane + __ffsll((unsigned long long)above) - 1 : kWave - 1;
            float v = xsum;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1)
            {
                const float o = __shfl_down(v, d, kWave);
                if (lane + d <= last) v += o;
            }
            const float vn = __shfl_down(v, 1, kWave);
            float S        = lane < last ? vn : 0.f;
            if (valid) S += s.carry[p];
            if (valid && head) s.carry[p] += v;
            if (give)
            {
                const float g[4]   = {g4.x, g4.y, g4.z, g4.w};
                const float Tc     = T * c;
                const float gconf  = dot * T - S / ((1.f - c) + 1e-9f);
                float gp0 = 0.f, gp1 = 0.f, cnt = 0.f;
                if (s.point[p] & 1)
                {
                    const float4 ax4 = s.ax[p], ay4 = s.ay[p];
                    const float2 b2  = s.bxy[p];
                    const float ax[4] = {ax4.x, ax4.y, ax4.z, ax4.w}, ay[4] = {ay4.x, ay4.y, ay4.z, ay4.w};
                    float dR_dpx = b2.x, dR_dpy = b2.y;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci)
                    {
                        dR_dpx += t[ci] * ax[ci];
                        dR_dpy += t[ci] * ay[ci];
                    }
                    // image-space gradient at the layer's resolution, brought to pixels of layer 0 (the crop transform
                    // of layer l is that of layer 0 times 0.5^l, src/lib/rendering/RenderBackward.cu:1381-1385; the
                    // factor is a power of two, so it commutes with the Jacobian chain the per-point kernel applies)
                    gp0 = (dR_dpx / (float)C) * layer_scale;
                    gp1 = (dR_dpy / (float)C) * layer_scale;
                    cnt = 1.f;
                }
                float gt[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ci = 0; ci < C; ++ci) gt[ci] = Tc * g[ci];
                if constexpr (HEAVY)
                {
                    partial_l[2 * (size_t)target]     = make_float4(gt[0], gt[1], gt[2], gt[3]);
                    partial_l[2 * (size_t)target + 1] = make_float4(gconf, gp0, gp1, cnt);
                }
                else if constexpr (ROWS == kRowsInMemory)
                {
                    const float4 lo = row[0], hi = row[1];
                    row[0]          = make_float4(lo.x + gt[0], lo.y + gt[1], lo.z + gt[2], lo.w + gt[3]);
                    row[1]          = make_float4(hi.x + gconf, hi.y + gp0, hi.z + gp1, hi.w + cnt);
                }
                else
                {
                    const float4 lo = s_lo[target];
                    s_lo[target]    = make_float4(lo.x + gt[0], lo.y + gt[1], lo.z + gt[2], lo.w + gt[3]);
                    s_hi[3 * target] += gconf;
                    s_hi[3 * target + 1] += gp0;
                    s_hi[3 * target + 2] += gp1;
                    if (cnt != 0.f) s_n[target] += 1;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
    if constexpr (HEAVY)
    {
        // fragments behind the cut: their rows are read by the per-point kernel like any other, so they are zeros
        uint64_t todo = __ballot(count > n);
        while (todo != 0ull)
        {
            const int src = __ffsll((unsigned long long)todo) - 1;
            todo &= todo - 1ull;
            const uint32_t o = (uint32_t)__shfl((int)off, src, kWave);
            const uint32_t c0 = (uint32_t)__shfl((int)n, src, kWave), c1 = (uint32_t)__shfl((int)count, src, kWave);
            for (uint32_t jj = c0 + lane; jj < c1; jj += kWave)
            {
                const uint32_t id = (uint32_t)a.list_key[list_base + o + jj];
                if (id < (uint32_t)a.N)
                {
                    partial_l[2 * (size_t)id]     = make_float4(0.f, 0.f, 0.f, 0.f);
                    partial_l[2 * (size_t)id + 1] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        }
    }
}

constexpr int kRegionAccRows = 256;  // records whose gradient rows a workgroup keeps in LDS

template <int C>
__global__ void __launch_bounds__(kBlock) region_backward_kernel(RegionBackwardPass a)
{
    constexpr int kWaves = kBlock / kWave;
    __shared__ RegionWaveShared s_wave[kWaves];
    __shared__ float4 s_lo[kRegionAccRows];     // per record: d descriptor
    __shared__ float s_hi[3 * kRegionAccRows];  // d confidence, d image x, d image y
    __shared__ uint8_t s_n[kRegionAccRows];     // fragments of the record that got a position gradient
    __shared__ float red[kWaves][C + 1];
    clear_small_accumulators(a.clear);
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const RegionTable& rt = a.rt;
    const uint32_t region = blockIdx.x;
    const uint32_t n_all  = (uint32_t)__builtin_amdgcn_readfirstlane((int)a.region_count[region]);
    if (region_plane(n_all) != blockIdx.y) return;
    const uint4* room = a.rooms + 2 * (size_t)region * kRegionRoom;
    // first list place of the region: its own stretch of list_slot / list_T, or what a heavy region drew from the cursor
    const size_t list_base = n_all > (uint32_t)kRegionRoom
                                 ? (size_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)a.region_info[region].x)
                                 : (size_t)region * a.list_places;
    float bg_grad[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) bg_grad[ci] = 0.f;
    float leak = 0.f;
    // The layers are taken one after the other, coarsest first, with a barrier in between: a record's row is added to
    // by one fragment at a time, in a fixed order.
    if (n_all <= (uint32_t)kRegionAccRows)
    {
        for (uint32_t r = tid; r < n_all; r += kBlock)
        {
            s_lo[r] = make_float4(0.f, 0.f, 0.f, 0.f);
            s_hi[3 * r] = s_hi[3 * r + 1] = s_hi[3 * r + 2] = 0.f;
            s_n[r] = 0;
        }
        __syncthreads();
        for (int l = rt.L - 1; l >= 0; --l)
        {
            region_backward_layer<C, kRowsInLds>(a, region, l, list_base, s_wave[wave], s_lo, s_hi, s_n, bg_grad, leak, lane, wave);
            __syncthreads();
        }
        // one row per record, at the place of the first layer the record covers
        for (uint32_t r = tid; r < n_all; r += kBlock)
        {
            const uint32_t idm = room[2 * (size_t)r].z;
            const uint32_t id  = idm & kRegionIdMask;
            const int fl       = __ffs((int)(idm >> kRegionIdBits)) - 1;
            if (fl < 0 || id >= (uint32_t)a.N) continue;  // guard: never true for records the scatter pass wrote
            float4* row = a.partial + 2 * ((size_t)fl * a.N + id);
            row[0]      = s_lo[r];
            row[1]      = make_float4(s_hi[3 * r], s_hi[3 * r + 1], s_hi[3 * r + 2], (float)s_n[r]);
        }
    }
    else if (n_all <= (uint32_t)kRegionRoom)
    {
        for (uint32_t r = tid; r < n_all; r += kBlock)
        {
            const uint32_t idm = room[2 * (size_t)r].z;
            const uint32_t id  = idm & kRegionIdMask;
            const int fl       = __ffs((int)(idm >> kRegionIdBits)) - 1;
            if (fl < 0 || id >= (uint32_t)a.N) continue;
            float4* row = a.partial + 2 * ((size_t)fl * a.N + id);
            row[0]      = make_float4(0.f, 0.f, 0.f, 0.f);
            row[1]      = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        __threadfence_block();
        __syncthreads();
        for (int l = rt.L - 1; l >= 0; --l)
        {
            region_backward_layer<C, kRowsInMemory>(a, region, l, list_base, s_wave[wave], s_lo, s_hi, s_n, bg_grad, leak, lane, wave);
            __threadfence_block();
            __syncthreads();
        }
    }
    else
    {
        for (int l = rt.L - 1; l >= 0; --l)
            region_backward_layer<C, kRowsPerLayer>(a, region, l, list_base, s_wave[wave], s_lo, s_hi, s_n, bg_grad, leak, lane, wave);
    }
#pragma unroll
    for (int ci = 0; ci < C; ++ci)
    {
        const float sum = wave_sum(bg_grad[ci]);
        if (lane == 0) red[wave][ci] = sum;
    }
    {
        const float sum = wave_sum(leak);
        if (lane == 0) red[wave][C] = sum;
    }
    __syncthreads();
    if (threadIdx.x <= C)
        a.background_partial[(size_t)blockIdx.x * kBackgroundRow + threadIdx.x] =
            (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

struct RegionGatherPass
{
    ViewPass vp;  // vp.ly is not used
    RegionTable rt;
    const uint32_t* region_count;
    const float4* partial;
    float* grad_texture;
    float* grad_confidence;
    float* grad_points;
    float* grad_point_count;
    double* camera_partial;
    int need_point_gradient;
    int accumulate;
    const float* background_rows;
    int num_background_rows;
    float* grad_background;
    int add_leak;
    int background_accumulate;
    const float* texture_raw;
    const float* background_raw;
    int texture_abs;
};

// One thread per point: the rows its records got from region_backward_kernel (one per region the point touches; one
// per layer where the region is a heavy one), summed in layer order, then the projection Jacobian chain of
// gather_point_gradients_kernel applied once to the summed image-space gradient (it is linear in it).
template <int C, bool DISTORT>
__global__ void __launch_bounds__(kBlock) region_gather_kernel(RegionGatherPass a)
{
    const int i      = blockIdx.x * blockDim.x + threadIdx.x;
    const bool alive = i < a.vp.N;
    float gt[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) gt[ci] = 0.f;
    float gc = 0.f, gx = 0.f, gy = 0.f, gz = 0.f, cnt = 0.f, sx = 0.f, sy = 0.f;
    bool hit = false;
    constexpr int kSums = DISTORT ? kCameraSums : 10;
    float cam_sum[kSums];
#pragma unroll
    for (int k = 0; k < kSums; ++k) cam_sum[k] = 0.f;
    Projected p;
    const DeviceView& cam = *a.vp.view;
    const RegionTable& rt = a.rt;
    const float4 wp       = alive ? a.vp.position[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    const float reach     = (float)(1 << (rt.L - 1)) + 1.f;
    if (alive && !point_is_skipped(a.vp, i) && project_point(cam, wp, p) && p.ipx >= -reach &&
        p.ipx <= (float)rt.w[0] + reach && p.ipy >= -reach && p.ipy <= (float)rt.h[0] + reach)
    {
        float ipx = p.ipx, ipy = p.ipy, radius = p.radius;
        uint32_t reg[VETRAST_MAX_LAYERS];
        uint32_t hits = 0;
        bool dropped  = false;
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
        {
            reg[l] = 0;
            if (l >= rt.L) continue;
            if (a.vp.drop_by_radius && radius < a.vp.radius_threshold) dropped = true;
            const float fx = rintf(ipx), fy = rintf(ipy);
            if (dropped || !(fx >= 0.f && fx < (float)rt.w[l] && fy >= 0.f && fy < (float)rt.h[l])) continue;
            const int sl = kRegionLog - l;
            reg[l]       = ((uint32_t)(int)fy >> sl) * rt.regions_x + ((uint32_t)(int)fx >> sl);
            hits |= 1u << l;
        }
        uint32_t heavy_layers = 0;  // layers whose region is a heavy one
#pragma unroll
        for (int l = 0; l < VETRAST_MAX_LAYERS; ++l)
        {
            if (!(hits & (1u << l))) continue;
            bool first = true, heavy = false;
#pragma unroll
            for (int k = 0; k < l; ++k)
                if ((hits & (1u << k)) && reg[k] == reg[l])
                {
                    first = false;
                    heavy = (heavy_layers >> k) & 1u;
                }
            if (first) heavy = a.region_count[reg[l]] > (uint32_t)kRegionRoom;
            if (heavy) heavy_layers |= 1u << l;
            if (!first && !heavy) continue;  // the row of the region's first layer holds this layer's part as well
            const size_t rec = (size_t)l * a.vp.N + i;
            const float4 r0  = a.partial[2 * rec];
            const float4 r1  = a.partial[2 * rec + 1];
            const float r[4] = {r0.x, r0.y, r0.z, r0.w};
#pragma unroll
            for (int ci = 0; ci < C; ++ci) gt[ci] += r[ci];
            gc += r1.x;
            sx += r1.y;
            sy += r1.z;
            cnt += r1.w;
            hit = true;
        }
        if (a.need_point_gradient && cnt > 0.f)
        {
            // ProjectPointPinholeBackward (src/lib/rendering/PointRendererHelper.h:317-372): crop rotation^T, crop K^T,
            // K^T, distortion^T, divide-by-z Jacobian^T, R^T, on the image-space gradient in pixels of layer 0
            const float vx = ((cam.r[0] * wp.x + cam.r[1] * wp.y) + cam.r[2] * wp.z) + cam.t[0];
            const float vy = ((cam.r[3] * wp.x + cam.r[4] * wp.y) + cam.r[5] * wp.z) + cam.t[1];
            const float vz = ((cam.r[6] * wp.x + cam.r[7] * wp.y) + cam.r[8] * wp.z) + cam.t[2];
            const float ar = cam.rot[0] * sx + cam.rot[2] * sy;
            const float br = cam.rot[1] * sx + cam.rot[3] * sy;
            const float a2 = cam.crop[0] * ar;
            const float b2 = cam.crop[4] * ar + cam.crop[1] * br;
            float d0 = cam.fx * a2;
            float d1 = cam.s * a2 + cam.fy * b2;
            float nx = vx / vz, ny = vy / vz;
            if constexpr (DISTORT)
            {
                float J[4], Jd[16], xd, yd;
                distort_point_jacobians(cam.dist, nx, ny, xd, yd, J, Jd);
#pragma unroll
                for (int k = 0; k < 8; ++k) cam_sum[10 + k] = Jd[2 * k] * d0 + Jd[2 * k + 1] * d1;
                const float n0 = J[0] * d0 + J[2] * d1, n1 = J[1] * d0 + J[3] * d1;
                d0 = n0, d1 = n1;
                nx = xd, ny = yd;
            }
            const float iz = 1.f / vz;
            const float e0 = iz * d0, e1 = iz * d1;
            const float e2 = (-vx * iz * iz) * d0 + (-vy * iz * iz) * d1;
            gx = (cam.r[0] * e0 + cam.r[3] * e1) + cam.r[6] * e2;
            gy = (cam.r[1] * e0 + cam.r[4] * e1) + cam.r[7] * e2;
            gz = (cam.r[2] * e0 + cam.r[5] * e1) + cam.r[8] * e2;
            if (a.camera_partial)
            {
                cam_sum[0] = e0;
                cam_sum[1] = e1;
                cam_sum[2] = e2;
                cam_sum[3] = vy * e2 - vz * e1;
                cam_sum[4] = vz * e0 - vx * e2;
                cam_sum[5] = vx * e1 - vy * e0;
                cam_sum[6] = nx * a2;
                cam_sum[7] = ny * b2;
                cam_sum[8] = a2;
                cam_sum[9] = b2;
            }
        }
    }
    if (a.camera_partial)
    {
        __shared__ double cam_red[kBlock / kWave][kCameraRow];
        const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
        for (int k = 0; k <= kCameraSums; ++k)
        {
            double v = (k < kSums) ? (double)cam_sum[k < kSums ? k : 0] : (k == kCameraSums ? (double)cnt : 0.0);
#pragma unroll
            for (int d = kWave / 2; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
            if (lane == 0) cam_red[wave][k] = v;
        }
        __syncthreads();
        if (threadIdx.x <= kCameraSums)
            a.camera_partial[(size_t)blockIdx.x * kCameraRow + threadIdx.x] =
                (cam_red[0][threadIdx.x] + cam_red[1][threadIdx.x]) + (cam_red[2][threadIdx.x] + cam_red[3][threadIdx.x]);
    }
    const int N = a.vp.N;
    if (alive && (a.vp.confidence_activation || a.texture_abs))
    {
        const int row = a.vp.index ? a.vp.index[i] : i;
        if ((uint32_t)row < (uint32_t)N)
        {
            if (a.vp.confidence_activation)
            {
                const float s = sigmoid_canon(a.vp.confidence_scale * a.vp.confidence[row]);
                gc            = gc * ((a.vp.confidence_scale * s) * (1.f - s));
            }
            if (a.texture_abs)
            {
#pragma unroll
                for (int ci = 0; ci < C; ++ci) gt[ci] = gt[ci] * sign_of(a.texture_raw[(size_t)ci * N + row]);
            }
        }
    }
    if (!alive)
    {
    }
    else if (a.vp.index)
    {
        const int ti = a.vp.index[i];
        if ((uint32_t)ti < (uint32_t)N)
        {
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
                if (gt[ci] != 0.f) atomicAdd(&a.grad_texture[(size_t)ci * N + ti], gt[ci]);
            if (gc != 0.f) atomicAdd(&a.grad_confidence[ti], gc);
        }
    }
    else if (a.accumulate)
    {
        if (hit)
        {
#pragma unroll
            for (int ci = 0; ci < C; ++ci) a.grad_texture[(size_t)ci * N + i] += gt[ci];
            a.grad_confidence[i] += gc;
        }
    }
    else
    {
#pragma unroll
        for (int ci = 0; ci < C; ++ci) a.grad_texture[(size_t)ci * N + i] = gt[ci];
        a.grad_confidence[i] = gc;
    }
    if (alive && a.grad_points)
    {
        float4* gp = reinterpret_cast<float4*>(a.grad_points) + i;
        if (a.accumulate)
        {
            if (cnt > 0.f)
            {
                const float4 o = *gp;
                *gp            = make_float4(o.x + gx, o.y + gy, o.z + gz, 0.f);
                a.grad_point_count[i] += cnt;
            }
        }
        else
        {
            *gp                   = make_float4(gx, gy, gz, 0.f);
            a.grad_point_count[i] = cnt;
        }
    }
    if (blockIdx.x == 0)
    {
        __syncthreads();
        float leak_factor = 1.f;
        if (a.vp.confidence_activation && a.add_leak)
        {
            const float s0 = sigmoid_canon(a.vp.confidence_scale * a.vp.confidence[0]);
            leak_factor    = (a.vp.confidence_scale * s0) * (1.f - s0);
        }
        sum_background_rows<kBlock>(a.background_rows, a.num_background_rows, C, a.grad_background, a.grad_confidence,
                                    a.add_leak, a.background_accumulate, a.vp.index != nullptr,
                                    a.texture_abs ? a.background_raw : nullptr, leak_factor);
    }
}

}  // namespace vetrast
