// Error lifting: the per-pixel error of one rendered view is added to every cell of the scene grid whose projected box
// covers the pixel (FillSceneGridWithLossRasterize, src/lib/rendering/RenderForward.cu:639-761).
//
// The reference gives every cell one 32-lane warp, whatever the size of the cell on screen. Here a wave64 owns a cell
// whose pixel box holds at most kLiftWaveLimit pixels and finishes it without atomics; larger boxes (cells close to the
// camera can cover the whole image) are queued and cut into chunks of kLiftChunk pixels that the workgroups of a second
// launch share, so no wave runs much longer than the others.
#pragma once
#include "common.h"
#include "forward_kernels.h"

namespace vetrast
{
constexpr int kLiftWaveLimit = 4096;  // pixels a single wave rasterizes by itself: 64 rounds
constexpr int kLiftChunk     = 4096;  // pixels per workgroup step of the shared path: 16 per thread
constexpr int kLiftHeader    = 256;   // bytes in front of the queue: DeviceView (160), queue length at 176, flag word at 192
static_assert(sizeof(DeviceView) <= VETRAST_LIFT_QUEUE_LENGTH_OFFSET && VETRAST_LIFT_QUEUE_LENGTH_OFFSET + 4 <= VETRAST_LIFT_FLAGS_OFFSET,
              "the header's three parts must not overlap");

struct LiftPass
{
    const float* bb_min;
    const float* bb_length;
    float* value;
    int32_t* access_count;
    const float* loss;  // [channels][height][width]
    int64_t num_cells;
    int channels, height, width, border;
    // workspace
    const DeviceView* view;
    uint32_t* queue_length;
    uint2* queue;   // {cell, pixels of its box}
    double* sums;   // per queue slot
    unsigned long long* starts;  // per queue slot: chunks in front of it; [length] = all chunks
};

// One thread: the camera constants of the view, and an empty queue.
__global__ void lift_prepare_kernel(ViewSource src, const double* __restrict__ poses_se3,
                                    const float* __restrict__ intrinsics, DeviceView* __restrict__ view,
                                    uint32_t* __restrict__ queue_length, uint32_t* __restrict__ flags)
{
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    bool distorted = false;
    *view          = make_device_view(src, poses_se3, intrinsics, distorted);
    view->has_dist = 0u;  // cameras with distortion are refused here (the flag below)
    *queue_length  = 0u;
    *flags         = distorted ? 1u : 0u;
}

// Screen footprint of a cell, identical in every lane of the wave that computed it.
struct CellFootprint
{
    float px[8], py[8];  // projected corners
    float min_x, min_y;  // clamped pixel box origin
    int x_size, y_size;
    uint32_t first_faces;  // bit f: face f (triangles 2f, 2f+1) is tested in the first round
};

// tris_indices of the reference (src/lib/rendering/RenderForward.cu:665-666): two triangles per face of the box.
constexpr int kLiftTriangles[12][3] = {{0, 1, 4}, {0, 4, 2}, {1, 5, 7}, {1, 7, 4}, {5, 3, 6}, {5, 6, 7},
                                       {3, 0, 6}, {0, 6, 2}, {3, 0, 5}, {0, 5, 1}, {2, 4, 6}, {4, 6, 7}};

// sign() and PointInTriangle() of src/lib/rendering/RenderForward.cu:605-625.
__device__ __forceinline__ float edge_sign(float p1x, float p1y, float p2x, float p2y, float p3x, float p3y)
{
    return (p1x - p3x) * (p2y - p3y) - (p2x - p3x) * (p1y - p3y);
}

__device__ __forceinline__ bool point_in_triangle(float x, float y, float ax, float ay, float bx, float by, float cx,
                                                  float cy)
{
    const float d1     = edge_sign(x, y, ax, ay, bx, by);
    const float d2     = edge_sign(x, y, bx, by, cx, cy);
    const float d3     = edge_sign(x, y, cx, cy, ax, ay);
    // has_neg = one of them < 0, has_pos = one of them > 0; fminf / fmaxf drop a NaN like the comparisons do
    const bool has_neg = fminf(fminf(d1, d2), d3) < 0.f;
    const bool has_pos = fmaxf(fmaxf(d1, d2), d3) > 0.f;
    return !(has_neg && has_pos);
}

// Lanes 0..7 of the calling wave project one corner each (src/lib/rendering/RenderForward.cu:679-704); the pixel box of
// the projections is cut to the image minus the border (:706-728). False when the cell does not take part: a corner at
// or behind the camera plane, or a box outside the bordered image. All 64 lanes must call.
__device__ __forceinline__ bool cell_footprint(const LiftPass& a, const DeviceView& view, int64_t cell, int lane,
                                               CellFootprint& f)
{
    float ipx = 0.f, ipy = 0.f;
    bool behind = false;
    if (lane < 8)
    {
        // corner order of bb_facs: 000 100 010 001 110 101 011 111
        const int fx = (0xB2 >> lane) & 1, fy = (0xD4 >> lane) & 1, fz = (0xE8 >> lane) & 1;
        const float* mn = a.bb_min + 3 * cell;
        const float* ln = a.bb_length + 3 * cell;
        float4 p;
        p.x = mn[0] + ln[0] * (float)fx;
        p.y = mn[1] + ln[1] * (float)fy;
        p.z = mn[2] + ln[2] * (float)fz;
        p.w = 0.f;
        Projected o;
        behind = !project_point(view, p, o);
        ipx    = behind ? 0.f : o.ipx;
        ipy    = behind ? 0.f : o.ipy;
    }
    if (__ballot(behind) != 0ull) return false;
    float max_x = -10000000.f, max_y = -10000000.f, min_x = 10000000.f, min_y = 10000000.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        f.px[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ipx), i));
        f.py[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ipy), i));
        max_x   = fmaxf(f.px[i], max_x);
        max_y   = fmaxf(f.py[i], max_y);
        min_x   = fminf(f.px[i], min_x);
        min_y   = fminf(f.py[i], min_y);
    }
    const float border = (float)a.border;
    const float right  = (float)(a.width - a.border);
    const float bottom = (float)(a.height - a.border);
    if (max_x < border || min_x >= right || max_y < border || min_y >= bottom) return false;
    min_x    = fmaxf(min_x, border);
    min_y    = fmaxf(min_y, border);
    max_x    = fminf(max_x, right);
    max_y    = fminf(max_y, bottom);
    f.min_x  = min_x;
    f.min_y  = min_y;
    f.y_size = (int)(max_y - min_y);
    f.x_size = (int)(max_x - min_x);
    // The faces that wind one way on screen cover the whole projection of the box by themselves (they are its near or
    // its far side). Testing them first lets a wave whose pixels all lie inside stop after half of the triangles; the
    // result does not depend on the order, every pixel still gets the "inside any of the 12" answer.
    uint32_t faces = 0u;
#pragma unroll
    for (int face = 0; face < 6; ++face)
    {
        const int i = kLiftTriangles[2 * face][0], j = kLiftTriangles[2 * face][1], k = kLiftTriangles[2 * face][2];
        if (edge_sign(f.px[i], f.py[i], f.px[j], f.py[j], f.px[k], f.py[k]) > 0.f) faces |= 1u << face;
    }
    f.first_faces = (uint32_t)__builtin_amdgcn_readfirstlane((int)faces);  // the same in every lane: keep it scalar
    return true;
}

// Pixel number xy of the box -> is it covered, and what does it add (src/lib/rendering/RenderForward.cu:731-759).
// 0 <= xy < x_size * y_size < 2^24, so the float quotient is off by at most one and one correction step fixes it.
__device__ __forceinline__ void lift_pixel(const LiftPass& a, const CellFootprint& f, float inv_x_size, int xy,
                                           double& sum, int& count)
{
    int row = (int)((float)xy * inv_x_size);
    int col = xy - row * f.x_size;
    if (col < 0) col += f.x_size, row -= 1;
    if (col >= f.x_size) col -= f.x_size, row += 1;
    const int x_c = (int)((float)col + f.min_x);
    const int y_c = (int)((float)row + f.min_y);
    const float x = (float)x_c, y = (float)y_c;
    bool inside = false;
#pragma unroll
    for (int round = 0; round < 2; ++round)
    {
#pragma unroll
        for (int face = 0; face < 6; ++face)
        {
            if ((((f.first_faces >> face) & 1u) != 0u) != (round == 0)) continue;  // uniform over the wave
#pragma unroll
            for (int t = 2 * face; t < 2 * face + 2; ++t)
                inside |= point_in_triangle(x, y, f.px[kLiftTriangles[t][0]], f.py[kLiftTriangles[t][0]],
                                            f.px[kLiftTriangles[t][1]], f.py[kLiftTriangles[t][1]],
                                            f.px[kLiftTriangles[t][2]], f.py[kLiftTriangles[t][2]]);
        }
        // every lane still in the loop is inside: the other faces cannot change that
        if (round == 0 && __ballot(!inside) == 0ull) break;
    }
    if (!inside) return;
    // the box lies inside the bordered image by construction; the guard keeps a negative border from reading outside
    if (x_c < 0 || x_c >= a.width || y_c < 0 || y_c >= a.height) return;
    float grad = 0.f;
    const size_t plane = (size_t)a.height * a.width;
    const float* px    = a.loss + (size_t)y_c * a.width + x_c;
    for (int c = 0; c < a.channels; ++c) grad += fabsf(px[c * plane]);
    sum += (double)grad;
    count += 1;
}

__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}

__device__ __forceinline__ int wave_sum(int v)
{
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}

// One wave per cell. Small boxes are finished here; large ones go to the queue.
__global__ void __launch_bounds__(kBlock) lift_cells_kernel(LiftPass a)
{
    const int lane     = threadIdx.x & (kWave - 1);
    const int64_t cell = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
    if (cell >= a.num_cells) return;  // whole waves leave together
    const DeviceView view = *a.view;
    CellFootprint f;
    if (!cell_footprint(a, view, cell, lane, f)) return;
    const int pixels = f.x_size * f.y_size;
    if (pixels <= 0) return;
    if (pixels > kLiftWaveLimit)
    {
        if (lane == 0)
        {
            const uint32_t slot = atomicAdd(a.queue_length, 1u);
            a.queue[slot]       = make_uint2((uint32_t)cell, (uint32_t)pixels);
            a.sums[slot]        = 0.0;
        }
        return;
    }
    const float inv_x_size = 1.0f / (float)f.x_size;
    double sum             = 0.0;
    int count              = 0;
    for (int xy = lane; xy < pixels; xy += kWave) lift_pixel(a, f, inv_x_size, xy, sum, count);
    sum   = wave_sum(sum);
    count = wave_sum(count);
    if (lane == 0 && count > 0)
    {
        a.value[cell]        = (float)((double)a.value[cell] + sum);
        a.access_count[cell] = a.access_count[cell] + count;
    }
}

// Queued cells: exclusive prefix sum of their chunk counts, starts[slot], with the total in starts[length]. One
// workgroup; the queue rarely holds more than a few thousand cells.
constexpr int kLiftScanBlock = 1024;
__global__ void __launch_bounds__(kLiftScanBlock) lift_scan_kernel(LiftPass a)
{
    __shared__ unsigned long long s_wave[kLiftScanBlock / kWave];
    __shared__ unsigned long long s_carry;
    const uint32_t length = *a.queue_length;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_carry = 0ull;
    __syncthreads();
    for (uint32_t base = 0; base < length; base += kLiftScanBlock)
    {
        const uint32_t i             = base + threadIdx.x;
        const unsigned long long own = i < length ? (a.queue[i].y + kLiftChunk - 1) / kLiftChunk : 0ull;
        unsigned long long incl      = own;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1)
        {
            const unsigned long long up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == kWave - 1) s_wave[wave] = incl;
        __syncthreads();
        unsigned long long before = s_carry;
        for (int w = 0; w < wave; ++w) before += s_wave[w];
        if (i < length) a.starts[i] = before + incl - own;
        __syncthreads();
        if (threadIdx.x == kLiftScanBlock - 1) s_carry = before + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) a.starts[length] = s_carry;
}

// Queued cells: all their chunks, numbered through the queue, are split into equal contiguous runs, one per workgroup.
// A workgroup finds the cell its run starts in by bisection of starts[], then walks on cell by cell; every quantity
// that steers the loops is the same in all of its threads.
__global__ void __launch_bounds__(kBlock) lift_queued_kernel(LiftPass a)
{
    __shared__ double s_sum[kBlock / kWave];
    __shared__ int s_count[kBlock / kWave];
    const int lane        = threadIdx.x & (kWave - 1);
    const int wave        = threadIdx.x >> 6;
    const uint32_t length = *a.queue_length;
    if (length == 0) return;
    const unsigned long long total = a.starts[length];
    const unsigned long long per   = (total + gridDim.x - 1) / gridDim.x;
    unsigned long long g           = min(total, per * blockIdx.x);
    const unsigned long long g_end = min(total, g + per);
    if (g >= g_end) return;
    uint32_t lo = 0, hi = length;  // starts[lo] <= g < starts[hi]
    while (hi - lo > 1)
    {
        const uint32_t mid = (lo + hi) / 2;
        if (a.starts[mid] <= g)
            lo = mid;
        else
            hi = mid;
    }
    const DeviceView view = *a.view;
    for (uint32_t slot = lo; g < g_end; ++slot)
    {
        const uint2 entry                = a.queue[slot];
        const unsigned long long first   = a.starts[slot];
        const unsigned long long cell_end = min(g_end, a.starts[slot + 1]);
        CellFootprint f;
        const bool ok          = cell_footprint(a, view, (int64_t)entry.x, lane, f);
        const int pixels       = ok ? f.x_size * f.y_size : 0;  // a queued cell always has a footprint
        const float inv_x_size = 1.0f / (float)(ok ? f.x_size : 1);
        double sum             = 0.0;
        int count              = 0;
        for (; g < cell_end; ++g)
        {
            const int begin = (int)(g - first) * kLiftChunk;
            const int end   = min(begin + kLiftChunk, pixels);
            for (int xy = begin + (int)threadIdx.x; xy < end; xy += kBlock) lift_pixel(a, f, inv_x_size, xy, sum, count);
        }
        sum   = wave_sum(sum);
        count = wave_sum(count);
        __syncthreads();  // the previous cell's readers are done
        if (lane == 0) s_sum[wave] = sum, s_count[wave] = count;
        __syncthreads();
        if (threadIdx.x == 0)
        {
            double cell_sum = 0.0;
            int n           = 0;
            for (int w = 0; w < kBlock / kWave; ++w) cell_sum += s_sum[w], n += s_count[w];
            if (n > 0)
            {
                atomicAdd(&a.sums[slot], cell_sum);
                atomicAdd(&a.access_count[entry.x], n);
            }
        }
    }
}

// Queued cells: the double sums go into cell_value with one rounding.
__global__ void __launch_bounds__(kBlock) lift_finish_kernel(LiftPass a)
{
    const uint32_t length = *a.queue_length;
    for (uint32_t slot = blockIdx.x * blockDim.x + threadIdx.x; slot < length; slot += gridDim.x * blockDim.x)
    {
        const uint32_t cell = a.queue[slot].x;
        a.value[cell]       = (float)((double)a.value[cell] + a.sums[slot]);
    }
}

}  // namespace vetrast
