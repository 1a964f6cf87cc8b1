// Backward kernels: gradients of the blend with respect to descriptors, confidence, background and point positions.
//
// A point lands in exactly one pixel per layer, so a fragment is identified by (layer, point id). The per-pixel kernel
// therefore STORES each kept fragment's gradient contribution as one 32-byte record at partial[layer][point] instead
// of adding it to the gradient tensors with global atomics, and a per-point kernel sums a point's (at most L) records
// in a fixed order and writes the gradient tensors with plain coalesced stores. Device-scope float atomics, which the
// reference issues per fragment and channel (src/lib/rendering/RenderBackward.cu:1152,1157,1177,1405-1407), were the
// single largest cost on MI355X; without them the gradients are also reproducible run to run.
#pragma once
#include <type_traits>

#include "common.h"

namespace vetrast
{
// Small accumulators of the call (pose and intrinsics gradients and their counts) that have to start at zero: the first
// workgroup of the first view's per-pixel kernel clears them, which is in front of every kernel that adds to them in
// stream order and saves the launches of a fill kernel each.
struct ClearJob
{
    uint32_t* ptr[4];
    uint32_t count[4];  // 32-bit words; 0 = nothing to clear
};
__device__ __forceinline__ void clear_small_accumulators(const ClearJob& job)
{
    if (blockIdx.x != 0 || blockIdx.y != 0) return;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        for (uint32_t i = threadIdx.x; i < job.count[k]; i += blockDim.x) job.ptr[k][i] = 0u;
}

struct BackwardPass
{
    const uint32_t* offsets;
    const uint32_t* kept;        // per pixel, BILINEAR_BLEND: fragments of its list that took part in the forward blend
    const uint64_t* fragments;
    const float* transmittance;  // per blended fragment, saved by the forward blend
    const float* weight;         // per pixel: transmittance behind the last blended fragment
    const float2* projected;     // BILINEAR_BLEND: [N] where a point projects to at layer 0 (a fragment's alpha and its
                                 // derivative depend on it); written by the forward pass
    const int32_t* index;
    const float4* packed;
    const float* background;
    const float* grad_out[VETRAST_MAX_LAYERS];  // already offset to this view
    const float* out[VETRAST_MAX_LAYERS];       // forward result, already offset to this view
    float4* partial;          // records of 2 float4: (d tex0..3), (d conf, d image x, d image y, 0), at gradient_record
    int point_major_records;  // layout of the record array, see gradient_record
    float* background_partial;  // [workgroups][8]: per-workgroup sums of d background[0..C) and of the leak term
    LayerTable ly;
    TileMap tiles;
    int N;
    int K;
    int use_environment_map;
    int need_point_gradient;
    int quirk_background_confidence_leak;
    ClearJob clear;
};

// Sum over the 64 lanes (xor butterfly, widest step first); every lane gets the total. The four steps inside a row of
// 16 lanes are DPP moves, only the two widest go through the LDS crossbar.
__device__ __forceinline__ float wave_sum(float v)
{
    const int lane = threadIdx.x & (kWave - 1);
    v += __uint_as_float(lane_xor<32>(__float_as_uint(v), lane));
    v += __uint_as_float(lane_xor<16>(__float_as_uint(v), lane));
    v += __uint_as_float(lane_xor<8>(__float_as_uint(v), lane));
    v += __uint_as_float(lane_xor<4>(__float_as_uint(v), lane));
    v += __uint_as_float(lane_xor<2>(__float_as_uint(v), lane));
    v += __uint_as_float(lane_xor<1>(__float_as_uint(v), lane));
    return v;
}

// Pixels closer than 3 to the border get no position gradient: distanceFromEdge(y, x) > 2,
// src/lib/rendering/RenderBackward.cu:1187.
__device__ __forceinline__ bool interior_pixel(int x, int y, int w, int h)
{
    return min(min(x, y), min(w - 1 - x, h - 1 - y)) > 2;
}

// Per-pixel part of the backward pass; all layers of a view in one launch. Counterpart of BlendBackwards2<C>
// (src/lib/rendering/RenderBackward.cu:1083-1513).
//
// Arithmetic. With the transmittance T_j the forward pass stored, the reference's inner loop over all fragments in
// front (src/lib/rendering/RenderBackward.cu:1160-1178, n(n-1)/2 atomics per pixel) is a suffix sum:
//   S_j         = sum_{i>j} sum_ci g[ci] * t_i[ci] * T_i * c_i          (the background counts as the last fragment)
//   d conf_j    = T_j * (t_j . g)  -  S_j / (1 - c_j + 1e-9)
//   d tex_j[ci] = T_j * c_j * g[ci]
// i.e. the same terms added in a different order. The position term is the neighbour-difference heuristic of
// src/lib/rendering/RenderBackward.cu:1346-1377, stored as an image-space gradient; the per-point kernel applies the
// projection Jacobian.
//
// Work distribution. A wave owns 16x4 pixels, but at the fine layers most pixels hold no or one fragment while a few
// hold several, so one-thread-per-pixel loops leave most lanes idle. Instead the wave lays the kept fragments of its
// 64 pixels out as one dense item list (in windows of 16 fragments per pixel), and every lane processes one FRAGMENT:
// per-pixel data (upstream gradient, neighbour samples) is staged in LDS, the suffix sum is a segmented scan over the
// lanes of a pixel plus a per-pixel carry, rounds run from the deepest fragments to the nearest.
constexpr int kWindow     = 16;                 // fragments per pixel in one window
constexpr int kWaveItems  = kWave * kWindow;    // item table of a wave

//
// BILINEAR_BLEND (BlendBackwardsBilinear<C>, src/lib/rendering/RenderBackward.cu:2893-3232) has the same structure with
// alpha_j = bilinear weight_j * confidence_j in place of c_j: d alpha_j = T_j * (t_j . g) - S_j / (1 - alpha_j + 1e-9),
// the background only counts if the forward blend reached it (transmittance still >= 0.001), and, at pixels more than
// 2 away from the border only, d conf_j = weight_j * d alpha_j and the position gradient is the analytic
// d weight_j / d position * confidence_j * d alpha_j. A record goes to partial[layer][corner][point].
template <int C, bool BILINEAR>
__device__ __forceinline__ void blend_backward(const BackwardPass& a)
{
    constexpr int kWaves = kBlock / kWave;
    __shared__ uint32_t s_off[kWaves][kWave];
    __shared__ uint32_t s_base[kWaves][kWave];
    __shared__ float s_carry[kWaves][kWave];
    __shared__ float4 s_g[kWaves][kWave];
    // position heuristic of a pixel as coefficients: d image x = (t . ax + bx) / C, d image y = (t . ay + by) / C
    __shared__ float4 s_ax[kWaves][kWave];
    __shared__ float4 s_ay[kWaves][kWave];
    __shared__ float2 s_bxy[kWaves][kWave];
    __shared__ uint8_t s_point[kWaves][kWave];
    __shared__ uint8_t s_item[kWaves][kWaveItems];
    __shared__ float red[kWaves][C + 1];

    clear_small_accumulators(a.clear);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const TilePixel px = tile_pixel(a.tiles, a.ly);
    const int l        = px.l;
    float bg_grad[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) bg_grad[ci] = 0.f;
    float leak = 0.f;
    uint32_t off = 0, n = 0;

    if (px.active)
    {
        const int lw = a.ly.w[l], lh = a.ly.h[l];
        const size_t plane   = (size_t)lw * lh;
        const uint32_t local = px.local;
        const float* G       = a.grad_out[l];
        float g[4]           = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ci = 0; ci < C; ++ci) g[ci] = G[ci * plane + local];
        off = a.offsets[px.q];
        if constexpr (BILINEAR)
            n = a.kept[px.q];
        else
        {
            n = a.offsets[px.q + 1] - off;
            if (a.K > 0) n = min(n, (uint32_t)a.K);
        }

        float S = 0.f;
        const float Tn = a.use_environment_map ? 0.f : a.weight[px.q];
        // BILINEAR_BLEND leaves the background out once the transmittance is below 0.001 (RenderBackward.cu:3014-3019:
        // the loop stops before the background element)
        if (!a.use_environment_map && !(BILINEAR && (double)Tn < 0.001))
        {
            float dot      = 0.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                const float bgc = a.background[ci];
                bg_grad[ci]     = (Tn * 1.f) * g[ci];
                dot += bgc * g[ci];
                S += ((g[ci] * bgc) * Tn) * 1.f;
            }
            if (!BILINEAR && a.quirk_background_confidence_leak) leak = dot * Tn;
        }
        const bool inner    = interior_pixel(px.x, px.y, lw, lh);
        const bool do_point = a.need_point_gradient && n > 0 && inner;
        s_off[wave][lane]   = off;
        s_carry[wave][lane] = S;
        s_g[wave][lane]     = make_float4(g[0], g[1], g[2], g[3]);
        s_point[wave][lane] = (do_point ? 1 : 0) | (inner ? 2 : 0);
        if (do_point && !BILINEAR)
        {
            // The reference evaluates, per fragment with descriptor t and per channel,
            //   1/2 * ( -(t - I(x-1)) * G(x-1) + (t - I(x+1)) * G(x+1) )        (RenderBackward.cu:1364-1371)
            // and the same in y. That is linear in t: t * 1/2 (G(x+1) - G(x-1)) + 1/2 (I(x-1) G(x-1) - I(x+1) G(x+1)),
            // so the neighbour samples are folded once per pixel into C slopes and one offset per axis.
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
            s_ax[wave][lane]  = make_float4(ax[0], ax[1], ax[2], ax[3]);
            s_ay[wave][lane]  = make_float4(ay[0], ay[1], ay[2], ay[3]);
            s_bxy[wave][lane] = make_float2(bx, by);
        }
    }

    // ---- fragments: windows of kWindow per pixel, deepest window first ------------------------------------------
    uint32_t max_n = n;
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) max_n = max(max_n, (uint32_t)__shfl_xor((int)max_n, d, kWave));
    float4* partial_l = a.partial;  // (records are addressed by gradient_record)
    // Windows run from the deepest list places to the nearest. Where only a few pixels of the wave still have fragments
    // that deep (uncut lists of hundreds of fragments at a handful of pixels), a window of 16 places would fill a
    // quarter of the lanes or less and every window costs a dependent chain of memory round trips, so the window is
    // widened to 64 places (at most 16 pixels reach into it) or 256 places (at most 4): the item table never holds
    // more than kWaveItems entries.
    for (uint32_t top = (max_n + kWindow - 1) / kWindow * kWindow; top > 0;)
    {
        uint32_t width = kWindow;
        if (top >= 4u * kWindow && __popcll(__ballot(n + 4u * kWindow > top)) <= kWave / 4)
        {
            width = 4u * kWindow;
            if (top >= 16u * kWindow && __popcll(__ballot(n + 16u * kWindow > top)) <= kWave / 16) width = 16u * kWindow;
        }
        top -= width;
        const uint32_t jw = top;
        const uint32_t nw = (n > jw) ? min(n - jw, width) : 0u;
        const uint32_t incl = wave_inclusive_scan(nw, lane);
        const uint32_t base  = incl - nw;
        const uint32_t total = __shfl(incl, kWave - 1, kWave);
        s_base[wave][lane]   = base;
        for (uint32_t j = 0; j < nw; ++j) s_item[wave][base + j] = (uint8_t)lane;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // BILINEAR_BLEND asks for the key and the transmittance of a step's fragments one step ahead: they only depend
        // on the item table, and the step's own chain (key -> descriptor record and position -> arithmetic -> store)
        // is then one memory round trip shorter (per-pixel backward kernel of a 1080p frame 247 -> 237 us). With one
        // fragment per point and layer it gains nothing at one view and costs 4 % at four (measured), so there the
        // step asks for its own.
        int p_next = -1;
        uint32_t low_next = 0;
        float T_next      = 0.f;
        auto fetch = [&](int k0) {
            const uint32_t k = (uint32_t)k0 + lane;
            p_next           = k < total ? (int)s_item[wave][k] : -1;  // lane of the pixel this fragment belongs to
            if (p_next >= 0)
            {
                const uint32_t pos = s_off[wave][p_next] + jw + (k - s_base[wave][p_next]);
                low_next           = (uint32_t)a.fragments[pos];
                T_next             = a.transmittance[pos];
            }
        };
        const int k_first = total > 0 ? (int)((total - 1) / kWave) * kWave : -1;
        if (BILINEAR && k_first >= 0) fetch(k_first);
        for (int k0 = k_first; k0 >= 0; k0 -= kWave)
        {
            if constexpr (!BILINEAR) fetch(k0);
            const int p        = p_next;
            const bool valid   = p >= 0;
            const uint32_t low = low_next;
            float x = 0.f, T = T_next, c = 0.f, dot = 0.f;
            if (BILINEAR && k0 >= kWave) fetch(k0 - kWave);
            float t[4] = {0.f, 0.f, 0.f, 0.f};
            float4 g4  = make_float4(0.f, 0.f, 0.f, 0.f);
            int id = -1, ti = -1, corner = 0;
            if (valid)
            {
                id                 = BILINEAR ? (int)(low >> 2) : (int)low;
                corner             = BILINEAR ? (int)(low & 3u) : 0;
                // guards the gathers; never false for a workspace the forward pass wrote
                if ((uint32_t)id < (uint32_t)a.N) ti = a.index ? a.index[id] : id;
                if ((uint32_t)ti >= (uint32_t)a.N) ti = -1;
                g4 = s_g[wave][p];
            }
            float conf = 0.f, fac = 1.f, fac_du = 0.f, fac_dv = 0.f;
            if (ti >= 0)
            {
                const float4 t4 = a.packed[2 * (size_t)ti];
                conf            = a.packed[2 * (size_t)ti + 1].x;
                c               = conf;
                if constexpr (BILINEAR)
                {
                    // alpha = bilinear weight of this pixel's corner at the point's position in this layer x confidence;
                    // the position is the one the scatter pass stored for the forward blend
                    const float2 ip = a.projected[id];
                    float u = ip.x, v = ip.y;
                    for (int h = 0; h < l; ++h) u *= 0.5f, v *= 0.5f;
                    fac = bilinear_weight(u, v, corner, &fac_du, &fac_dv);
                    c = fac * conf;
                }
                t[0] = t4.x, t[1] = t4.y, t[2] = t4.z, t[3] = t4.w;
                const float g[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
                for (int ci = 0; ci < C; ++ci)
                {
                    dot += t[ci] * g[ci];
                    x += ((g[ci] * t[ci]) * T) * c;
                }
            }
            // suffix sum over the fragments of the same pixel that sit in higher lanes of this step. The fragments of a
            // pixel are neighbouring lanes: `last` is the end of this lane's run, found from the mask of run starts, so
            // that the scan steps only have to move the sums.
            const int pp         = __shfl_up(p, 1, kWave);
            const bool head      = lane == 0 || pp != p;
            const uint64_t heads = __ballot(head);
            const uint64_t above = lane == kWave - 1 ? 0ull : heads >> (lane + 1);
            const int last       = above != 0ull ? lane + __ffsll((unsigned long long)above) - 1 : kWave - 1;
            float v = x;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1)
            {
                const float o = __shfl_down(v, d, kWave);
                if (lane + d <= last) v += o;
            }
            const float vn = __shfl_down(v, 1, kWave);
            float S        = lane < last ? vn : 0.f;                     // deeper fragments of this step
            if (valid) S += s_carry[wave][p];                            // and of the steps / windows before
            if (valid && head) s_carry[wave][p] += v;                    // one lane per pixel moves the carry on
            float4 rec_lo = make_float4(0.f, 0.f, 0.f, 0.f), rec_hi = rec_lo;
            if (ti >= 0)
            {
                const float g[4]  = {g4.x, g4.y, g4.z, g4.w};
                const float Tc     = T * c;
                const float galpha = dot * T - S / ((1.f - c) + 1e-9f);
                float gconf        = galpha;
                float gp0 = 0.f, gp1 = 0.f;
                if constexpr (BILINEAR)
                {
                    // confidence and position gradients only at pixels more than 2 away from the border
                    // (RenderBackward.cu:3044); dA/dc = weight, dA/dweight = confidence (:3075-3088)
                    const int flags = s_point[wave][p];
                    gconf           = (flags & 2) ? fac * galpha : 0.f;
                    if (flags & 1)
                    {
                        const float single = conf * galpha;
                        gp0                = fac_du * single;
                        gp1                = fac_dv * single;
                    }
                }
                else if (s_point[wave][p] & 1)
                {
                    const float4 ax4 = s_ax[wave][p], ay4 = s_ay[wave][p];
                    const float2 b2  = s_bxy[wave][p];
                    const float ax[4] = {ax4.x, ax4.y, ax4.z, ax4.w}, ay[4] = {ay4.x, ay4.y, ay4.z, ay4.w};
                    float dR_dpx = b2.x, dR_dpy = b2.y;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci)
                    {
                        dR_dpx += t[ci] * ax[ci];
                        dR_dpy += t[ci] * ay[ci];
                    }
                    gp0 = dR_dpx / (float)C;  // image-space gradient of this fragment at the layer's resolution;
                    gp1 = dR_dpy / (float)C;  // the per-point kernel pushes it through the projection Jacobian
                }
                float gt[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ci = 0; ci < C; ++ci) gt[ci] = Tc * g[ci];
                rec_lo = make_float4(gt[0], gt[1], gt[2], gt[3]);
                rec_hi = make_float4(gconf, gp0, gp1, 0.f);
            }
            {
                // Record stores, two lanes per record: first the even lane's record (even lane its low half, odd lane
                // the high half), then the odd lane's, so that each instruction issues one 32-byte request per record.
                const int odd        = lane & 1;
                const int own        = ti >= 0 ? (int)gradient_record(a.point_major_records, a.N, a.ly.L, BILINEAR ? 4 : 1, l, corner, id) : -1;
                const int other      = pair_other(own);
                const float4 o_lo    = pair_other(rec_lo);
                const float4 o_hi    = pair_other(rec_hi);
                const int id_first   = odd ? other : own;
                const int id_second  = odd ? own : other;
                const float4 v_first = odd ? o_hi : rec_lo;
                const float4 v_second = odd ? rec_hi : o_lo;
                // own/other are record numbers
                if (id_first >= 0) partial_l[2 * (size_t)id_first + odd] = v_first;
                if (id_second >= 0) partial_l[2 * (size_t)id_second + odd] = v_second;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }

    // Every pixel adds to the same C background values. Atomics on one address serialise (the reference issues one per
    // pixel and channel, src/lib/rendering/RenderBackward.cu:1150-1152), so each workgroup reduces its 256 pixels and
    // stores one row of partial sums; reduce_background_kernel adds the rows up.
#pragma unroll
    for (int ci = 0; ci < C; ++ci)
    {
        const float s = wave_sum(bg_grad[ci]);
        if (lane == 0) red[wave][ci] = s;
    }
    {
        const float s = wave_sum(leak);
        if (lane == 0) red[wave][C] = s;
    }
    __syncthreads();
    if (threadIdx.x <= C)
        a.background_partial[(size_t)blockIdx.x * kBackgroundRow + threadIdx.x] =
            (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

template <int C, bool BILINEAR>
__global__ void __launch_bounds__(kBlock) blend_backward_kernel(BackwardPass a)
{
    blend_backward<C, BILINEAR>(a);
}

template <int C, bool BILINEAR>
__global__ void __launch_bounds__(kBlock) blend_backward_views_kernel(PerView<BackwardPass> views)
{
    blend_backward<C, BILINEAR>(views.v[blockIdx.y]);
}

// FUZZY_BLEND, per-pixel part of the backward pass: BlendBackwardsFuzzy<C>, src/lib/rendering/RenderBackward.cu:570-1080.
// Fragments are collected into a bucket while their depth stays within depth_accept of the bucket's first one (every
// bucket, unlike the forward kernel, which only averages the nearest one); the background, at depth 1e5, ends up in a
// bucket of its own. With the bucket's mean confidence c, mean descriptor t, m elements and the transmittance A in
// front of it:
//   d tex_e[ci] = (A * c * g[ci]) / m,   d conf_e = (A * (t . g)) / m  -  S_b / (1 - c + 1e-9)
// for each of its elements e, where S_b is the sum over all LATER buckets b' of sum_ci g[ci] t'[ci] A' c' (the
// reference hands every element in front of a bucket the bucket's whole term, :654-672). The reference walks all
// elements in front for every bucket, one thread per pixel; here the fragments of a pixel sit on neighbouring lanes and
// S_b is a sum from the back. The position part (:729-1080) is the neighbour-difference heuristic of the FULL_BLEND
// kernel. Records go to partial[layer][point] as there.

// Value the lane D places below (above) in the same row of 16 lanes holds; the lane's own value where the row has no
// such lane. DPP register moves; every lane of the wave must be active.
template <int D>
__device__ __forceinline__ float row_below(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x110 + D, 0xF, 0xF, false));
}
template <int D>
__device__ __forceinline__ float row_above(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), 0x100 + D, 0xF, 0xF, false));
}

// What the FUZZY_BLEND backward kernels know about a pixel before they look at its fragments.
struct FuzzyPixel
{
    uint32_t n, off;  // fragments after the cut, place of the first one
    bool do_point;
    float g[4], ax[4], ay[4], bx, by;  // upstream gradient; position heuristic in slope / offset form
};

template <int C>
__device__ __forceinline__ FuzzyPixel fuzzy_pixel(const BackwardPass& a, const TilePixel& px)
{
    FuzzyPixel f;
    f.n = f.off = 0, f.do_point = false, f.bx = f.by = 0.f;
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) f.g[ci] = f.ax[ci] = f.ay[ci] = 0.f;
    if (!px.active) return f;
    const int l = px.l, lw = a.ly.w[l], lh = a.ly.h[l];
    const size_t plane   = (size_t)lw * lh;
    const uint32_t local = px.local;
    const float* G       = a.grad_out[l];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) f.g[ci] = G[ci * plane + local];
    f.off = a.offsets[px.q];
    f.n   = a.offsets[px.q + 1] - f.off;
    if (a.K > 0) f.n = min(f.n, (uint32_t)a.K);
    f.do_point = a.need_point_gradient && f.n > 0 && interior_pixel(px.x, px.y, lw, lh);
    if (f.do_point)
    {
        // see blend_backward_kernel
        const float* I = a.out[l];
#pragma unroll
        for (int ci = 0; ci < C; ++ci)
        {
            const float* Ic = I + ci * plane + local;
            const float* Gc = G + ci * plane + local;
            const float Ix0 = Ic[-1], Ix1 = Ic[1], Iy0 = Ic[-lw], Iy1 = Ic[lw];
            const float Gx0 = Gc[-1], Gx1 = Gc[1], Gy0 = Gc[-lw], Gy1 = Gc[lw];
            f.ax[ci] = 0.5f * (Gx1 - Gx0);
            f.ay[ci] = 0.5f * (Gy1 - Gy0);
            f.bx += 0.5f * (Ix0 * Gx0 - Ix1 * Gx1);
            f.by += 0.5f * (Iy0 * Gy0 - Iy1 * Gy1);
        }
    }
    return f;
}

// Lists of up to kFuzzyDense fragments are laid out densely, one lane per FRAGMENT, as in blend_backward_kernel; what is
// different here is that a fragment's gradient depends on its whole bucket (means over the bucket's elements) and on
// all buckets of its pixel (transmittance in front, bucket terms behind), so a pixel's fragments must sit in one step
// of 64 lanes. Every pixel gets a slot of 1, 2, 4 ... 32 lanes (its list length rounded up to a power of two), the
// slots are handed out largest first, which keeps each aligned to its own size, and steps need no carries between
// them. A slot of up to kFuzzyNarrow lanes lies inside a row of 16 lanes: the sums over a bucket, the transmittance
// product and the sum of the bucket terms behind are shift-and-combine steps inside the row (register moves), and
// the step's code is compiled once per slot length so that shorter slots take fewer of them (the slots of a step
// are at most as long as its first). A slot of 32 lanes spans two rows: the same steps through the LDS crossbar, one
// more of them. Only the bucket boundaries are a sequential rule (a bucket starts where the depth leaves the range of
// the bucket's FIRST element), and that rule needs the depths alone: all lanes of a slot run it together over the
// slot's depths. Sums and products are combined pairwise instead of front to back, which moves the results by
// rounding only. The table that says which pixel a lane's fragment belongs to holds kWaveItems slots; a wave whose
// pixels need more goes through it in batches. Longer lists are left to blend_backward_fuzzy_long_kernel; the
// workgroup says in column kFuzzyLongColumn of its background row whether it has any.
constexpr int kFuzzyDense      = 32;  // longest list of the dense layout
constexpr int kFuzzyNarrow     = 16;  // longest slot that lies inside a row of 16 lanes
// The kernel is compiled for DENSE = kFuzzyNarrow (no slot spans rows: fewer registers, more waves per SIMD) and for
// DENSE = kFuzzyDense; the host takes the narrow one where the cut keeps every list that short, and also where lists
// beyond kFuzzyDense may exist: those go to blend_backward_fuzzy_long_kernel, which then is the faster one for the lists
// of 17 to 32 fragments as well (measured; slots of 64 lanes lost against it too).
constexpr int kFuzzyLongColumn = 6;   // background row, column 6: the workgroup has a list for the wave-per-list kernel
// The wave-per-list kernel is launched kFuzzyReplicas times over (grid.y): replica r takes every kFuzzyReplicas-th long
// list of a wave's pixels. Long lists cluster (where a surface is seen edge-on a whole strip of pixels holds hundreds
// of fragments each), and a wave takes its lists one after the other. Replica 0 adds its background sums to the row
// the dense kernel left for the workgroup; the others write rows of their own, which fold_background_rows_kernel adds up
// into kFuzzyFoldRows rows right behind the per-workgroup ones, so that the sum over the rows stays short:
// [workgroups] [kFuzzyFoldRows] [replica 1: workgroups] [replica 2: workgroups] ...
constexpr int kFuzzyReplicas   = 4;
constexpr int kFuzzyFoldRows   = 256;

template <int C, int DENSE>
__device__ __forceinline__ void blend_backward_fuzzy(const BackwardPass& a, float depth_accept)
{
    constexpr int kWaves = kBlock / kWave;
    __shared__ uint32_t s_off[kWaves][kWave];
    __shared__ uint16_t s_slot[kWaves][kWave];
    __shared__ uint8_t s_n[kWaves][kWave];
    __shared__ uint8_t s_point[kWaves][kWave];
    __shared__ float4 s_g[kWaves][kWave];
    __shared__ float4 s_ax[kWaves][kWave];
    __shared__ float4 s_ay[kWaves][kWave];
    __shared__ float2 s_bxy[kWaves][kWave];
    __shared__ uint8_t s_item[kWaves][kWaveItems];
    __shared__ float red[kWaves][C + 3];
    clear_small_accumulators(a.clear);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const TilePixel px = tile_pixel(a.tiles, a.ly);
    float4* partial_l  = a.partial;  // (records are addressed by gradient_record)
    const bool with_background = !a.use_environment_map;  // every list ends with the background element
    float bg_grad[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) bg_grad[ci] = 0.f;
    uint32_t n;
    {
        const FuzzyPixel f = fuzzy_pixel<C>(a, px);
        n                  = f.n;
        // an empty list: the background is the only bucket, one element of confidence 1 with nothing in front of it
        if (px.active && n == 0 && with_background)
#pragma unroll
            for (int ci = 0; ci < C; ++ci) bg_grad[ci] = f.g[ci];
        s_off[wave][lane]   = f.off;
        s_point[wave][lane] = f.do_point ? 1 : 0;
        s_g[wave][lane]     = make_float4(f.g[0], f.g[1], f.g[2], f.g[3]);
        if (f.do_point)
        {
            s_ax[wave][lane]  = make_float4(f.ax[0], f.ax[1], f.ax[2], f.ax[3]);
            s_ay[wave][lane]  = make_float4(f.ay[0], f.ay[1], f.ay[2], f.ay[3]);
            s_bxy[wave][lane] = make_float2(f.bx, f.by);
        }
    }
    const bool dense = n > 0 && n <= (uint32_t)DENSE;
    s_n[wave][lane]  = (uint8_t)(dense ? n : 0);

    // ---- slots, largest first ---------------------------------------------------------------------------------------
    const uint32_t size = dense ? (n > 1 ? 1u << (32 - __clz((int)n - 1)) : 1u) : 0u;
    uint32_t slot = 0, total = 0;
#pragma unroll
    for (uint32_t cls = DENSE; cls >= 1; cls >>= 1)
    {
        const uint64_t members = __ballot(size == cls);
        if (size == cls) slot = total + cls * (uint32_t)__popcll(members & ((1ull << lane) - 1ull));
        total += cls * (uint32_t)__popcll(members);
    }
    s_slot[wave][lane] = (uint16_t)slot;
    // the item table holds kWaveItems slots at a time: those from batch0 on (all of them unless slots span rows)
    constexpr bool kBatched = DENSE * kWave > kWaveItems;
    uint32_t batch0         = 0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // One step: 64 lanes, slots of at most BOUND lanes.
    auto step = [&](uint32_t k0, auto bound_constant) {
        constexpr uint32_t BOUND = decltype(bound_constant)::value;
        const uint32_t k = k0 + lane;
        const int p      = k < total ? (int)s_item[wave][k - batch0] : 255;
        const bool item  = p != 255;
        uint32_t np = 0, j = 0;
        int first = lane;  // first lane of the slot
        float depth = 0.f, conf = 0.f;
        float t[4]  = {0.f, 0.f, 0.f, 0.f};
        float g[4]  = {0.f, 0.f, 0.f, 0.f};
        int id = -1;
        if (item)
        {
            np    = s_n[wave][p];
            j     = k - s_slot[wave][p];
            first = lane - (int)j;
            const uint64_t key = a.fragments[s_off[wave][p] + j];
            depth              = __uint_as_float((uint32_t)(key >> 32));
            const int point    = (int)(uint32_t)key;
            int ti             = -1;
            // guards the gathers; never false for a workspace the forward pass wrote. An element that fails them
            // counts as a fragment with a zero descriptor and confidence and gets no record.
            if ((uint32_t)point < (uint32_t)a.N) ti = a.index ? a.index[point] : point;
            if ((uint32_t)ti < (uint32_t)a.N)
            {
                const float4 t4 = a.packed[2 * (size_t)ti];
                conf            = a.packed[2 * (size_t)ti + 1].x;
                t[0] = t4.x, t[1] = t4.y, t[2] = t4.z, t[3] = t4.w;
                id = point;
            }
            const float4 g4 = s_g[wave][p];
            g[0] = g4.x, g[1] = g4.y, g[2] = g4.z, g[3] = g4.w;
        }
        // bucket boundaries (src/lib/rendering/RenderBackward.cu:706-714): element 0 opens the first bucket whether or
        // not it resets the range
        float last_min = 0.f;
        uint32_t heads = 1u;
        if constexpr (BOUND > 1)
        {
            float d[BOUND];
#pragma unroll
            for (uint32_t i = 0; i < BOUND; ++i) d[i] = __shfl(depth, (first + (int)i) & (kWave - 1), kWave);
#pragma unroll
            for (uint32_t i = 0; i < BOUND; ++i)
                if (i < np && !(d[i] - last_min < depth_accept))
                {
                    last_min = d[i];
                    heads |= 1u << i;
                }
        }
        else if (!(depth - last_min < depth_accept))
            last_min = depth;
        // The background (depth MAX_DEPTH_CONST = 1e5, src/lib/rendering/RenderConstants.h:30) is a bucket of its own
        // unless the last bucket's range reaches that far: then it is one more element of that bucket.
        const bool bg_joins = with_background && (100000.f - last_min < depth_accept);

        const uint32_t head  = 31u - (uint32_t)__clz((int)(heads & ((2u << j) - 1u)));  // first element of this bucket
        const uint32_t later = heads >> (j + 1u);
        const uint32_t next  = later ? j + (uint32_t)__ffs((int)later) : np;  // first element of the next bucket
        const uint32_t dist  = j - head;
        const bool opens     = item && dist == 0u;
        const bool in_last   = item && next == np;
        const float inv      = 1.f / (float)(item ? next - head + (bg_joins && in_last ? 1u : 0u) : 1u);

        // sums over the bucket: inclusive scan from the bucket's first lane, the last lane of the bucket has the sums
        float sums[C + 1];
        sums[C] = conf;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) sums[ci] = t[ci];
        if constexpr (BOUND > 1)
        {
            const int last_lane = item ? first + (int)next - 1 : lane;
#pragma unroll
            for (int v = 0; v <= C; ++v)
            {
                float x = sums[v], o;
                o = row_below<1>(x); if (dist >= 1u) x += o;
                if constexpr (BOUND > 2) { o = row_below<2>(x); if (dist >= 2u) x += o; }
                if constexpr (BOUND > 4) { o = row_below<4>(x); if (dist >= 4u) x += o; }
                if constexpr (BOUND > 8) { o = row_below<8>(x); if (dist >= 8u) x += o; }
                sums[v] = __shfl(x, last_lane, kWave);
            }
        }
        if (bg_joins && in_last)
        {
            sums[C] += 1.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci) sums[ci] += a.background[ci];
        }
        const float bconf = sums[C] * inv;
        float dot = 0.f;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) dot += (sums[ci] * inv) * g[ci];
        // transmittance in front of the bucket: product of (1 - mean confidence) over the buckets before it
        float P = opens ? 1.f - bconf : 1.f;
        float A = 1.f, A_end = P;
        if constexpr (BOUND > 1)
        {
            float o;
            o = row_below<1>(P); if (j >= 1u) P *= o;
            if constexpr (BOUND > 2) { o = row_below<2>(P); if (j >= 2u) P *= o; }
            if constexpr (BOUND > 4) { o = row_below<4>(P); if (j >= 4u) P *= o; }
            if constexpr (BOUND > 8) { o = row_below<8>(P); if (j >= 8u) P *= o; }
            const float P_before = __shfl(P, (item && head > 0u) ? first + (int)head - 1 : lane, kWave);
            A_end                = __shfl(P, item ? first + (int)np - 1 : lane, kWave);  // behind the last bucket
            if (head > 0u) A = P_before;
        }
        // bucket terms behind this bucket (the background's included): suffix sum over the slot
        float x = 0.f;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) x += ((g[ci] * (sums[ci] * inv)) * A) * bconf;
        float S = 0.f;
        if constexpr (BOUND > 1)
        {
            float Q = opens ? x : 0.f, o;
            o = row_above<1>(Q); if (j + 1u < np) Q += o;
            if constexpr (BOUND > 2) { o = row_above<2>(Q); if (j + 2u < np) Q += o; }
            if constexpr (BOUND > 4) { o = row_above<4>(Q); if (j + 4u < np) Q += o; }
            if constexpr (BOUND > 8) { o = row_above<8>(Q); if (j + 8u < np) Q += o; }
            const float Q_next = __shfl(Q, (item && next < np) ? first + (int)next : lane, kWave);
            if (next < np) S = Q_next;
        }
        if (with_background && !bg_joins)
        {
            float xb = 0.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci) xb += ((g[ci] * a.background[ci]) * A_end) * 1.f;
            S += xb;
        }
        if (with_background && item && j + 1u == np)
        {
            // the background's share: an element of the last bucket, or a bucket of its own behind all others
            const float scale = bg_joins ? A * bconf : A_end * 1.f;
            const float share = bg_joins ? inv : 1.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci) bg_grad[ci] += (scale * g[ci]) * share;
        }
        float4 rec_lo = make_float4(0.f, 0.f, 0.f, 0.f), rec_hi = rec_lo;
        const bool give = item && id >= 0;
        if (give)
        {
            const float gconf = (dot * A) * inv - S / ((1.f - bconf) + 1e-9f);
            float gt[4]       = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ci = 0; ci < C; ++ci) gt[ci] = ((A * bconf) * g[ci]) * inv;
            float gp0 = 0.f, gp1 = 0.f;
            if (s_point[wave][p] & 1)
            {
                // the position part of an element's record depends on its own descriptor, not on the bucket's
                const float4 ax4 = s_ax[wave][p], ay4 = s_ay[wave][p];
                const float2 b2  = s_bxy[wave][p];
                const float ax[4] = {ax4.x, ax4.y, ax4.z, ax4.w}, ay[4] = {ay4.x, ay4.y, ay4.z, ay4.w};
                float dR_dpx = b2.x, dR_dpy = b2.y;
#pragma unroll
                for (int ci = 0; ci < C; ++ci)
                {
                    dR_dpx += t[ci] * ax[ci];
                    dR_dpy += t[ci] * ay[ci];
                }
                gp0 = dR_dpx / (float)C;
                gp1 = dR_dpy / (float)C;
            }
            rec_lo = make_float4(gt[0], gt[1], gt[2], gt[3]);
            rec_hi = make_float4(gconf, gp0, gp1, 0.f);
        }
        {
            // record stores, two lanes per record (see blend_backward_kernel)
            const int odd         = lane & 1;
            const int own         = give ? (int)gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, id) : -1;
            const int other       = pair_other(own);
            const float4 o_lo     = pair_other(rec_lo);
            const float4 o_hi     = pair_other(rec_hi);
            const int id_first    = odd ? other : own;
            const int id_second   = odd ? own : other;
            const float4 v_first  = odd ? o_hi : rec_lo;
            const float4 v_second = odd ? rec_hi : o_lo;
            if (id_first >= 0) partial_l[2 * (size_t)id_first + odd] = v_first;
            if (id_second >= 0) partial_l[2 * (size_t)id_second + odd] = v_second;
        }
    };
    // The same for slots that span rows (DENSE lanes at most): the combine steps go through the LDS crossbar instead of
    // register moves inside a row, and more of them reach across the slot. `bound`: the length of the step's first slot.
    auto step_wide = [&](uint32_t k0, uint32_t bound) {
        const uint32_t k = k0 + lane;
        const int p      = k < total ? (int)s_item[wave][k - batch0] : 255;
        const bool item  = p != 255;
        uint32_t np = 0, j = 0;
        int first = lane;  // first lane of the slot
        float depth = 0.f, conf = 0.f;
        float t[4]  = {0.f, 0.f, 0.f, 0.f};
        float g[4]  = {0.f, 0.f, 0.f, 0.f};
        int id = -1;
        if (item)
        {
            np    = s_n[wave][p];
            j     = k - s_slot[wave][p];
            first = lane - (int)j;
            const uint64_t key = a.fragments[s_off[wave][p] + j];
            depth              = __uint_as_float((uint32_t)(key >> 32));
            const int point    = (int)(uint32_t)key;
            int ti             = -1;
            // guards the gathers; never false for a workspace the forward pass wrote. An element that fails them
            // counts as a fragment with a zero descriptor and confidence and gets no record.
            if ((uint32_t)point < (uint32_t)a.N) ti = a.index ? a.index[point] : point;
            if ((uint32_t)ti < (uint32_t)a.N)
            {
                const float4 t4 = a.packed[2 * (size_t)ti];
                conf            = a.packed[2 * (size_t)ti + 1].x;
                t[0] = t4.x, t[1] = t4.y, t[2] = t4.z, t[3] = t4.w;
                id = point;
            }
            const float4 g4 = s_g[wave][p];
            g[0] = g4.x, g[1] = g4.y, g[2] = g4.z, g[3] = g4.w;
        }
        // bucket boundaries (src/lib/rendering/RenderBackward.cu:706-714): element 0 opens the first bucket whether or
        // not it resets the range
        float last_min = 0.f;
        uint64_t heads = 1ull;
        for (uint32_t i = 0; i < bound; ++i)
        {
            const float di = __shfl(depth, (first + (int)i) & (kWave - 1), kWave);
            if (i < np && !(di - last_min < depth_accept))
            {
                last_min = di;
                heads |= 1ull << i;
            }
        }
        // The background (depth MAX_DEPTH_CONST = 1e5, src/lib/rendering/RenderConstants.h:30) is a bucket of its own
        // unless the last bucket's range reaches that far: then it is one more element of that bucket.
        const bool bg_joins = with_background && (100000.f - last_min < depth_accept);

        const uint32_t head  = 63u - (uint32_t)__clzll((long long)(heads & (j >= 63u ? ~0ull : (2ull << j) - 1ull)));  // first element of this bucket
        const uint64_t later = j >= 63u ? 0ull : heads >> (j + 1u);
        const uint32_t next  = later ? j + (uint32_t)__ffsll((unsigned long long)later) : np;  // first element of the next bucket
        const uint32_t dist  = j - head;
        const bool opens     = item && dist == 0u;
        const bool in_last   = item && next == np;
        const float inv      = 1.f / (float)(item ? next - head + (bg_joins && in_last ? 1u : 0u) : 1u);

        // sums over the bucket: inclusive scan from the bucket's first lane, the last lane of the bucket has the sums
        float sums[C + 1];
        sums[C] = conf;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) sums[ci] = t[ci];
        {
            const int last_lane = item ? first + (int)next - 1 : lane;
#pragma unroll
            for (int v = 0; v <= C; ++v)
            {
                float x = sums[v];
#pragma unroll
                for (int d = 1; d < DENSE; d <<= 1)  // no slot is longer
                {
                    const float o = __shfl_up(x, d, kWave);
                    if (dist >= (uint32_t)d) x += o;
                }
                sums[v] = __shfl(x, last_lane, kWave);
            }
        }
        if (bg_joins && in_last)
        {
            sums[C] += 1.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci) sums[ci] += a.background[ci];
        }
        const float bconf = sums[C] * inv;
        float dot = 0.f;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) dot += (sums[ci] * inv) * g[ci];
        // transmittance in front of the bucket: product of (1 - mean confidence) over the buckets before it
        float P = opens ? 1.f - bconf : 1.f;
        float A = 1.f, A_end = P;
        {
#pragma unroll
            for (int d = 1; d < DENSE; d <<= 1)  // no slot is longer
            {
                const float o = __shfl_up(P, d, kWave);
                if (j >= (uint32_t)d) P *= o;
            }
            const float P_before = __shfl(P, (item && head > 0u) ? first + (int)head - 1 : lane, kWave);
            A_end                = __shfl(P, item ? first + (int)np - 1 : lane, kWave);  // behind the last bucket
            if (head > 0u) A = P_before;
        }
        // bucket terms behind this bucket (the background's included): suffix sum over the slot
        float x = 0.f;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) x += ((g[ci] * (sums[ci] * inv)) * A) * bconf;
        float S = 0.f;
        {
            float Q = opens ? x : 0.f;
#pragma unroll
            for (int d = 1; d < DENSE; d <<= 1)  // no slot is longer
            {
                const float o = __shfl_down(Q, d, kWave);
                if (j + (uint32_t)d < np) Q += o;
            }
            const float Q_next = __shfl(Q, (item && next < np) ? first + (int)next : lane, kWave);
            if (next < np) S = Q_next;
        }
        if (with_background && !bg_joins)
        {
            float xb = 0.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci) xb += ((g[ci] * a.background[ci]) * A_end) * 1.f;
            S += xb;
        }
        if (with_background && item && j + 1u == np)
        {
            // the background's share: an element of the last bucket, or a bucket of its own behind all others
            const float scale = bg_joins ? A * bconf : A_end * 1.f;
            const float share = bg_joins ? inv : 1.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci) bg_grad[ci] += (scale * g[ci]) * share;
        }
        float4 rec_lo = make_float4(0.f, 0.f, 0.f, 0.f), rec_hi = rec_lo;
        const bool give = item && id >= 0;
        if (give)
        {
            const float gconf = (dot * A) * inv - S / ((1.f - bconf) + 1e-9f);
            float gt[4]       = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ci = 0; ci < C; ++ci) gt[ci] = ((A * bconf) * g[ci]) * inv;
            float gp0 = 0.f, gp1 = 0.f;
            if (s_point[wave][p] & 1)
            {
                // the position part of an element's record depends on its own descriptor, not on the bucket's
                const float4 ax4 = s_ax[wave][p], ay4 = s_ay[wave][p];
                const float2 b2  = s_bxy[wave][p];
                const float ax[4] = {ax4.x, ax4.y, ax4.z, ax4.w}, ay[4] = {ay4.x, ay4.y, ay4.z, ay4.w};
                float dR_dpx = b2.x, dR_dpy = b2.y;
#pragma unroll
                for (int ci = 0; ci < C; ++ci)
                {
                    dR_dpx += t[ci] * ax[ci];
                    dR_dpy += t[ci] * ay[ci];
                }
                gp0 = dR_dpx / (float)C;
                gp1 = dR_dpy / (float)C;
            }
            rec_lo = make_float4(gt[0], gt[1], gt[2], gt[3]);
            rec_hi = make_float4(gconf, gp0, gp1, 0.f);
        }
        {
            // record stores, two lanes per record (see blend_backward_kernel)
            const int odd         = lane & 1;
            const int own         = give ? (int)gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, id) : -1;
            const int other       = pair_other(own);
            const float4 o_lo     = pair_other(rec_lo);
            const float4 o_hi     = pair_other(rec_hi);
            const int id_first    = odd ? other : own;
            const int id_second   = odd ? own : other;
            const float4 v_first  = odd ? o_hi : rec_lo;
            const float4 v_second = odd ? rec_hi : o_lo;
            if (id_first >= 0) partial_l[2 * (size_t)id_first + odd] = v_first;
            if (id_second >= 0) partial_l[2 * (size_t)id_second + odd] = v_second;
        }
    };
    for (uint32_t b0 = 0; b0 < total; b0 += kWaveItems)
    {
        if constexpr (kBatched) batch0 = b0;
        if (kBatched && batch0 != 0u)
        {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();  // every lane is done with the table of the batch before
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        // slots are aligned to their size and the table's size is a multiple of every size: none lies across two batches
        if (size != 0u && slot >= batch0 && slot < batch0 + (uint32_t)kWaveItems)
            for (uint32_t j = 0; j < size; ++j) s_item[wave][slot - batch0 + j] = j < n ? (uint8_t)lane : (uint8_t)255;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint32_t batch_end = min(total, batch0 + (uint32_t)kWaveItems);
        for (uint32_t k0 = batch0; k0 < batch_end; k0 += kWave)
        {
            // the first slot of a step is its longest
            const uint32_t n0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_n[wave][s_item[wave][k0 - batch0]]);
            if (DENSE > kFuzzyNarrow && n0 > (uint32_t)kFuzzyNarrow)
            {
                if constexpr (DENSE > kFuzzyNarrow) step_wide(k0, n0 > 32u ? 64u : 32u);
            }
            else if (n0 > 8)
                step(k0, std::integral_constant<uint32_t, 16>{});
            else if (n0 > 4)
                step(k0, std::integral_constant<uint32_t, 8>{});
            else if (n0 > 2)
                step(k0, std::integral_constant<uint32_t, 4>{});
            else if (n0 > 1)
                step(k0, std::integral_constant<uint32_t, 2>{});
            else
                step(k0, std::integral_constant<uint32_t, 1>{});
        }
        if constexpr (!kBatched) break;
    }

#pragma unroll
    for (int ci = 0; ci < C; ++ci)
    {
        const float s = wave_sum(bg_grad[ci]);
        if (lane == 0) red[wave][ci] = s;
    }
    {
        const bool longest = __ballot(n > (uint32_t)DENSE) != 0ull;
        if (lane == 0) red[wave][C] = 0.f;  // no background-confidence leak in this mode (guarded, RenderBackward.cu:643)
        if (lane == 0) red[wave][C + 1] = longest ? 1.f : 0.f;
    }
    __syncthreads();
    float* row = a.background_partial + (size_t)blockIdx.x * kBackgroundRow;
    if (threadIdx.x <= C) row[threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
    if (threadIdx.x == C + 1)
        row[kFuzzyLongColumn] = (red[0][C + 1] + red[1][C + 1]) + (red[2][C + 1] + red[3][C + 1]);
}

template <int C, int DENSE>
__global__ void __launch_bounds__(kBlock) blend_backward_fuzzy_kernel(BackwardPass a, float depth_accept)
{
    blend_backward_fuzzy<C, DENSE>(a, depth_accept);
}

template <int C, int DENSE>
__global__ void __launch_bounds__(kBlock) blend_backward_fuzzy_views_kernel(PerView<BackwardPass> views, float depth_accept)
{
    blend_backward_fuzzy<C, DENSE>(views.v[blockIdx.y], depth_accept);
}

// The lists blend_backward_fuzzy_kernel left out (more than `dense_max` fragments), one after the other, each by the
// whole wave: 64 consecutive fragments per step, front to back, one lane per fragment. The bucket boundaries of a step
// are found by a loop over its buckets that every lane runs alike (the rule is sequential, but it needs the depths
// only: all lanes test their depth against the open range at once, the first that fails opens the next bucket); sums
// over a bucket, the transmittance product over the buckets in front and the running sum of the bucket
// terms are scans over the lanes. What crosses a step boundary is carried in registers: the open bucket (sums, number
// of elements, first element), the depth its range started at, the transmittance in front of it and the sum of the
// bucket terms so far. A bucket's gradient needs the sum of the terms of all LATER buckets, so the list is processed
// twice: the first pass only adds up the terms, the second has the total and writes (a list of up to 64 fragments has
// its total inside its one step and is processed once). The elements of a bucket that was
// still open at the end of their step get the position part of their record there and the bucket's part when it
// closes, from a loop over their keys. Same grid as the dense kernel; a workgroup without such a list leaves at once.
template <int C>
__device__ __forceinline__ void blend_backward_fuzzy_long(const BackwardPass& a, float depth_accept, uint32_t dense_max)
{
    constexpr int kWaves = kBlock / kWave;
    __shared__ float red[kWaves][C];
    const uint32_t replica = blockIdx.y;
    float* row      = a.background_partial + (size_t)blockIdx.x * kBackgroundRow;
    float* row_mine = replica == 0u ? row
                                    : a.background_partial + ((size_t)kFuzzyFoldRows + (size_t)replica * gridDim.x + blockIdx.x) * kBackgroundRow;
    if (row[kFuzzyLongColumn] == 0.f)
    {
        if (replica != 0u && threadIdx.x < (uint32_t)kBackgroundRow) row_mine[threadIdx.x] = 0.f;
        return;
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const TilePixel px = tile_pixel(a.tiles, a.ly);
    const FuzzyPixel f = fuzzy_pixel<C>(a, px);
    float4* partial_l  = a.partial;  // (records are addressed by gradient_record)
    const bool with_background = !a.use_environment_map;
    float bg_grad[C];  // summed over the wave at the end: every lane adds what it computes for lane 0's sake once
#pragma unroll
    for (int ci = 0; ci < C; ++ci) bg_grad[ci] = 0.f;
    auto everywhere = [&](float v, int src) { return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), src)); };

    uint64_t todo = __ballot(f.n > dense_max);
    for (uint32_t turn = 0; todo != 0ull; ++turn)
    {
        const int src = __ffsll((unsigned long long)todo) - 1;
        todo &= todo - 1ull;
        if (turn % (uint32_t)kFuzzyReplicas != replica) continue;
        // the pixel, the same on every lane
        const uint32_t n       = (uint32_t)__builtin_amdgcn_readlane((int)f.n, src);
        const uint64_t* list   = a.fragments + (uint32_t)__builtin_amdgcn_readlane((int)f.off, src);
        const bool do_point    = __builtin_amdgcn_readlane((int)f.do_point, src) != 0;
        float g[4], ax[4], ay[4];
#pragma unroll
        for (int ci = 0; ci < 4; ++ci) g[ci] = everywhere(f.g[ci], src), ax[ci] = everywhere(f.ax[ci], src), ay[ci] = everywhere(f.ay[ci], src);
        const float bx = everywhere(f.bx, src), by = everywhere(f.by, src);

        // A list that fits one step needs no first pass: the total is known inside the step.
        const bool one_step = n <= (uint32_t)kWave;
        double total = 0.0;
#pragma unroll 1
        for (int pass = one_step ? 1 : 0; pass < 2; ++pass)
        {
            // carried from step to step (the same on every lane)
            float open_sums[C + 1];
#pragma unroll
            for (int v = 0; v <= C; ++v) open_sums[v] = 0.f;
            uint32_t open_m = 0, open_start = 0;
            float last_min = 0.f, A_front = 1.f;  // transmittance in front of the open bucket
            double prefix  = 0.0;                 // bucket terms of the closed buckets
#pragma unroll 1
            for (uint32_t begin = 0; begin < n; begin += kWave)
            {
                const uint32_t valid = min((uint32_t)kWave, n - begin);
                const bool last_step = begin + kWave >= n;
                const bool has       = (uint32_t)lane < valid;
                float depth = 0.f, conf = 0.f;
                float t[4]  = {0.f, 0.f, 0.f, 0.f};
                int id = -1;
                if (has)
                {
                    const uint64_t key = list[begin + lane];
                    depth              = __uint_as_float((uint32_t)(key >> 32));
                    const int point    = (int)(uint32_t)key;
                    int ti             = -1;
                    if ((uint32_t)point < (uint32_t)a.N) ti = a.index ? a.index[point] : point;
                    if ((uint32_t)ti < (uint32_t)a.N)
                    {
                        const float4 t4 = a.packed[2 * (size_t)ti];
                        conf            = a.packed[2 * (size_t)ti + 1].x;
                        t[0] = t4.x, t[1] = t4.y, t[2] = t4.z, t[3] = t4.w;
                        id = point;
                    }
                }
                // ---- bucket boundaries of this step (src/lib/rendering/RenderBackward.cu:706-714); element 0 of the
                // list opens the first bucket whether or not it resets the range
                // One trip per bucket, not per element: the elements that do not fit the open range are found by all
                // lanes at once, the first of them opens the next bucket and sets the next range.
                uint64_t heads = begin == 0 ? 1ull : 0ull;
                for (uint64_t beyond = __ballot(has && !(depth - last_min < depth_accept)); beyond != 0ull;)
                {
                    const int i = __ffsll((unsigned long long)beyond) - 1;
                    heads |= 1ull << i;
                    last_min = everywhere(depth, i);
                    beyond   = __ballot(has && lane > i && !(depth - last_min < depth_accept));
                }
                // the background (depth 1e5) behind the last fragment: one more element of the last bucket if that
                // bucket's range reaches it, else a bucket of its own
                const bool bg_joins = last_step && with_background && (100000.f - last_min < depth_accept);

                // ---- a bucket that was open and has no element in this step closes in front of it
                if (open_m != 0u && (heads & 1ull))
                {
                    const float inv   = 1.f / (float)open_m;
                    const float bconf = open_sums[C] * inv;
                    float dot = 0.f, x = 0.f;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci)
                    {
                        const float tb = open_sums[ci] * inv;
                        dot += tb * g[ci];
                        x += ((g[ci] * tb) * A_front) * bconf;
                    }
                    if (pass == 0)
                        total += (double)x;
                    else
                    {
                        prefix += (double)x;
                        const float S     = (float)(total - prefix);
                        const float gconf = (dot * A_front) * inv - S / ((1.f - bconf) + 1e-9f);
                        float gt[4]       = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int ci = 0; ci < C; ++ci) gt[ci] = ((A_front * bconf) * g[ci]) * inv;
                        for (uint32_t e = open_start + lane; e < begin; e += kWave)
                        {
                            const int point = (int)(uint32_t)list[e];
                            int ti          = -1;
                            if ((uint32_t)point < (uint32_t)a.N) ti = a.index ? a.index[point] : point;
                            if ((uint32_t)ti >= (uint32_t)a.N) continue;
                            partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, point)] = make_float4(gt[0], gt[1], gt[2], gt[3]);
                            reinterpret_cast<float*>(&partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, point) + 1])[0] = gconf;
                        }
                    }
                    A_front = (1.f - bconf) * A_front;
                    open_m  = 0u;
#pragma unroll
                    for (int v = 0; v <= C; ++v) open_sums[v] = 0.f;
                }

                // ---- this lane's bucket inside the step
                const uint64_t upto  = heads & (lane == kWave - 1 ? ~0ull : (2ull << lane) - 1ull);
                const bool joined    = upto == 0ull;  // belongs to the bucket that was open when the step began
                const uint32_t first = joined ? 0u : 63u - (uint32_t)__clzll((long long)upto);
                const uint64_t later = lane == kWave - 1 ? 0ull : heads >> (lane + 1);
                uint32_t next        = later ? (uint32_t)lane + (uint32_t)__ffsll((unsigned long long)later) : valid;
                next                 = min(next, valid);
                const uint32_t dist  = (uint32_t)lane - first;
                const bool closes    = has && (next < valid || last_step);  // the bucket ends in this step
                const bool tail      = has && next == valid;                // the last bucket of the step
                // sums over the bucket's elements of this step: inclusive scan from its first lane, read at its last
                float sums[C + 1];
                sums[C] = conf;
#pragma unroll
                for (int ci = 0; ci < C; ++ci) sums[ci] = t[ci];
                const int last_lane = has ? (int)next - 1 : lane;
#pragma unroll
                for (int v = 0; v <= C; ++v)
                {
                    float x = sums[v];
#pragma unroll
                    for (int d = 1; d < kWave; d <<= 1)
                    {
                        const float o = __shfl_up(x, d, kWave);
                        if (dist >= (uint32_t)d) x += o;
                    }
                    sums[v] = __shfl(x, last_lane, kWave);
                    if (joined) sums[v] = open_sums[v] + sums[v];
                }
                uint32_t m = has ? (next - first) + (joined ? open_m : 0u) : 1u;
                if (bg_joins && tail)
                {
                    sums[C] += 1.f;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci) sums[ci] += a.background[ci];
                    m += 1u;
                }
                const float inv   = 1.f / (float)m;
                const float bconf = sums[C] * inv;
                float dot = 0.f;
#pragma unroll
                for (int ci = 0; ci < C; ++ci) dot += (sums[ci] * inv) * g[ci];
                // transmittance in front: product of (1 - mean confidence) over the buckets that close in this step in
                // front of this one, times what was in front of the step
                const bool closing_lane = closes && lane == last_lane;
                float P = closing_lane ? 1.f - bconf : 1.f;
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1)
                {
                    const float o = __shfl_up(P, d, kWave);
                    if (lane >= d) P *= o;
                }
                const float P_before = __shfl(P, first > 0u ? (int)first - 1 : lane, kWave);
                const float A        = first > 0u ? A_front * P_before : A_front;
                const float P_end    = everywhere(P, (int)valid - 1);  // over all buckets that close in this step
                float x = 0.f;
#pragma unroll
                for (int ci = 0; ci < C; ++ci) x += ((g[ci] * (sums[ci] * inv)) * A) * bconf;
                // Terms of the buckets that close in this step, summed from the back: a bucket needs the terms of the
                // buckets BEHIND it, and taking them as (all) - (those in front) would cancel to rounding noise deep in
                // a list, where what is left behind is a millionth of what lies in front.
                float X = closing_lane ? x : 0.f;
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1)
                {
                    const float o = __shfl_down(X, d, kWave);
                    if (lane + d < kWave) X += o;
                }
                const float X_end = everywhere(X, 0);  // all of them
                if (one_step)
                {
                    // what the first pass would have left, from the same terms in the same order
                    total = (double)X_end;
                    if (with_background && !bg_joins)
                    {
                        float xb = 0.f;
#pragma unroll
                        for (int ci = 0; ci < C; ++ci) xb += ((g[ci] * a.background[ci]) * (A_front * P_end)) * 1.f;
                        total += (double)xb;
                    }
                }
                if (pass == 1)
                {
                    // behind this lane's bucket inside the step
                    // (the exchange is made by every lane, then the lanes with nothing behind them drop what they got)
                    const float X_next   = __shfl(X, min(last_lane + 1, kWave - 1), kWave);
                    const float X_behind = last_lane + 1 < kWave ? X_next : 0.f;
                    float gp0 = 0.f, gp1 = 0.f;
                    if (has && id >= 0 && do_point)
                    {
                        float dR_dpx = bx, dR_dpy = by;
#pragma unroll
                        for (int ci = 0; ci < C; ++ci)
                        {
                            dR_dpx += t[ci] * ax[ci];
                            dR_dpy += t[ci] * ay[ci];
                        }
                        gp0 = dR_dpx / (float)C;
                        gp1 = dR_dpy / (float)C;
                    }
                    // ... and behind the step: both sums are made of the same float terms, so this difference is exact
                    const float S     = X_behind + (float)(total - (prefix + (double)X_end));
                    const float gconf = (dot * A) * inv - S / ((1.f - bconf) + 1e-9f);
                    float gt[4]       = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ci = 0; ci < C; ++ci) gt[ci] = ((A * bconf) * g[ci]) * inv;
                    if (has && id >= 0)
                    {
                        if (closes)
                        {
                            partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, id)]     = make_float4(gt[0], gt[1], gt[2], gt[3]);
                            partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, id) + 1] = make_float4(gconf, gp0, gp1, 0.f);
                        }
                        else
                        {
                            // the bucket stays open: its part of the record follows when it closes
                            float* rec = reinterpret_cast<float*>(&partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, id) + 1]);
                            rec[1] = gp0, rec[2] = gp1, rec[3] = 0.f;
                        }
                    }
                    // the elements an earlier step left with a bucket that closes here
                    const bool joined_closes = open_m != 0u && __builtin_amdgcn_readlane((int)(closes && joined), 0) != 0;
                    if (joined_closes)
                    {
                        float gt0[4];
#pragma unroll
                        for (int ci = 0; ci < 4; ++ci) gt0[ci] = everywhere(gt[ci], 0);
                        const float gconf0 = everywhere(gconf, 0);
                        for (uint32_t e = open_start + lane; e < begin; e += kWave)
                        {
                            const int point = (int)(uint32_t)list[e];
                            int ti          = -1;
                            if ((uint32_t)point < (uint32_t)a.N) ti = a.index ? a.index[point] : point;
                            if ((uint32_t)ti >= (uint32_t)a.N) continue;
                            partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, point)] = make_float4(gt0[0], gt0[1], gt0[2], gt0[3]);
                            reinterpret_cast<float*>(&partial_l[2 * gradient_record(a.point_major_records, a.N, a.ly.L, 1, px.l, 0, point) + 1])[0] = gconf0;
                        }
                    }
                    if (last_step && with_background && lane == (int)valid - 1)
                    {
                        // the background's share: an element of the last bucket, or a bucket of its own behind all
                        const float scale = bg_joins ? A * bconf : (A_front * P_end) * 1.f;
                        const float share = bg_joins ? inv : 1.f;
#pragma unroll
                        for (int ci = 0; ci < C; ++ci) bg_grad[ci] += (scale * g[ci]) * share;
                    }
                }
                // ---- what the next step inherits
                if (pass == 0)
                    total += (double)X_end;
                else
                    prefix += (double)X_end;
                if (last_step)
                {
                    if (pass == 0 && with_background && !bg_joins)
                    {
                        float xb = 0.f;
#pragma unroll
                        for (int ci = 0; ci < C; ++ci) xb += ((g[ci] * a.background[ci]) * (A_front * P_end)) * 1.f;
                        total += (double)xb;
                    }
                }
                else
                {
                    // the last bucket of the step stays open (valid = 64 here)
                    const bool all_joined   = heads == 0ull;
                    const uint32_t open_pos = all_joined ? 0u : 63u - (uint32_t)__clzll((long long)heads);
#pragma unroll
                    for (int v = 0; v <= C; ++v) open_sums[v] = everywhere(sums[v], kWave - 1);
                    open_m     = (uint32_t)kWave - open_pos + (all_joined ? open_m : 0u);
                    open_start = all_joined ? open_start : begin + open_pos;
                    A_front    = A_front * P_end;
                }
            }
        }
    }
#pragma unroll
    for (int ci = 0; ci < C; ++ci)
    {
        const float s = wave_sum(bg_grad[ci]);
        if (lane == 0) red[wave][ci] = s;
    }
    __syncthreads();
    if (threadIdx.x < (uint32_t)kBackgroundRow)
    {
        const float sum = threadIdx.x < C ? (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]) : 0.f;
        if (replica == 0u)
        {
            if (threadIdx.x < C) row[threadIdx.x] += sum;
        }
        else
            row_mine[threadIdx.x] = sum;
    }
}

template <int C>
__global__ void __launch_bounds__(kBlock) blend_backward_fuzzy_long_kernel(BackwardPass a, float depth_accept, uint32_t dense_max)
{
    blend_backward_fuzzy_long<C>(a, depth_accept, dense_max);
}

// (blockIdx.y is the replica here)
template <int C>
__global__ void __launch_bounds__(kBlock) blend_backward_fuzzy_long_views_kernel(PerView<BackwardPass> views, float depth_accept,
                                                                                 uint32_t dense_max)
{
    blend_backward_fuzzy_long<C>(views.v[blockIdx.z], depth_accept, dense_max);
}

// Adds `num_rows` rows of kBackgroundRow floats up into kFuzzyFoldRows rows: workgroup j takes rows j, j + 256, ... in a
// fixed order (32 threads per column, each every 32nd of the workgroup's rows, then the 32 partial sums one after the other).
__device__ __forceinline__ void fold_background_rows(const float* __restrict__ rows, int num_rows, float* __restrict__ folded)
{
    __shared__ float part[kBlock / kBackgroundRow][kBackgroundRow];
    const int column = threadIdx.x % kBackgroundRow, sub = threadIdx.x / kBackgroundRow;
    float sum = 0.f;
    for (int r = blockIdx.x + kFuzzyFoldRows * sub; r < num_rows; r += kFuzzyFoldRows * (kBlock / kBackgroundRow))
        sum += rows[(size_t)r * kBackgroundRow + column];
    part[sub][column] = sum;
    __syncthreads();
    if (threadIdx.x < (uint32_t)kBackgroundRow)
    {
        float total = 0.f;
        for (int k = 0; k < kBlock / kBackgroundRow; ++k) total += part[k][threadIdx.x];
        folded[(size_t)blockIdx.x * kBackgroundRow + threadIdx.x] = total;
    }
}

__global__ void __launch_bounds__(kBlock) fold_background_rows_kernel(const float* __restrict__ rows, int num_rows,
                                                                      float* __restrict__ folded)
{
    fold_background_rows(rows, num_rows, folded);
}

struct FoldArgs
{
    const float* rows;
    int num_rows;
    float* folded;
};

__global__ void __launch_bounds__(kBlock) fold_background_rows_views_kernel(PerView<FoldArgs> views)
{
    const FoldArgs& v = views.v[blockIdx.y];
    fold_background_rows(v.rows, v.num_rows, v.folded);
}

// Sums the per-workgroup background rows of one view (one workgroup, fixed order, so the result is reproducible) and
// adds the background pseudo-fragment's alpha gradient to confidence row 0 when that switch of the reference's
// behaviour is on (src/lib/rendering/RenderBackward.cu:1130-1131,1157).
// Sum of the per-workgroup background rows of one view by one workgroup of BLOCK threads, in a fixed order, so the
// result is reproducible. Also adds the background pseudo-fragment's alpha gradient to confidence row 0 when that switch
// of the reference's behaviour is on (src/lib/rendering/RenderBackward.cu:1130-1131,1157); with `leak_atomic` that
// add is an atomic (rows are being added to by other workgroups), otherwise the caller guarantees row 0 has its value.
template <int BLOCK>
__device__ __forceinline__ void sum_background_rows(const float* __restrict__ rows, int num_rows, int C,
                                                    float* __restrict__ grad_background,
                                                    float* __restrict__ grad_confidence, int add_leak, int accumulate,
                                                    int leak_atomic, const float* abs_of = nullptr,
                                                    float leak_factor = 1.f)
{
    __shared__ float red[BLOCK / kWave][kBackgroundRow];
    float acc[kBackgroundRow];
#pragma unroll
    for (int k = 0; k < kBackgroundRow; ++k) acc[k] = 0.f;
    // several independent row loads per thread and trip: one workgroup has to pull in ~10^4 rows and would otherwise
    // sit on one memory round trip per row
    constexpr int kUnroll = 4;
    for (int r0 = threadIdx.x; r0 < num_rows; r0 += BLOCK * kUnroll)
    {
        float4 a0[kUnroll];
        float a1[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const int r = r0 + u * BLOCK;
            a0[u]       = make_float4(0.f, 0.f, 0.f, 0.f);
            a1[u]       = 0.f;
            if (r < num_rows)
            {
                a0[u] = reinterpret_cast<const float4*>(rows)[2 * (size_t)r];
                a1[u] = rows[(size_t)r * kBackgroundRow + 4];
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            acc[0] += a0[u].x;
            acc[1] += a0[u].y;
            acc[2] += a0[u].z;
            acc[3] += a0[u].w;
            acc[4] += a1[u];
        }
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int k = 0; k < 5; ++k)
    {
        const float s = wave_sum(acc[k]);
        if (lane == 0) red[wave][k] = s;
    }
    __syncthreads();
    if (threadIdx.x <= C)
    {
        const int k = threadIdx.x;
        float s     = 0.f;
        for (int w = 0; w < BLOCK / kWave; ++w) s += red[w][k];
        if (k < C)
        {
            if (abs_of) s = s * (abs_of[k] > 0.f ? 1.f : (abs_of[k] < 0.f ? -1.f : 0.f));  // background = |raw|
            grad_background[k] = accumulate ? grad_background[k] + s : s;
        }
        else if (add_leak)
        {
            s = s * leak_factor;  // chain rule of a fused confidence activation for row 0
            if (leak_atomic)
                atomicAdd(&grad_confidence[0], s);
            else
                grad_confidence[0] += s;
        }
    }
}

// Stand-alone form for a cloud without points (the per-point kernel, which otherwise does this sum, is not launched).
constexpr int kReduceBlock = 1024;
__global__ void __launch_bounds__(kReduceBlock) reduce_background_kernel(const float* __restrict__ rows, int num_rows,
                                                                          int C, float* __restrict__ grad_background,
                                                                          float* __restrict__ grad_confidence,
                                                                          int add_leak, int accumulate,
                                                                          const float* __restrict__ abs_of)
{
    sum_background_rows<kReduceBlock>(rows, num_rows, C, grad_background, grad_confidence, add_leak, accumulate, 0,
                                      abs_of);
}

struct GatherPass
{
    ViewPass vp;
    const uint32_t* offsets;
    const uint64_t* fragments;
    const uint8_t* list_is_cut;  // per pixel, written by the build pass
    const uint64_t* last_key;    // per pixel with list_is_cut: key of the last fragment that took part in the blend
    const uint32_t* kept;        // per pixel, BILINEAR_BLEND: fragments of its list that took part in the blend
    const float4* partial;
    float* grad_texture;      // [C,N]
    float* grad_confidence;   // [N]
    float* grad_points;       // [N,4] or null
    float* grad_point_count;  // [N]
    double* camera_partial;   // [workgroups][kCameraRow] per-workgroup pose / intrinsics sums, or null
    int K;
    int need_point_gradient;
    // One launch takes a round of up to kViewLanes views: the pointers above are those of the round's first view, view
    // v of the round lies v * the stride behind them (per-view arrays of the workspace; the record and background-row
    // arrays of the view's lane; a camera-row block per view). A point's position is read once for all of them and its
    // gradient rows are written once.
    int point_major_records;  // layout of the record array, see gradient_record
    int view_count;
    size_t dropout_stride, flags_stride, last_key_stride, kept_stride;  // elements of the respective arrays
    size_t partial_stride, background_rows_stride, camera_partial_stride;
    int accumulate;  // 0: overwrite the gradient rows (the call's first round), 1: add to them (further rounds)
    // background gradient: workgroup 0 also sums the rows the per-pixel kernel left (hidden behind the other workgroups)
    const float* background_rows;
    int num_background_rows;
    float* grad_background;
    int add_leak;
    int background_accumulate;  // for the round's first view; the others always add
    // chain rule of the fused preparation steps (confidence = sigmoid(scale * raw), texture = |raw|, background = |raw|):
    // the gradients written are those of the raw tensors
    const float4* packed;      // prepared confidence of a row: packed[2 * row + 1].x
    const float* texture_raw;  // [C,N]
    const float* background_raw;
    int confidence_activation;
    float confidence_scale;
    int texture_abs;
};

__device__ __forceinline__ float sign_of(float x)
{
    return x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f);  // torch's abs backward: grad * sign(x)
}

constexpr int kCameraRow  = 20;  // doubles per workgroup row: 6 pose tangent, fx, fy, cx, cy, 8 distortion, fragment count, pad
constexpr int kCameraSums = 18;  // of them sums of per-fragment terms

// One thread per point: find the pixel the point fell into in every layer (the same projection as the scatter pass), decide
// whether its fragment survived the top-K cut (its key is not larger than the K-th key of that pixel's sorted list), and
// sum the stored records. With a texture index indirection several points may share a descriptor row; only then the
// descriptor and confidence sums are added with atomics (onto rows the host zero-filled).
// HITS = 4 (BILINEAR_BLEND): a point has up to four fragments per layer, one per corner of its 2x2 pixels, with records
// at partial[layer][corner][point].
// MANY: the launch takes a round of several views (a.view_count of them); otherwise one view, and the loop over the
// views and its address arithmetic fold away (the kernel then needs 58 registers instead of 71 to 77, and it lives
// off the number of waves in flight).
template <int C, int HITS, bool DISTORT = false, bool MANY = false>
__global__ void __launch_bounds__(kBlock) gather_point_gradients_kernel(GatherPass a)
{
    const int view_count = MANY ? a.view_count : 1;
    const int i      = blockIdx.x * blockDim.x + threadIdx.x;
    const bool alive = i < a.vp.N;
    const int N      = a.vp.N;
    // sums over the fragments of the point in all views of the round
    float gt[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) gt[ci] = 0.f;
    float gc = 0.f, gx = 0.f, gy = 0.f, gz = 0.f, cnt = 0.f;
    bool hit = false;   // the point has a blended fragment in one of the views
    constexpr int kSums = DISTORT ? kCameraSums : 10;
    const float4 wp     = alive ? a.vp.position[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    // skipped in every view alike (viewer cut-off), or in this view (drop-out mask)
    const bool never = !alive || point_is_skipped_in_all_views(a.vp, i);
  for (int view = 0; view < view_count; ++view)
  {
    const float* dropout       = a.vp.dropout ? a.vp.dropout + (size_t)view * a.dropout_stride : nullptr;
    const uint8_t* list_is_cut = a.list_is_cut + (size_t)view * a.flags_stride;
    const uint64_t* last_key   = a.last_key + (size_t)view * a.last_key_stride;
    const float4* partial      = a.partial + (size_t)view * a.partial_stride;
    // pose tangent (translation, rotation), fx, fy, cx, cy and, in the kernel for cameras with distortion, k1 .. p2:
    // per view
    float cam_sum[kSums];
#pragma unroll
    for (int k = 0; k < kSums; ++k) cam_sum[k] = 0.f;
    float view_cnt = 0.f;
    Projected p;
    const DeviceView& cam = a.vp.view[view];
    // (a position further outside the image than the coarsest layer's border pixels reach has no fragment in any
    // layer, see bin_scatter_kernel: most of the cloud, for a crop)
    const float reach = (float)(1 << (a.vp.ly.L - 1)) + 1.f;
    if (!never && !(dropout && dropout[i] == 1.f) && project_point(cam, wp, p) && p.ipx >= -reach &&
        p.ipx <= (float)a.vp.ly.w[0] + reach && p.ipy >= -reach && p.ipy <= (float)a.vp.ly.h[0] + reach)
    {
        // view-space position again, for the projection Jacobian (same expressions as project_point)
        const float vx = ((cam.r[0] * wp.x + cam.r[1] * wp.y) + cam.r[2] * wp.z) + cam.t[0];
        const float vy = ((cam.r[3] * wp.x + cam.r[4] * wp.y) + cam.r[5] * wp.z) + cam.t[1];
        const float vz = ((cam.r[6] * wp.x + cam.r[7] * wp.y) + cam.r[8] * wp.z) + cam.t[2];
        const uint64_t depth_key = (uint64_t)__float_as_uint(p.z) << 32;
        float ipx = p.ipx, ipy = p.ipy, radius = p.radius;
        const LayerTable& ly = a.vp.ly;
        for (int l = 0; l < ly.L; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
        {
            if (a.vp.drop_by_radius && radius < a.vp.radius_threshold) break;
#pragma unroll
          for (int h = 0; h < HITS; ++h)
          {
            const float fx = HITS == 1 ? rintf(ipx) : floorf(ipx) + (float)(h & 1);
            const float fy = HITS == 1 ? rintf(ipy) : floorf(ipy) + (float)(h >> 1);
            if (!(fx >= 0.f && fx < (float)ly.w[l] && fy >= 0.f && fy < (float)ly.h[l])) continue;
            const int x = (int)fx, y = (int)fy;
            const uint32_t q   = (ly.tile_base[l] + (uint32_t)(y / kTile) * (uint32_t)ly.tiles_x[l] + (uint32_t)(x / kTile)) * kTilePixels +
                               (uint32_t)(y % kTile) * kTile + (uint32_t)(x % kTile);
            // Did the fragment take part in the blend? Only where the pixel's list was not blended to its end (top-K
            // cut, saturation) the last blended key has to be looked up.
            // (FULL_BLEND without a cut never sets the flag; the K > 0 test keeps a corrupted flag byte from turning
            // K <= 0 into an index.)
            if (list_is_cut[q] && (HITS != 1 || a.K > 0))
            {
                const uint64_t key = depth_key | (HITS == 1 ? (uint32_t)i : (((uint32_t)i << 2) | (uint32_t)h));
                if (key > last_key[q]) continue;  // 0 where no fragment was blended: every key is beyond it
            }
            const size_t rec = gradient_record(a.point_major_records, a.vp.N, ly.L, HITS, l, h, i);
            const float4 r0  = partial[2 * rec];
            const float4 r1  = partial[2 * rec + 1];
            const float r[4] = {r0.x, r0.y, r0.z, r0.w};
#pragma unroll
            for (int ci = 0; ci < C; ++ci) gt[ci] += r[ci];
            gc += r1.x;
            hit = true;
            if (a.need_point_gradient && interior_pixel(x, y, ly.w[l], ly.h[l]))
            {
                // ProjectPointPinholeBackward (src/lib/rendering/PointRendererHelper.h:317-372) for zero distortion, with
                // the crop transform scaled by 0.5^layer (src/lib/rendering/RenderBackward.cu:1381-1385; 2^-l is exact):
                // crop rotation^T, crop K^T, K^T, divide-by-z Jacobian^T, R^T.
                const float scale = __uint_as_float((uint32_t)(127 - l) << 23);
                const float cfx = cam.crop[0] * scale, cfy = cam.crop[1] * scale, cs = cam.crop[4] * scale;
                const float gxp = r1.y, gyp = r1.z;
                const float ar = cam.rot[0] * gxp + cam.rot[2] * gyp;
                const float br = cam.rot[1] * gxp + cam.rot[3] * gyp;
                const float a2 = cfx * ar;
                const float b2 = cs * ar + cfy * br;
                float d0 = cam.fx * a2;
                float d1 = cam.s * a2 + cam.fy * b2;
                float nx = vx / vz, ny = vy / vz;  // the point K is applied to
                if constexpr (DISTORT)
                {
                    // J_dis_dis^T and J_p_dis^T of the distortion (src/lib/rendering/PointRendererHelper.h:346-368). The
                    // kernel is compiled in this form for callers that have switched distortion on, whatever the
                    // coefficients are: where all of them are zero J is exactly the identity (the other gradients keep
                    // their bits) and the coefficient gradients are not zero (x r^2 and so on), so such a camera can
                    // start to learn its distortion.
                    float J[4], Jd[16], xd, yd;
                    distort_point_jacobians(cam.dist, nx, ny, xd, yd, J, Jd);
#pragma unroll
                    for (int k = 0; k < 8; ++k) cam_sum[10 + k] += Jd[2 * k] * d0 + Jd[2 * k + 1] * d1;
                    const float n0 = J[0] * d0 + J[2] * d1, n1 = J[1] * d0 + J[3] * d1;
                    d0 = n0, d1 = n1;
                    nx = xd, ny = yd;
                }
                const float iz = 1.f / vz;
                const float e0 = iz * d0, e1 = iz * d1;
                const float e2 = (-vx * iz * iz) * d0 + (-vy * iz * iz) * d1;
                gx += (cam.r[0] * e0 + cam.r[3] * e1) + cam.r[6] * e2;
                gy += (cam.r[1] * e0 + cam.r[4] * e1) + cam.r[7] * e2;
                gz += (cam.r[2] * e0 + cam.r[5] * e1) + cam.r[8] * e2;
                cnt += 1.f;
                view_cnt += 1.f;
                if (a.camera_partial)
                {
                    // pose: J_pose^T e with J_pose = [I | -[view_p]x] (tangent = translation, rotation; applied on the
                    // left, src/lib/rendering/PointRenderer.cu:1325-1341); K: d image / d (fx, fy, cx, cy)
                    // (src/lib/rendering/RenderBackward.cu:1418-1437, the skew column is zeroed there)
                    cam_sum[0] += e0;
                    cam_sum[1] += e1;
                    cam_sum[2] += e2;
                    cam_sum[3] += vy * e2 - vz * e1;
                    cam_sum[4] += vz * e0 - vx * e2;
                    cam_sum[5] += vx * e1 - vy * e0;
                    cam_sum[6] += nx * a2;
                    cam_sum[7] += ny * b2;
                    cam_sum[8] += a2;
                    cam_sum[9] += b2;
                }
            }
          }
        }
    }
    if (a.camera_partial)
    {
        // workgroup sums in double, one row per workgroup; reduce_camera_kernel adds the rows of a view
        __shared__ double cam_red[kBlock / kWave][kCameraRow];
        const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
        for (int k = 0; k <= kCameraSums; ++k)
        {
            double v = (k < kSums) ? (double)cam_sum[k < kSums ? k : 0] : (k == kCameraSums ? (double)view_cnt : 0.0);
#pragma unroll
            for (int d = kWave / 2; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
            if (lane == 0) cam_red[wave][k] = v;
        }
        __syncthreads();
        if (threadIdx.x <= kCameraSums)
            a.camera_partial[(size_t)view * a.camera_partial_stride + (size_t)blockIdx.x * kCameraRow + threadIdx.x] =
                (cam_red[0][threadIdx.x] + cam_red[1][threadIdx.x]) + (cam_red[2][threadIdx.x] + cam_red[3][threadIdx.x]);
        __syncthreads();  // (the next view of the round uses the array again)
    }
  }
    if (alive && (a.confidence_activation || a.texture_abs))
    {
        const int row = a.vp.index ? a.vp.index[i] : i;
        if ((uint32_t)row < (uint32_t)N)
        {
            if (a.confidence_activation && hit)  // (a point without a fragment has no gradient, and its row may not be packed)
            {
                const float s = a.packed[2 * (size_t)row + 1].x;  // d sigmoid(k x) / dx = k s (1 - s)
                gc            = gc * ((a.confidence_scale * s) * (1.f - s));
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
        // a later view of the batch: rows of points the view does not see are left as they are
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
            if (cnt > 0.f)  // gx, gy, gz are sums over the cnt fragments that got a position gradient
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
        // Without an index indirection confidence row 0 has just been written by thread 0 of this workgroup, which is
        // also the thread that adds the leak term; with one, rows are added to with atomics by every workgroup.
        __syncthreads();
        float leak_factor = 1.f;
        if (a.confidence_activation && a.add_leak)
        {
            const float s0 = sigmoid_canon(a.confidence_scale * a.vp.confidence[0]);  // (row 0 may not be packed)
            leak_factor    = (a.confidence_scale * s0) * (1.f - s0);
        }
        for (int v = 0; v < view_count; ++v)
        {
            sum_background_rows<kBlock>(a.background_rows + (size_t)v * a.background_rows_stride, a.num_background_rows, C,
                                        a.grad_background, a.grad_confidence, a.add_leak,
                                        (v > 0 || a.background_accumulate) ? 1 : 0, a.vp.index != nullptr,
                                        a.texture_abs ? a.background_raw : nullptr, leak_factor);
            __syncthreads();
        }
    }
}

// Adds the per-workgroup camera rows of one view to the pose row image_index (double) and the intrinsics row
// camera_index (fx, fy, cx, cy times K_gradient_factor, the skew column stays zero; the distortion columns where
// distortion is switched on), and the scaled fragment
// count to both count arrays, as src/lib/rendering/RenderBackward.cu:1418-1459 does per fragment with atomics.
__global__ void __launch_bounds__(kBlock) reduce_camera_kernel(const double* __restrict__ rows, int num_rows,
                                                                int image_index, int camera_index, float k_factor,
                                                                double* __restrict__ grad_pose,
                                                                float* __restrict__ grad_pose_count,
                                                                float* __restrict__ grad_intrinsics,
                                                                float* __restrict__ grad_intrinsics_count,
                                                                float pose_count_step, int with_distortion,
                                                                float distortion_factor)
{
    constexpr int kTerms = kCameraSums + 1;
    __shared__ double red[kBlock / kWave][kCameraRow];
    double acc[kTerms];
#pragma unroll
    for (int k = 0; k < kTerms; ++k) acc[k] = 0.0;
    for (int r = threadIdx.x; r < num_rows; r += kBlock)
    {
        const double* row = rows + (size_t)r * kCameraRow;
#pragma unroll
        for (int k = 0; k < kTerms; ++k) acc[k] += row[k];
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int k = 0; k < kTerms; ++k)
    {
        double v = acc[k];
#pragma unroll
        for (int d = kWave / 2; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
        if (lane == 0) red[wave][k] = v;
    }
    __syncthreads();
    if (threadIdx.x < kTerms)
    {
        const int k    = threadIdx.x;
        const double s = (red[0][k] + red[1][k]) + (red[2][k] + red[3][k]);
        if (k < 6)
        {
            if (grad_pose) grad_pose[6 * (size_t)image_index + k] += s;
        }
        else if (k < 10)
        {
            if (grad_intrinsics)
                grad_intrinsics[13 * (size_t)camera_index + (k - 6)] += (float)((double)k_factor * s);
        }
        else if (k < kCameraSums)
        {
            // the distortion columns with the weights of src/lib/rendering/RenderBackward.cu:1440-1455:
            // k3 x 0.25, k4..k6 and p1, p2 x 0.1, all x distortion_gradient_factor
            const int c       = k - 10;
            const double w8 = c < 2 ? 1.0 : c == 2 ? 0.25 : 0.1;
            if (grad_intrinsics && with_distortion)
                grad_intrinsics[13 * (size_t)camera_index + 5 + c] += (float)((double)distortion_factor * (s * w8));
        }
        else
        {
            // per fragment the reference adds 1/1024 to both counts in FULL_BLEND, but 1 to the pose count in
            // BILINEAR_BLEND (src/lib/rendering/RenderBackward.cu:1425,1458 and :3146,3174)
            if (grad_pose) grad_pose_count[image_index] += (float)(s * (double)pose_count_step);
            if (grad_intrinsics) grad_intrinsics_count[camera_index] += (float)(s / 1024.0);
        }
    }
}

// Rows divided by their counts: NormalizeGradientDevTensor<double,6> on the poses and NormalizeGradient<float,13> on the
// intrinsics (src/lib/rendering/PointRenderer.cu:1092-1109,1253-1308).
__global__ void __launch_bounds__(kBlock) normalize_camera_gradients_kernel(double* __restrict__ grad_pose,
                                                                             const float* __restrict__ pose_count,
                                                                             int num_poses,
                                                                             float* __restrict__ grad_intrinsics,
                                                                             const float* __restrict__ intrinsics_count,
                                                                             int num_cameras)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (grad_pose && i < num_poses)
    {
        const float c = pose_count[i];
        if (c > 0.f)
            for (int k = 0; k < 6; ++k) grad_pose[6 * (size_t)i + k] = grad_pose[6 * (size_t)i + k] / c;
    }
    if (grad_intrinsics && i < num_cameras)
    {
        const float c = intrinsics_count[i];
        if (c > 0.f)
            for (int k = 0; k < 13; ++k) grad_intrinsics[13 * (size_t)i + k] = grad_intrinsics[13 * (size_t)i + k] / c;
    }
}

// Division of the accumulated position gradient by the number of contributing fragments.
// mode 1: row i of the [N,4] buffer by count[i]. mode 2: the reference's literal behaviour, which walks the same
// memory as N vec3 (src/lib/rendering/PointRenderer.cu:1072-1090,1278-1279), i.e. flat elements 3i..3i+2 by count[i].
__global__ void __launch_bounds__(kBlock) normalize_point_gradient_kernel(float* __restrict__ grad_points,
                                                                           const float* __restrict__ count, int N,
                                                                           int mode)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const float c = count[i];
    if (!(c > 0.f)) return;
    const size_t base = (mode == 2 ? 3 : 4) * (size_t)i;
#pragma unroll
    for (int k = 0; k < 3; ++k) grad_points[base + k] = grad_points[base + k] / c;
}

}  // namespace vetrast
