// Backward kernels: gradients of the blend with respect to descriptors, confidence, background and point positions.
#pragma once
#include "common.h"

namespace vetrast
{
struct BackwardPass
{
    const uint32_t* offsets;
    const uint64_t* fragments;
    const float* transmittance;  // per kept fragment, saved by the forward blend
    const float* weight;         // per pixel: transmittance behind the last kept fragment
    const int32_t* index;
    const float4* packed;
    const float4* position;
    const float* background;
    const DeviceView* view;
    const float* grad_out[VETRAST_MAX_LAYERS];  // already offset to this view
    const float* out[VETRAST_MAX_LAYERS];       // forward result, already offset to this view
    float* grad_texture;     // [C,N]
    float* grad_confidence;  // [N]
    float* grad_background;  // [C]
    float* grad_points;      // [N,4] or null
    float* grad_point_count; // [N]
    LayerTable ly;
    uint32_t P;
    int N;
    int K;
    int use_environment_map;
    int need_point_gradient;
    int quirk_background_confidence_leak;
};

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

// One thread per pixel, all layers of a view in one launch. The list is walked back to front with the transmittance
// T_j the forward pass stored, so the reference's inner loop over all fragments in front
// (src/lib/rendering/RenderBackward.cu:1160-1178, n(n-1)/2 atomics per pixel) becomes a running suffix sum:
//   S_j         = sum_{i>j} sum_ci g[ci] * t_i[ci] * T_i * c_i          (the background counts as the last fragment)
//   d conf_j    = T_j * (t_j . g)  -  S_j / (1 - c_j + 1e-9)
//   d tex_j[ci] = T_j * c_j * g[ci]
// which is the same sum in a different order. Position gradient: the neighbour-difference heuristic of
// src/lib/rendering/RenderBackward.cu:1346-1377 pushed through the pinhole chain of
// src/lib/rendering/PointRendererHelper.h:317-372 (zero distortion), J_point = R.
// Counterpart of BlendBackwards2<C> (src/lib/rendering/RenderBackward.cu:1083-1513).
template <int C>
__global__ void __launch_bounds__(kBlock) blend_backward_kernel(BackwardPass a)
{
    const uint32_t q  = blockIdx.x * blockDim.x + threadIdx.x;
    const bool active = q < a.P;
    float bg_grad[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) bg_grad[ci] = 0.f;
    float leak = 0.f;

    if (active)
    {
        const int l          = layer_of_pixel(a.ly, q);
        const int lw = a.ly.w[l], lh = a.ly.h[l];
        const size_t plane   = (size_t)lw * lh;
        const uint32_t local = q - a.ly.base[l];
        const int gy = (int)(local / (uint32_t)lw), gx = (int)(local - (uint32_t)gy * lw);
        const float* G = a.grad_out[l];
        float g[C];
#pragma unroll
        for (int ci = 0; ci < C; ++ci) g[ci] = G[ci * plane + local];

        const uint32_t off = a.offsets[q];
        uint32_t n         = a.offsets[q + 1] - off;
        if (a.K > 0) n = min(n, (uint32_t)a.K);

        float S = 0.f;
        if (!a.use_environment_map)
        {
            const float Tn = a.weight[q];
            float dot      = 0.f;
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                const float bgc = a.background[ci];
                bg_grad[ci]     = (Tn * 1.f) * g[ci];
                dot += bgc * g[ci];
                S += ((g[ci] * bgc) * Tn) * 1.f;
            }
            if (a.quirk_background_confidence_leak) leak = dot * Tn;
        }

        // neighbour samples for the position heuristic, shared by every fragment of the pixel
        const int edge      = min(min(gx, gy), min(lw - 1 - gx, lh - 1 - gy));
        const bool do_point = a.need_point_gradient && a.grad_points && edge > 2 && n > 0;
        float Ix0[C], Ix1[C], Iy0[C], Iy1[C], Gx0[C], Gx1[C], Gy0[C], Gy1[C];
        float cfx = 0.f, cfy = 0.f, cs = 0.f;
        if (do_point)
        {
            const float* I = a.out[l];
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                const float* Ic = I + ci * plane + local;
                const float* Gc = G + ci * plane + local;
                Ix0[ci] = Ic[-1];
                Ix1[ci] = Ic[1];
                Iy0[ci] = Ic[-lw];
                Iy1[ci] = Ic[lw];
                Gx0[ci] = Gc[-1];
                Gx1[ci] = Gc[1];
                Gy0[ci] = Gc[-lw];
                Gy1[ci] = Gc[lw];
            }
            const float scale = powf(0.5f, (float)l);
            cfx               = a.view->crop[0] * scale;
            cfy               = a.view->crop[1] * scale;
            cs                = a.view->crop[4] * scale;
        }

        const uint64_t* list = a.fragments + off;
        const float* Tlist   = a.transmittance + off;
        for (int j = (int)n - 1; j >= 0; --j)
        {
            const int id = (int)(uint32_t)list[j];
            if ((uint32_t)id >= (uint32_t)a.N) continue;  // guards the gathers; never true for a valid workspace
            const int ti = a.index ? a.index[id] : id;
            if ((uint32_t)ti >= (uint32_t)a.N) continue;
            const float4 t4  = a.packed[2 * (size_t)ti];
            const float c    = a.packed[2 * (size_t)ti + 1].x;
            const float T    = Tlist[j];
            const float t[4] = {t4.x, t4.y, t4.z, t4.w};
            float dot = 0.f, x = 0.f;
            const float Tc = T * c;
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                atomicAdd(&a.grad_texture[(size_t)ci * a.N + ti], Tc * g[ci]);
                dot += t[ci] * g[ci];
                x += ((g[ci] * t[ci]) * T) * c;
            }
            atomicAdd(&a.grad_confidence[ti], dot * T - S / ((1.f - c) + 1e-9f));
            S += x;

            if (do_point)
            {
                float dR_dpx = 0.f, dR_dpy = 0.f;
#pragma unroll
                for (int ci = 0; ci < C; ++ci)
                {
                    const float d_x0 = -(t[ci] - Ix0[ci]) * Gx0[ci];
                    const float d_x1 = (t[ci] - Ix1[ci]) * Gx1[ci];
                    const float d_y0 = -(t[ci] - Iy0[ci]) * Gy0[ci];
                    const float d_y1 = (t[ci] - Iy1[ci]) * Gy1[ci];
                    dR_dpx += 0.5f * (d_x0 + d_x1);
                    dR_dpy += 0.5f * (d_y0 + d_y1);
                }
                const float gxp = dR_dpx / (float)C, gyp = dR_dpy / (float)C;
                const DeviceView& cam = *a.view;
                const float4 p        = a.position[id];
                const float vx = ((cam.r[0] * p.x + cam.r[1] * p.y) + cam.r[2] * p.z) + cam.t[0];
                const float vy = ((cam.r[3] * p.x + cam.r[4] * p.y) + cam.r[5] * p.z) + cam.t[1];
                const float vz = ((cam.r[6] * p.x + cam.r[7] * p.y) + cam.r[8] * p.z) + cam.t[2];
                float gp0 = 0.f, gp1 = 0.f, gp2 = 0.f;
                if (vz > 0.f)
                {
                    const float ar = cam.rot[0] * gxp + cam.rot[2] * gyp;
                    const float br = cam.rot[1] * gxp + cam.rot[3] * gyp;
                    const float a2 = cfx * ar;
                    const float b2 = cs * ar + cfy * br;
                    const float d0 = cam.fx * a2;
                    const float d1 = cam.s * a2 + cam.fy * b2;
                    const float iz = 1.f / vz;
                    const float e0 = iz * d0, e1 = iz * d1;
                    const float e2 = (-vx * iz * iz) * d0 + (-vy * iz * iz) * d1;
                    gp0            = (cam.r[0] * e0 + cam.r[3] * e1) + cam.r[6] * e2;
                    gp1            = (cam.r[1] * e0 + cam.r[4] * e1) + cam.r[7] * e2;
                    gp2            = (cam.r[2] * e0 + cam.r[5] * e1) + cam.r[8] * e2;
                }
                float* gpt = a.grad_points + 4 * (size_t)id;
                atomicAdd(gpt + 0, gp0);
                atomicAdd(gpt + 1, gp1);
                atomicAdd(gpt + 2, gp2);
                atomicAdd(a.grad_point_count + id, 1.f);
            }
        }
    }

    // Every pixel adds to the same C background values: reduce over the wave first, one atomic per wave and channel
    // (the reference issues one atomic per pixel and channel, src/lib/rendering/RenderBackward.cu:1150-1152).
    if (!a.use_environment_map)
    {
        const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
        for (int ci = 0; ci < C; ++ci)
        {
            const float s = wave_sum(bg_grad[ci]);
            if (lane == 0 && s != 0.f) atomicAdd(&a.grad_background[ci], s);
        }
        if (a.quirk_background_confidence_leak)
        {
            const float s = wave_sum(leak);
            if (lane == 0 && s != 0.f) atomicAdd(&a.grad_confidence[0], s);
        }
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
