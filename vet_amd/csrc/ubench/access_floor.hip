// The bare memory access pattern of the per-pixel backward kernel, without its arithmetic: one thread per list place
// streams the key and the transmittance, gathers the 32-byte descriptor record of the key's point and/or stores a
// 32-byte gradient record at the point's place. Run on the real lists of a frame (bench.py --access-floor) it tells how
// long the gathers and scatters alone take, i.e. what no rearrangement of the kernel's arithmetic can get below.
// A stand-alone measurement library: nothing in the product depends on it.
#include <hip/hip_runtime.h>

#include <cstdint>

// what: bit 0 = gather the descriptor records, bit 1 = store the gradient records
__global__ void __launch_bounds__(256) access_floor_kernel(const uint64_t* __restrict__ fragments, const float* __restrict__ transmittance,
                                                           const float4* __restrict__ packed, float4* __restrict__ partial,
                                                           uint32_t F, uint32_t N, uint32_t first1, uint32_t first2, uint32_t first3, int what)
{
    const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= F) return;
    const uint32_t id = (uint32_t)fragments[j];
    const float T     = transmittance[j];
    if (id >= N) return;
    float4 t4 = make_float4(1.f, 1.f, 1.f, 1.f), c4 = t4;
    if (what & 1)
    {
        t4 = packed[2 * (size_t)id];
        c4 = packed[2 * (size_t)id + 1];
    }
    const uint32_t layer = (j >= first1) + (j >= first2) + (j >= first3);  // list places are laid out layer after layer
    const float Tc       = T * c4.x;
    const float4 lo = make_float4(Tc * t4.x, Tc * t4.y, Tc * t4.z, Tc * t4.w), hi = make_float4(t4.x + t4.y, t4.z, t4.w, 0.f);
    float4* rec = partial + 2 * ((size_t)layer * N + id);
    if (what & 2)
    {
        rec[0] = lo;
        rec[1] = hi;
    }
    else if (lo.x + hi.x == 123.456f)  // keeps the loads alive
        rec[0] = lo;
}

extern "C" int access_floor_run(const void* fragments, const void* transmittance, const void* packed, void* partial, uint32_t F,
                                uint32_t N, uint32_t first1, uint32_t first2, uint32_t first3, int what, void* stream)
{
    if (F == 0) return 0;
    hipLaunchKernelGGL(access_floor_kernel, dim3((F + 255) / 256), dim3(256), 0, (hipStream_t)stream, (const uint64_t*)fragments,
                       (const float*)transmittance, (const float4*)packed, (float4*)partial, F, N, first1, first2, first3, what);
    return (int)hipGetLastError();
}
