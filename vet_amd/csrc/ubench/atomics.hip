// Throughput of scattered global atomics, loads and stores (4, 8 and 32 bytes) on one GPU: the figures the binning design rests on
// (one returning atomic per wave group and bin instead of one per fragment). A stand-alone program, not part of the
// library: built by vet_amd/build.py next to it, run by `python bench.py --atomics-ubench`.
//
// 2 M threads x 4 operations on pseudo-random 4-byte addresses out of 32 400 (one counter per 16x16 tile of the four
// 1080p layers), 2 754 000 (one per pixel) or 64 M (beyond every cache); best of 5 launches each.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#define CK(x)                                                                      \
    do                                                                             \
    {                                                                              \
        hipError_t e = (x);                                                        \
        if (e != hipSuccess)                                                       \
        {                                                                          \
            printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__);   \
            return 1;                                                              \
        }                                                                          \
    } while (0)

__device__ __forceinline__ uint32_t hash32(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

enum Mode
{
    kAtomicReturning = 0,
    kAtomicNoReturn,
    kStore4,
    kLoad4,
    kStore8,
    kStore32,
    kLoad32,
    kModes
};

template <int MODE>
__global__ void scattered_ops(uint32_t* words, uint32_t num_words, uint32_t* out, int n, int per_thread)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint32_t acc = 0;
    for (int k = 0; k < per_thread; ++k)
    {
        const uint32_t a = hash32(i * 4 + k) % num_words;
        if (MODE == kAtomicReturning) acc += atomicAdd(&words[a], 1u);
        if (MODE == kAtomicNoReturn) atomicAdd(&words[a], 1u);
        if (MODE == kStore4) words[a] = i;
        if (MODE == kLoad4) acc += words[a];
        if (MODE == kStore8) ((uint64_t*)words)[a >> 1] = i;
        if (MODE == kStore32)
        {
            const float4 v                     = make_float4(i, i, i, i);
            ((float4*)words)[(a >> 3) * 2]     = v;
            ((float4*)words)[(a >> 3) * 2 + 1] = v;
        }
        if (MODE == kLoad32)
        {
            const float4 lo = ((const float4*)words)[(a >> 3) * 2], hi = ((const float4*)words)[(a >> 3) * 2 + 1];
            acc += __float_as_uint(lo.x + hi.w);
        }
    }
    if (MODE == kAtomicReturning || MODE == kLoad4 || MODE == kLoad32) out[i] = acc;
}

int main()
{
    const int n = 2000000, per_thread = 4;
    const char* names[kModes] = {"atomic add, returning", "atomic add, no return", "store 4 B", "load 4 B", "store 8 B", "store 32 B", "load 32 B"};
    const uint32_t sizes[]    = {32400u, 2754000u, 64000000u};
    uint32_t *words, *out;
    CK(hipMalloc(&words, (size_t)64000000u * 4));
    CK(hipMalloc(&out, (size_t)n * 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const dim3 g((n + 255) / 256), b(256);
    for (uint32_t num_words : sizes)
        for (int mode = 0; mode < kModes; ++mode)
        {
            CK(hipMemset(words, 0, (size_t)num_words * 4));
            float best = 1e9f;
            for (int rep = 0; rep < 5; ++rep)
            {
                CK(hipEventRecord(e0));
                switch (mode)
                {
                    case kAtomicReturning: hipLaunchKernelGGL(scattered_ops<kAtomicReturning>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                    case kAtomicNoReturn: hipLaunchKernelGGL(scattered_ops<kAtomicNoReturn>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                    case kStore4: hipLaunchKernelGGL(scattered_ops<kStore4>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                    case kLoad4: hipLaunchKernelGGL(scattered_ops<kLoad4>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                    case kStore8: hipLaunchKernelGGL(scattered_ops<kStore8>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                    case kStore32: hipLaunchKernelGGL(scattered_ops<kStore32>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                    default: hipLaunchKernelGGL(scattered_ops<kLoad32>, g, b, 0, 0, words, num_words, out, n, per_thread); break;
                }
                CK(hipEventRecord(e1));
                CK(hipEventSynchronize(e1));
                float ms;
                CK(hipEventElapsedTime(&ms, e0, e1));
                if (ms < best) best = ms;
            }
            printf("addresses=%9u  %-22s  %8.1f us  %7.2f Gops/s\n", num_words, names[mode], best * 1e3, n * (double)per_thread / best / 1e6);
            fflush(stdout);
        }
    // one address: what a counter every thread hits costs per operation
    {
        CK(hipMemset(words, 0, 4));
        float best = 1e9f;
        for (int rep = 0; rep < 5; ++rep)
        {
            CK(hipEventRecord(e0));
            hipLaunchKernelGGL(scattered_ops<kAtomicNoReturn>, dim3(64), b, 0, 0, words, 1u, out, 64 * 256, per_thread);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (ms < best) best = ms;
        }
        printf("addresses=%9u  %-22s  %8.1f us  %7.2f ns per wave instruction (64 lanes, one address)\n", 1u, "atomic add, no return", best * 1e3,
               best * 1e6 / (64.0 * 256 / 64 * per_thread));
    }
    CK(hipFree(words));
    CK(hipFree(out));
    return 0;
}
