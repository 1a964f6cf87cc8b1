// Per-pixel sort of the fragment lists by the 64-bit key (depth bits << 32 | point id), ascending, with the top-K cut.
//
// A wave owns up to 64 consecutive pixels of a bin, whose lists are one contiguous stretch of the fragment buffer (or of
// the bin's copy in LDS). Lists are grouped by padded power-of-two length m = 2,4,...,64 and 64/m lists are
// sorted at a time by one bitonic network held in registers (one key per lane, partner exchange by lane shuffles).
// Lists longer than 64 keep the K smallest keys with a streaming wave-wide selection, or are sorted in place in
// global memory when no cut applies.
//
// Counterpart of SegmentedSortBitonicHelper2 and its kernels (src/lib/rendering/AlphaListSort.cu:601-703): that one
// buckets lists into <=32 / <=256 / <=1024 / <=4096 with two extra passes and a device->host read of the bucket sizes,
// sorts by depth only and leaves lists beyond 4096 entries partly unsorted (:290). Here the order is total
// (depth, then point id) and exact for every length.
#pragma once
#include "common.h"

namespace vetrast
{
__device__ __forceinline__ uint64_t shfl_u64(uint64_t v, int src)
{
    const uint32_t lo = __shfl((uint32_t)v, src, kWave);
    const uint32_t hi = __shfl((uint32_t)(v >> 32), src, kWave);
    return ((uint64_t)hi << 32) | lo;
}

// One compare-exchange stage with partner lane ^ M: lanes for which keep_min holds keep the smaller key of the pair.
template <int M>
__device__ __forceinline__ uint64_t exchange(uint64_t key, int lane, bool keep_min)
{
    const uint32_t lo    = lane_xor<M>((uint32_t)key, lane);
    const uint32_t hi    = lane_xor<M>((uint32_t)(key >> 32), lane);
    const uint64_t other = ((uint64_t)hi << 32) | lo;
    const bool take      = keep_min ? (other < key) : (other > key);
    return take ? other : key;
}

template <int K2, int J>
__device__ __forceinline__ uint64_t halving_steps(uint64_t key, int lane)
{
    if constexpr (J >= 1)
    {
        key = exchange<J>(key, lane, (lane & J) == 0);
        key = halving_steps<K2, (J >> 1)>(key, lane);
    }
    return key;
}

template <int K2, int MAXK>
__device__ __forceinline__ uint64_t bitonic_stages(uint64_t key, int lane)
{
    if constexpr (K2 <= MAXK)
    {
        key = exchange<K2 - 1>(key, lane, (lane & (K2 >> 1)) == 0);  // mirror step inside every block of K2 lanes
        key = halving_steps<K2, (K2 >> 2)>(key, lane);
        key = bitonic_stages<K2 * 2, MAXK>(key, lane);
    }
    return key;
}

// Ascending bitonic sort of every aligned group of 2^LOG lanes (all-ascending form: a mirror step, then halving
// steps), LOG = 1..6.
template <int LOG>
__device__ __forceinline__ uint64_t bitonic_sort_groups(uint64_t key, int lane)
{
    return bitonic_stages<2, (1 << LOG)>(key, lane);
}

// Halving steps only: sorts a bitonic sequence held by the 64 lanes.
__device__ __forceinline__ uint64_t bitonic_merge64(uint64_t key, int lane)
{
    return halving_steps<64, 32>(key, lane);
}

// Sort `count` lists of class LOG (2^(LOG-1) < n <= 2^LOG) found in the wave; src_lane[r] is the lane that owns the r-th.
template <int LOG>
__device__ __forceinline__ void sort_class(uint64_t* fragments, const uint8_t* src_lane, int count,
                                           uint32_t off, uint32_t n, int lane, int K)
{
    constexpr int m        = 1 << LOG;
    constexpr int per_pass = kWave >> LOG;
    const int g = lane >> LOG, e = lane & (m - 1);
    for (int first = 0; first < count; first += per_pass)
    {
        const int li     = first + g;
        const bool valid = li < count;
        const int src    = valid ? src_lane[li] : 0;
        const uint32_t o = __shfl(off, src, kWave);
        uint32_t nn      = __shfl(n, src, kWave);
        if (!valid) nn = 0;
        uint64_t key = ((uint32_t)e < nn) ? fragments[o + e] : kInfKey;
        key          = bitonic_sort_groups<LOG>(key, lane);
        const uint32_t keep = (K > 0) ? min(nn, (uint32_t)K) : nn;
        if ((uint32_t)e < keep) fragments[o + e] = key;
    }
}

// K smallest keys (K <= 64) of a list longer than 64, sorted, written to its first K places. The wave keeps the 64
// smallest keys seen so far in sorted order; a chunk of 64 further keys is looked at only if one of them beats the
// current K-th smallest.
__device__ __forceinline__ void select_smallest(uint64_t* list, uint32_t n, int lane, int K)
{
    uint64_t best = list[lane];  // n > 64
    best          = bitonic_sort_groups<6>(best, lane);
    for (uint32_t base = kWave; base < n; base += kWave)
    {
        const uint64_t v   = (base + lane < n) ? list[base + lane] : kInfKey;
        const uint64_t thr = shfl_u64(best, K - 1);
        if (__ballot(v < thr) == 0ull) continue;
        const uint64_t sorted = bitonic_sort_groups<6>(v, lane);
        const uint64_t mirror = shfl_u64(sorted, kWave - 1 - lane);
        best                  = (mirror < best) ? mirror : best;  // 64 smallest of the 128, a bitonic sequence
        best                  = bitonic_merge64(best, lane);
    }
    if (lane < K) list[lane] = best;
}

// In-place bitonic sort of a list of any length in global memory by one wave; places beyond n act as +infinity and
// are never touched. Slow path: only lists longer than 64 with no usable cut come here.
__device__ __forceinline__ void sort_in_memory(uint64_t* list, uint32_t n, int lane)
{
    uint32_t m = 1;
    while (m < n) m <<= 1;
    const uint32_t half = m >> 1;
    for (uint32_t k = 2; k <= m; k <<= 1)
    {
        const uint32_t hk = k >> 1;
        for (uint32_t p = lane; p < half; p += kWave)
        {
            const uint32_t blk = p / hk, r = p % hk;
            const uint32_t i = blk * k + r, j = blk * k + (k - 1 - r);
            if (j < n)
            {
                const uint64_t a = list[i], b = list[j];
                if (b < a)
                {
                    list[i] = b;
                    list[j] = a;
                }
            }
        }
        __threadfence_block();
        for (uint32_t jj = k >> 2; jj >= 1; jj >>= 1)
        {
            for (uint32_t p = lane; p < half; p += kWave)
            {
                const uint32_t i = (p / jj) * 2 * jj + (p % jj), j = i + jj;
                if (j < n)
                {
                    const uint64_t a = list[i], b = list[j];
                    if (b < a)
                    {
                        list[i] = b;
                        list[j] = a;
                    }
                }
            }
            __threadfence_block();
        }
    }
}

// Sorts a list of 64 < n <= 64 * CH keys by one wave with the keys in registers, CH keys per lane (chunk q holds places
// 64 q .. 64 q + 63; places beyond n act as +infinity). Every chunk is sorted by the 64-lane network, then chunks are
// merged pairwise, level by level, in the all-ascending form of the bitonic network: the mirror step and the halving
// steps over 64 or more places pair whole chunks register against register (the mirror step with the partner chunk
// reversed across the wave), the last six halving steps of a level run inside every chunk. One load and one store per key.
template <int CH>
__device__ __forceinline__ void sort_in_registers(uint64_t* list, uint32_t n, int lane)
{
    uint64_t c[CH];
#pragma unroll
    for (int q = 0; q < CH; ++q)
    {
        const uint32_t idx = q * kWave + lane;
        c[q]               = idx < n ? list[idx] : kInfKey;
    }
#pragma unroll
    for (int q = 0; q < CH; ++q) c[q] = bitonic_sort_groups<6>(c[q], lane);
    auto reversed = [&](uint64_t v) {
        const uint32_t lo = lane_xor<63>((uint32_t)v, lane), hi = lane_xor<63>((uint32_t)(v >> 32), lane);
        return ((uint64_t)hi << 32) | lo;
    };
#pragma unroll
    for (int w = 2; w <= CH; w <<= 1)  // w chunks per block of this level
    {
#pragma unroll
        for (int q = 0; q < CH; ++q)
            if ((q % w) < w / 2)
            {
                const int p        = q - (q % w) + (w - 1 - (q % w));
                const uint64_t r   = reversed(c[p]);
                const uint64_t mn  = r < c[q] ? r : c[q], mx = r < c[q] ? c[q] : r;
                c[q]               = mn;
                c[p]               = reversed(mx);
            }
#pragma unroll
        for (int d = w / 4; d >= 1; d >>= 1)
#pragma unroll
            for (int q = 0; q < CH; ++q)
                if ((q & d) == 0)
                {
                    const uint64_t x = c[q], y = c[q + d];
                    c[q]             = y < x ? y : x;
                    c[q + d]         = y < x ? x : y;
                }
#pragma unroll
        for (int q = 0; q < CH; ++q) c[q] = bitonic_merge64(c[q], lane);
    }
#pragma unroll
    for (int q = 0; q < CH; ++q)
    {
        const uint32_t idx = q * kWave + lane;
        if (idx < n) list[idx] = c[q];
    }
}

constexpr uint32_t kRegisterSortKeys = 256;  // longest list sort_wave_lists sorts in registers

// Sorts the lists of one wave: lane i holds the start `off` (an index into `fragments`) and the length `n` of its list
// (n = 0 for lanes without a list). `fragments` may point to global memory or to LDS. Lists that have to be sorted in
// full and hold more than kRegisterSortKeys and up to `skip_longer` keys are left alone: the caller sorts them by other
// means.
__device__ __forceinline__ void sort_wave_lists(uint64_t* fragments, uint8_t* src_lane, uint32_t off, uint32_t n,
                                                int lane, int K, uint32_t skip_longer = 0)
{
    // class = ceil(log2(n)) for 2 <= n <= 64, 0 for n <= 1 (nothing to do), 7 for n > 64
    int cls = 0;
    if (n > 64)
        cls = 7;
    else if (n > 1)
        cls = 32 - __clz((int)(n - 1));

    const uint64_t lanes_below = (1ull << lane) - 1ull;
#pragma unroll
    for (int c = 1; c <= 6; ++c)
    {
        const uint64_t mask = __ballot(cls == c);
        if (mask == 0ull) continue;
        if (cls == c) src_lane[__popcll(mask & lanes_below)] = (uint8_t)lane;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int count = __popcll(mask);
        switch (c)
        {
            case 1: sort_class<1>(fragments, src_lane, count, off, n, lane, K); break;
            case 2: sort_class<2>(fragments, src_lane, count, off, n, lane, K); break;
            case 3: sort_class<3>(fragments, src_lane, count, off, n, lane, K); break;
            case 4: sort_class<4>(fragments, src_lane, count, off, n, lane, K); break;
            case 5: sort_class<5>(fragments, src_lane, count, off, n, lane, K); break;
            default: sort_class<6>(fragments, src_lane, count, off, n, lane, K); break;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    uint64_t long_mask = __ballot(cls == 7);
    while (long_mask != 0ull)
    {
        const int src = __ffsll((unsigned long long)long_mask) - 1;
        long_mask &= long_mask - 1ull;
        const uint32_t o  = __shfl(off, src, kWave);
        const uint32_t nn = __shfl(n, src, kWave);
        if (K > 0 && K <= kWave)
            select_smallest(fragments + o, nn, lane, K);
        else if (nn <= 2 * kWave)
            sort_in_registers<2>(fragments + o, nn, lane);
        else if (nn <= kRegisterSortKeys)
            sort_in_registers<4>(fragments + o, nn, lane);
        else if (nn <= skip_longer)
            continue;  // the caller sorts lists of this length with the whole workgroup
        else
            sort_in_memory(fragments + o, nn, lane);
    }
}

}  // namespace vetrast
