// Per-bin list building: the last step of the forward binning (see forward_kernels.h for the whole scheme).
#pragma once
#include "common.h"
#include "forward_kernels.h"
#include "sort_kernels.h"

namespace vetrast
{
// One workgroup per bin turns the bin's records into sorted per-pixel lists: count per pixel and rank inside the pixel
// with LDS atomics, scan of the (at most 256) counts, keys scattered to list start + rank, lists sorted by the waves
// with the same register networks as the stand-alone sort pass, and the whole stretch written out coalesced. That
// holds for bins of up to kBuildCap records, which is what the bin sizes are chosen for. Bigger bins (far more points
// in one place than the layer's average) stream their records twice from global memory instead and sort their lists in
// place in the fragment buffer.
constexpr int kBuildPerThread = 8;
constexpr int kBuildCap       = kBlock * kBuildPerThread;  // 2048 records = 16 KB of keys in LDS

struct BuildPass
{
    const uint32_t* bin_offsets;  // [bins + 1] exclusive scan of the bin counts
    const uint4* binned;
    uint32_t* offsets;    // [P + 1] per pixel: start of its list; [P] = fragments of the view
    uint64_t* fragments;
    uint8_t* list_is_cut;    // [P]
    LayerTable ly;
    uint32_t num_bins;
    int K;
};

__global__ void __launch_bounds__(kBlock) bin_build_kernel(BuildPass a)
{
    __shared__ uint32_t s_cnt[kTilePixels];
    __shared__ uint32_t s_prefix[kTilePixels];
    __shared__ uint32_t s_wave_tot[kBlock / kWave];
    __shared__ uint8_t s_src_lane[kBlock / kWave][kWave];
    __shared__ uint64_t s_keys[kBuildCap];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t bin = a.num_bins - 1u - blockIdx.x;  // coarse layers first
    int l              = 0;
#pragma unroll
    for (int k = 1; k < VETRAST_MAX_LAYERS; ++k)
        if (k < a.ly.L && bin >= a.ly.bin_base[k]) l = k;
    const int shift       = a.ly.bin_shift[l];
    const uint32_t pixels = 1u << shift;  // pixels of this bin
    const uint32_t q0     = a.ly.base[l] + ((bin - a.ly.bin_base[l]) << shift);
    const uint32_t begin  = a.bin_offsets[bin];
    const uint32_t n      = a.bin_offsets[bin + 1] - begin;
    const uint4* recs     = a.binned + begin;
    const bool in_lds     = n <= (uint32_t)kBuildCap;
    s_cnt[tid] = 0u;
    __syncthreads();

    // ---- count per pixel; the LDS atomic also hands every record its rank inside the pixel
    uint64_t key[kBuildPerThread];
    uint32_t where[kBuildPerThread];  // pixel in bin | rank in pixel << 8
    if (in_lds)
    {
#pragma unroll
        for (int k = 0; k < kBuildPerThread; ++k)
        {
            const uint32_t r = (uint32_t)(k * kBlock + tid);
            where[k]         = 0xFFFFFFFFu;
            key[k]           = 0ull;
            if (r < n)
            {
                const uint4 rec     = recs[r];
                const uint32_t px   = rec.z & (pixels - 1u);
                const uint32_t rank = atomicAdd(&s_cnt[px], 1u);
                key[k]              = ((uint64_t)rec.y << 32) | rec.x;
                where[k]            = px | (rank << 8);
            }
        }
    }
    else
    {
        for (uint32_t r0 = 0; r0 < n; r0 += kBlock * 4)
        {
            uint32_t px[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const uint32_t r = r0 + k * kBlock + tid;
                px[k]            = r < n ? (recs[r].z & (pixels - 1u)) : 0xFFFFFFFFu;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (px[k] != 0xFFFFFFFFu) atomicAdd(&s_cnt[px[k]], 1u);
        }
    }
    __syncthreads();

    // ---- scan of the pixel counts: list starts
    const uint32_t c    = s_cnt[tid];
    const uint32_t incl = wave_inclusive_scan(c, lane);
    if (lane == kWave - 1) s_wave_tot[wave] = incl;
    __syncthreads();
    uint32_t start = incl - c;
    for (int k = 0; k < wave; ++k) start += s_wave_tot[k];
    s_prefix[tid] = start;
    if ((uint32_t)tid < pixels)
    {
        const uint32_t q = q0 + tid;
        a.offsets[q]     = begin + start;
        if (bin == a.num_bins - 1u && (uint32_t)tid == pixels - 1u) a.offsets[q + 1] = begin + n;
        // one byte per pixel: does the top-K cut drop fragments here? The backward per-point kernel only has to look up
        // the K-th key of a pixel where this is set.
        a.list_is_cut[q] = (a.K > 0 && c > (uint32_t)a.K) ? 1 : 0;
    }
    __syncthreads();

    // wave w sorts the lists of its quarter of the bin's pixels
    const uint32_t per_wave = pixels >> 2;  // >= 1
    uint32_t list_off = 0, list_len = 0;
    if ((uint32_t)lane < per_wave)
    {
        const uint32_t px = wave * per_wave + lane;
        list_off          = s_prefix[px];
        list_len          = s_cnt[px];
    }
    if (in_lds)
    {
#pragma unroll
        for (int k = 0; k < kBuildPerThread; ++k)
            if (where[k] != 0xFFFFFFFFu) s_keys[s_prefix[where[k] & 0xFF] + (where[k] >> 8)] = key[k];
        __syncthreads();
        sort_wave_lists(s_keys, s_src_lane[wave], list_off, list_len, lane, a.K);
        __syncthreads();
        for (uint32_t r = tid; r < n; r += kBlock) a.fragments[begin + r] = s_keys[r];
    }
    else
    {
        // second pass over the records: a fresh cursor per pixel hands out the places inside the list (any order is
        // fine, the lists are sorted afterwards)
        __syncthreads();  // every wave has read its list lengths
        s_cnt[tid] = 0u;
        __syncthreads();
        for (uint32_t r0 = 0; r0 < n; r0 += kBlock * 4)
        {
            uint4 rec[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const uint32_t r = r0 + k * kBlock + tid;
                rec[k]           = r < n ? recs[r] : make_uint4(0u, 0u, 0xFFFFFFFFu, 0u);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                if (rec[k].z == 0xFFFFFFFFu) continue;
                const uint32_t px   = rec[k].z & (pixels - 1u);
                const uint32_t rank = atomicAdd(&s_cnt[px], 1u);
                a.fragments[begin + s_prefix[px] + rank] = ((uint64_t)rec[k].y << 32) | rec[k].x;
            }
        }
        __threadfence_block();  // the keys other waves stored are read below
        __syncthreads();
        sort_wave_lists(a.fragments + begin, s_src_lane[wave], list_off, list_len, lane, a.K);
    }
}

}  // namespace vetrast
