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
//
// A bin that was sorted in LDS is blended right there as well (BlendMulti, src/lib/rendering/RenderForward.cu:1303-1357):
// all 256 threads gather the descriptor records of a stretch of kept fragments into an LDS stage (one independent
// gather per lane), then the thread that owns a pixel walks its fragments of that stretch front to back in exactly the
// reference's order: out += (T*c)*t, T = (1-c)*T. The transmittance in front of every fragment is parked in the high
// half of its key in LDS (the depth bits have gone out to the fragment buffer by then) and written out coalesced.
// Bins that did not fit walk their lists in the fragment buffer, one thread per pixel.
//
// The LDS capacity is a trade: 2048 records (16 KB of keys, 30 KB in all) kept all but 58 of config 3's 14 400 bins in
// LDS but let only 5 workgroups share a CU, and a workgroup's life is a chain of memory round trips; with 1024 records
// (19.8 KB in all, 8 workgroups per CU, the most the hardware holds) 608 bins stream instead and the pass is still 12 % faster there and 20 % faster
// on the 10 M point cloud.
constexpr int kBuildPerThread = 4;
constexpr int kBuildCap       = kBlock * kBuildPerThread;  // 1024 records = 8 KB of keys in LDS
static_assert(kPrimaryCapSmall >= kBuildCap, "a bin built in LDS must find all its records in its own room");
constexpr int kStage          = 256;                       // descriptor records staged per round (8 KB)

struct BuildPass
{
    const uint32_t* bin_offsets;  // [bins + 1] exclusive scan of the bin counts
    const uint4* primary;         // the bins' rooms (LayerTable::room_base): the first room_cap[l] records of every bin
    const uint4* binned;          // compact array: record r >= room_cap[l] of a bin sits at bin_offsets[bin] + r
    int compact_records;          // both hold 8-byte records (depth bits, point id << 8 | pixel in bin), see ScatterTargets
    uint32_t* offsets;    // [P + 1] per pixel: start of its list; [P] = fragments of the view
    uint64_t* fragments;
    uint8_t* list_is_cut;   // [P]
    uint64_t* last_key;     // [P] where list_is_cut: key of the last fragment that took part in the blend (0: none did)
    uint32_t* kept;         // [P] fragments of the pixel that took part in the blend
    // blending
    const float2* projected;  // BILINEAR_BLEND only: [N] where a point projects to at layer 0 (the alpha of a fragment
                              // depends on it)
    const int32_t* index;
    const float4* packed;
    const float* background;
    float* transmittance;  // per fragment, null unless the backward pass will run
    float* weight;         // per pixel
    float* out[VETRAST_MAX_LAYERS];       // already offset to this view
    float* out_mask[VETRAST_MAX_LAYERS];  // already offset to this view, or null
    float* out_weight[VETRAST_MAX_LAYERS];  // the same
    LayerTable ly;
    uint32_t num_bins;
    int N;
    int K;
    int use_environment_map;
    float mask_value;
    float depth_accept;  // FUZZY_BLEND: depth range of a bucket
};

// Alpha of a fragment: the point's confidence, in BILINEAR_BLEND times the bilinear weight of the pixel's corner at the
// point's position in this layer (BlendMultiBilinear, src/lib/rendering/RenderForward.cu:1586-1613). The position is
// the projection the scatter pass stored, so the weight is reproduced bit for bit.
template <bool BILINEAR>
__device__ __forceinline__ float fragment_alpha(const BuildPass& a, int l, uint32_t low, float confidence)
{
    if constexpr (!BILINEAR)
        return confidence;
    else
    {
        const float2 ip = a.projected[low >> 2];  // written by the scatter pass for every point that has fragments
        float u = ip.x, v = ip.y;
        for (int k = 0; k < l; ++k) u *= 0.5f, v *= 0.5f;
        return bilinear_weight(u, v, (int)(low & 3u)) * confidence;
    }
}

// BILINEAR_BLEND stops a pixel once its transmittance is below 0.001 (compared in double as in the reference,
// src/lib/rendering/RenderForward.cu:1626) and then leaves the background out as well (:1633).
template <bool BILINEAR>
__device__ __forceinline__ bool blend_is_saturated(float T)
{
    return BILINEAR && (double)T < 0.001;
}

// FUZZY_BLEND (BlendMultiFuzzy, src/lib/rendering/RenderForward.cu:1393-1503): fragments are collected while their depth
// stays within depth_accept of the bucket's first one; a bucket is blended as ONE fragment with the mean confidence and
// the mean descriptor of its elements. After the first bucket the reference sets its reference depth to -100000 (:1468)
// instead of the next fragment's depth, so every later fragment closes the bucket in front of it: only the nearest
// bucket ever holds more than one fragment, and a one-element bucket blends exactly like a FULL_BLEND fragment
// (x / 1.0f == x). So the state below only lives until the nearest bucket is closed; from then on the ordinary blend
// step runs. (That needs depth + 100000 >= depth_accept, which the host checks: depth_accept < 10000.)
template <int C>
struct FuzzyBucket
{
    bool open = true;  // the nearest bucket is still collecting
    float first_depth = 0.f, conf = 0.f;
    float t[C];
    int m = 0;
    __device__ __forceinline__ FuzzyBucket()
    {
#pragma unroll
        for (int ci = 0; ci < C; ++ci) t[ci] = 0.f;
    }
    // blends the collected elements into (T, color) as one fragment
    __device__ __forceinline__ void flush(float& T, float (&color)[C])
    {
        const float fm = (float)m;
        const float cf = conf / fm;
        const float Tc = T * cf;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) color[ci] = Tc * (t[ci] / fm) + color[ci];
        T    = (1.f - cf) * T;
        open = false;
    }
    // Fragment at depth d: true if it joined the nearest bucket; false if it lies behind it, in which case the bucket
    // has been blended and the caller blends the fragment by itself.
    __device__ __forceinline__ bool take(float d, float cf, const float (&td)[4], float depth_accept, float& T,
                                         float (&color)[C])
    {
        if (m == 0) first_depth = d;
        if (!(d - first_depth < depth_accept))
        {
            flush(T, color);
            return false;
        }
        conf += cf;
#pragma unroll
        for (int ci = 0; ci < C; ++ci) t[ci] += td[ci];
        ++m;
        return true;
    }
};

// Sorts list[0, n), n <= kBuildCap, by the whole workgroup through the LDS room `room` (kBuildCap keys). Copy in (padded
// with +infinity to a power of two), every wave sorts 64-key chunks in registers, then the chunks are merged pairwise,
// level by level, in the all-ascending form of the bitonic network: a mirror step and the halving steps over 64 or more
// places run on LDS with a barrier each, the last six halving steps of every level again in registers. A list of 512
// keys takes 13 barriers instead of the 45 of the plain network. Every thread of the workgroup must call.
__device__ __forceinline__ void block_sort_in_lds(uint64_t* list, uint32_t n, uint64_t* room, int tid)
{
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    uint32_t m = kWave;
    while (m < n) m <<= 1;  // <= kBuildCap
    for (uint32_t k = tid; k < m; k += kBlock) room[k] = k < n ? list[k] : kInfKey;
    __syncthreads();
    const uint32_t chunks = m / kWave;
    for (uint32_t c = wave; c < chunks; c += kBlock / kWave)
        room[c * kWave + lane] = bitonic_sort_groups<6>(room[c * kWave + lane], lane);
    __syncthreads();
    auto order = [&](uint32_t i, uint32_t j) {  // i < j: the smaller key to place i
        const uint64_t x = room[i], y = room[j];
        if (y < x)
        {
            room[i] = y;
            room[j] = x;
        }
    };
    for (uint32_t k = 2 * kWave; k <= m; k <<= 1)
    {
        const uint32_t hk = k >> 1;
        for (uint32_t p = tid; p < (m >> 1); p += kBlock)  // mirror step inside every block of k places
        {
            const uint32_t blk = p / hk, r = p % hk;
            order(blk * k + r, blk * k + (k - 1 - r));
        }
        __syncthreads();
        for (uint32_t jj = k >> 2; jj >= (uint32_t)kWave; jj >>= 1)
        {
            for (uint32_t p = tid; p < (m >> 1); p += kBlock)
            {
                const uint32_t i = (p / jj) * 2 * jj + (p % jj);
                order(i, i + jj);
            }
            __syncthreads();
        }
        for (uint32_t c = wave; c < chunks; c += kBlock / kWave)
            room[c * kWave + lane] = bitonic_merge64(room[c * kWave + lane], lane);
        __syncthreads();
    }
    for (uint32_t k = tid; k < n; k += kBlock) list[k] = room[k];
    __syncthreads();
}

template <int C, bool BILINEAR, bool FUZZY>
__device__ __forceinline__ void bin_build(const BuildPass& a)
{
    static_assert(!(BILINEAR && FUZZY), "one blend rule at a time");
    __shared__ uint32_t s_cnt[kTilePixels];
    __shared__ uint32_t s_prefix[kTilePixels];
    __shared__ uint32_t s_wave_tot[kBlock / kWave];
    __shared__ uint8_t s_src_lane[kBlock / kWave][kWave];
    __shared__ uint64_t s_block_sorted[kBlock / kWave];  // pixels whose lists the whole workgroup sorts, a mask per wave
    __shared__ uint64_t s_keys[kBuildCap];
    __shared__ uint8_t s_pix[kBuildCap];       // pixel (inside the bin) of every list place
    __shared__ float4 s_stage[2][kStage];      // descriptors, then confidences (and depths) of the staged fragments: two
                                               // planes, so that the lanes of a store or load are 16 bytes apart
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t bin = a.num_bins - 1u - blockIdx.x;  // coarse layers first
    int l              = 0;
#pragma unroll
    for (int k = 1; k < VETRAST_MAX_LAYERS; ++k)
        if (k < a.ly.L && bin >= a.ly.bin_base[k]) l = k;
    const int shift       = a.ly.bin_shift[l];
    const uint32_t pixels = 1u << shift;  // pixels of this bin
    const uint32_t q0     = a.ly.base[l] + ((bin - a.ly.bin_base[l]) << shift);
    // the same for every lane: tell the compiler, so that loops over the bin's records become scalar branches
    const uint32_t begin  = (uint32_t)__builtin_amdgcn_readfirstlane((int)a.bin_offsets[bin]);
    const uint32_t n      = (uint32_t)__builtin_amdgcn_readfirstlane((int)a.bin_offsets[bin + 1]) - begin;
    const uint32_t room_cap = a.ly.room_cap[l];
    const size_t room       = room_of_bin(a.ly, l, bin);
    // record r of the bin: its own room first, what did not fit there in the compact array; as (key low, key high,
    // pixel in bin, 0) whatever its form in memory
    auto record = [&](uint32_t r) {
        const size_t at = r < room_cap ? room + r : (size_t)begin + r;
        if (a.compact_records)
        {
            const uint2 v = reinterpret_cast<const uint2*>(r < room_cap ? a.primary : a.binned)[at];
            return make_uint4(v.y >> 8, v.x, v.y & 0xFFu, 0u);
        }
        return (r < room_cap ? a.primary : a.binned)[at];
    };
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
            where[k] = 0xFFFFFFFFu;
            key[k]   = 0ull;
        }
#pragma unroll
        for (int k = 0; k < kBuildPerThread; ++k)
        {
            if ((uint32_t)(k * kBlock) >= n) break;  // uniform: most bins hold a few hundred records
            const uint32_t r = (uint32_t)(k * kBlock + tid);
            if (r < n)
            {
                const uint4 rec     = record(r);
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
                px[k]            = r < n ? (record(r).z & (pixels - 1u)) : 0xFFFFFFFFu;
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
    const uint32_t keep = a.K > 0 ? min(c, (uint32_t)a.K) : c;  // fragments of this thread's pixel left by the top-K cut
    uint32_t used       = 0;                                    // ... that took part in the blend
    bool saturated      = false;
    float T = 1.f;
    float color[C];
#pragma unroll
    for (int ci = 0; ci < C; ++ci) color[ci] = 0.f;
    FuzzyBucket<C> fuzzy;  // FUZZY_BLEND only
    if (in_lds)
    {
#pragma unroll
        for (int k = 0; k < kBuildPerThread; ++k)
            if ((uint32_t)(k * kBlock) < n && where[k] != 0xFFFFFFFFu)
            {
                const uint32_t place = s_prefix[where[k] & 0xFF] + (where[k] >> 8);
                s_keys[place]        = key[k];
                s_pix[place]         = (uint8_t)(where[k] & 0xFF);
            }
        __syncthreads();
        sort_wave_lists(s_keys, s_src_lane[wave], list_off, list_len, lane, a.K);
        __syncthreads();
        for (uint32_t r = tid; r < n; r += kBlock) a.fragments[begin + r] = s_keys[r];
        __syncthreads();  // the depth halves have been read; they now hold the transmittances

        // ---- blend
        float* s_T = reinterpret_cast<float*>(s_keys);  // s_T[2 r + 1]: transmittance in front of the fragment at r
        const uint32_t* s_id = reinterpret_cast<const uint32_t*>(s_keys);  // s_id[2 r]: its point id
        for (uint32_t base = 0; base < n; base += kStage)
        {
#pragma unroll
            for (int k = 0; k < (kStage + kBlock - 1) / kBlock; ++k)
            {
                const uint32_t r = base + k * kBlock + tid;
                if (k * kBlock + tid >= kStage || r >= n) continue;
                const uint32_t px  = s_pix[r];
                const uint32_t len = a.K > 0 ? min(s_cnt[px], (uint32_t)a.K) : s_cnt[px];
                if (r - s_prefix[px] >= len) continue;  // cut away
                const uint32_t low = s_id[2 * r];
                const int id       = BILINEAR ? (int)(low >> 2) : (int)low;
                // an id or texture index out of range cannot come from a list the scatter pass wrote; such a fragment
                // blends as fully transparent (the reference asserts on the texture index, RenderForward.cu:1335-1336)
                int ti = -1;
                if ((uint32_t)id < (uint32_t)a.N) ti = a.index ? a.index[id] : id;
                float4 t4 = make_float4(0.f, 0.f, 0.f, 0.f), c4 = t4;
                if ((uint32_t)ti < (uint32_t)a.N)
                {
                    t4   = a.packed[2 * (size_t)ti];
                    c4   = a.packed[2 * (size_t)ti + 1];
                    c4.x = fragment_alpha<BILINEAR>(a, l, low, c4.x);
                }
                // FUZZY_BLEND buckets by depth: it rides along in the stage (the key's depth half is still intact here)
                if constexpr (FUZZY) c4.y = __uint_as_float(s_id[2 * r + 1]);
                s_stage[0][r - base] = t4;
                s_stage[1][r - base] = c4;
            }
            __syncthreads();
            if ((uint32_t)tid < pixels)
            {
                const uint32_t lo = max(start, base), hi = min(start + keep, base + (uint32_t)kStage);
                uint32_t r = lo;
                if constexpr (FUZZY)
                {
                    // The nearest bucket, in a loop of its own, so that the loop below is FULL_BLEND's (which the
                    // compiler unrolls, with the stage reads of several fragments in flight). What is stored is the
                    // transmittance in front of the bucket the fragment joins.
                    for (; r < hi && fuzzy.open; ++r)
                    {
                        const float4 t4 = s_stage[0][r - base];
                        const float2 cd = *reinterpret_cast<const float2*>(&s_stage[1][r - base]);  // confidence, depth
                        const float t[4] = {t4.x, t4.y, t4.z, t4.w};
                        const bool joined = fuzzy.take(cd.y, cd.x, t, a.depth_accept, T, color);
                        s_T[2 * r + 1] = T;
                        ++used;
                        if (joined) continue;
                        const float Tc = T * cd.x;
#pragma unroll
                        for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                        T = (1.f - cd.x) * T;
                    }
                }
                for (; r < hi && !saturated; ++r)
                {
                    const float4 t4 = s_stage[0][r - base];
                    const float cf  = s_stage[1][r - base].x;
                    const float t[4] = {t4.x, t4.y, t4.z, t4.w};
                    s_T[2 * r + 1]  = T;
                    const float Tc   = T * cf;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                    T = (1.f - cf) * T;
                    ++used;
                    saturated = blend_is_saturated<BILINEAR>(T);
                }
            }
            __syncthreads();
        }
        if constexpr (FUZZY)
            if (fuzzy.open && fuzzy.m > 0) fuzzy.flush(T, color);
        // fragments of the pixel that took part in the blend; the pixel counts are not needed any more (the last read
        // of them is in front of the closing barrier of the loop above), so their array takes the numbers
        s_cnt[tid] = used;
        __syncthreads();
        if (a.transmittance)
            for (uint32_t r = tid; r < n; r += kBlock)
            {
                const uint32_t px = s_pix[r];
                if (r - s_prefix[px] < s_cnt[px]) a.transmittance[begin + r] = s_T[2 * r + 1];
            }
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
                rec[k]           = r < n ? record(r) : make_uint4(0u, 0u, 0xFFFFFFFFu, 0u);
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
        // Lists that have to be sorted in full and are too long for a wave's registers are sorted by the whole
        // workgroup through the key array in LDS, which is not in use on this path, one list after the other (in global
        // memory every step of the network costs a memory round trip, and such a list needs dozens of steps).
        const bool full_sort = !(a.K > 0 && a.K <= kWave);
        sort_wave_lists(a.fragments + begin, s_src_lane[wave], list_off, list_len, lane, a.K,
                        /*skip_longer=*/(uint32_t)kBuildCap);
        __threadfence_block();
        __syncthreads();
        if (full_sort)
        {
            const bool mine = (uint32_t)tid < pixels && c > kRegisterSortKeys && c <= (uint32_t)kBuildCap;  // pixel tid
            const uint64_t wave_mask = __ballot(mine);
            if (lane == 0) s_block_sorted[wave] = wave_mask;
            __syncthreads();
            for (int w = 0; w < kBlock / kWave; ++w)  // the same trips for every thread
            {
                uint64_t todo = s_block_sorted[w];
                while (todo != 0ull)
                {
                    const uint32_t px = w * kWave + (__ffsll((unsigned long long)todo) - 1);
                    todo &= todo - 1ull;
                    block_sort_in_lds(a.fragments + begin + s_prefix[px], s_cnt[px], s_keys, tid);
                }
            }
        }
        __threadfence_block();
        __syncthreads();
        if (a.K <= 0 && n > 16u * pixels)
        {
            // Without a cut the lists of a streamed bin of few pixels run to hundreds of fragments. One thread walking such a list
            // with a memory round trip every few fragments would hold the whole workgroup up, so the bin is blended
            // like one in LDS: all threads gather the descriptor records of a stretch of list places into the stage,
            // then the pixel's thread walks its fragments of that stretch. Keys come from the fragment buffer and the
            // transmittances go straight to memory.
            const uint64_t* list_mem = a.fragments + begin;
            for (uint32_t base = 0; base < n; base += kStage)
            {
#pragma unroll
                for (int k = 0; k < (kStage + kBlock - 1) / kBlock; ++k)
                {
                    const uint32_t r = base + k * kBlock + tid;
                    if (k * kBlock + tid >= kStage || r >= n) continue;
                    const uint64_t k64 = list_mem[r];
                    const uint32_t low = (uint32_t)k64;
                    const int id       = BILINEAR ? (int)(low >> 2) : (int)low;
                    int ti             = -1;
                    if ((uint32_t)id < (uint32_t)a.N) ti = a.index ? a.index[id] : id;
                    float4 t4 = make_float4(0.f, 0.f, 0.f, 0.f), c4 = t4;
                    if ((uint32_t)ti < (uint32_t)a.N)
                    {
                        t4   = a.packed[2 * (size_t)ti];
                        c4   = a.packed[2 * (size_t)ti + 1];
                        c4.x = fragment_alpha<BILINEAR>(a, l, low, c4.x);
                    }
                    if constexpr (FUZZY) c4.y = __uint_as_float((uint32_t)(k64 >> 32));
                    s_stage[0][r - base] = t4;
                    s_stage[1][r - base] = c4;
                }
                __syncthreads();
                if ((uint32_t)tid < pixels)
                {
                    const uint32_t lo = max(start, base), hi = min(start + keep, base + (uint32_t)kStage);
                    uint32_t r = lo;
                    if constexpr (FUZZY)
                    {
                        for (; r < hi && fuzzy.open; ++r)  // the nearest bucket, as above
                        {
                            const float4 t4 = s_stage[0][r - base];
                            const float2 cd = *reinterpret_cast<const float2*>(&s_stage[1][r - base]);  // confidence, depth
                            const float t[4] = {t4.x, t4.y, t4.z, t4.w};
                            const bool joined = fuzzy.take(cd.y, cd.x, t, a.depth_accept, T, color);
                            if (a.transmittance) a.transmittance[begin + r] = T;
                            ++used;
                            if (joined) continue;
                            const float Tc = T * cd.x;
#pragma unroll
                            for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                            T = (1.f - cd.x) * T;
                        }
                    }
                    for (; r < hi && !saturated; ++r)
                    {
                        const float4 t4 = s_stage[0][r - base];
                        const float cf  = s_stage[1][r - base].x;
                        const float t[4] = {t4.x, t4.y, t4.z, t4.w};
                        if (a.transmittance) a.transmittance[begin + r] = T;
                        const float Tc = T * cf;
#pragma unroll
                        for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                        T = (1.f - cf) * T;
                        ++used;
                        saturated = blend_is_saturated<BILINEAR>(T);
                    }
                }
                __syncthreads();
            }
            if constexpr (FUZZY)
                if (fuzzy.open && fuzzy.m > 0) fuzzy.flush(T, color);
        }
        else if ((uint32_t)tid < pixels)
        {
            if constexpr (FUZZY)
            {
                const uint64_t* list = a.fragments + begin + start;
                for (uint32_t j = 0; j < keep; ++j)
                {
                    const uint64_t k = list[j];
                    const int id     = (int)(uint32_t)k;
                    int ti           = -1;
                    if ((uint32_t)id < (uint32_t)a.N) ti = a.index ? a.index[id] : id;
                    float4 t4 = make_float4(0.f, 0.f, 0.f, 0.f);
                    float cf  = 0.f;
                    if ((uint32_t)ti < (uint32_t)a.N)
                    {
                        t4 = a.packed[2 * (size_t)ti];
                        cf = a.packed[2 * (size_t)ti + 1].x;
                    }
                    const float t[4] = {t4.x, t4.y, t4.z, t4.w};
                    const bool joined =
                        fuzzy.open && fuzzy.take(__uint_as_float((uint32_t)(k >> 32)), cf, t, a.depth_accept, T, color);
                    if (a.transmittance) a.transmittance[begin + start + j] = T;
                    if (joined) continue;
                    const float Tc = T * cf;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                    T = (1.f - cf) * T;
                }
                if (fuzzy.open && fuzzy.m > 0) fuzzy.flush(T, color);
                used = keep;
            }
            else if constexpr (!BILINEAR)
            {
                blend_list_from_memory<C>(a.fragments + begin + start, keep, a.index, a.packed, a.N,
                                          a.transmittance ? a.transmittance + begin + start : nullptr, T, color);
                used = keep;
            }
            else
            {
                const uint64_t* list = a.fragments + begin + start;
                for (uint32_t j = 0; j < keep && !saturated; ++j)
                {
                    const uint32_t low = (uint32_t)list[j];
                    const int id       = (int)(low >> 2);
                    int ti             = -1;
                    if ((uint32_t)id < (uint32_t)a.N) ti = a.index ? a.index[id] : id;
                    float4 t4 = make_float4(0.f, 0.f, 0.f, 0.f);
                    float cf  = 0.f;
                    if ((uint32_t)ti < (uint32_t)a.N)
                    {
                        t4 = a.packed[2 * (size_t)ti];
                        cf = fragment_alpha<BILINEAR>(a, l, low, a.packed[2 * (size_t)ti + 1].x);
                    }
                    if (a.transmittance) a.transmittance[begin + start + j] = T;
                    const float t[4] = {t4.x, t4.y, t4.z, t4.w};
                    const float Tc   = T * cf;
#pragma unroll
                    for (int ci = 0; ci < C; ++ci) color[ci] = Tc * t[ci] + color[ci];
                    T = (1.f - cf) * T;
                    ++used;
                    saturated = blend_is_saturated<BILINEAR>(T);
                }
            }
        }
    }

    if ((uint32_t)tid < pixels)
    {
        // pixel number -> image coordinates
        const uint32_t q = q0 + tid;
        // How many fragments of the list took part, and one byte that says whether any did not (top-K cut, saturation):
        // the backward per-point kernel only has to look at the last blended key of a pixel where this is set.
        // (FULL_BLEND blends min(count, K) fragments, which the readers work out themselves: the array is not written.)
        if constexpr (BILINEAR) a.kept[q] = used;
        a.list_is_cut[q] = used < c ? 1 : 0;
        // ... and that key itself (the sorted keys of this bin went out to the fragment buffer before the blend)
        if (used < c) a.last_key[q] = used ? a.fragments[begin + start + used - 1u] : 0ull;
        // a bin lies inside one tile: the tile's coordinates are the same for the whole workgroup (scalar arithmetic)
        const uint32_t tile = (q0 - a.ly.base[l]) / kTilePixels;
        const uint32_t ty = tile / (uint32_t)a.ly.tiles_x[l], tx = tile - ty * (uint32_t)a.ly.tiles_x[l];
        const int x = (int)(tx * kTile + (q & (kTile - 1))), y = (int)(ty * kTile + ((q / kTile) & (kTile - 1)));
        if (x < a.ly.w[l] && y < a.ly.h[l])
        {
            const size_t plane   = (size_t)a.ly.w[l] * a.ly.h[l];
            const uint32_t local = (uint32_t)y * (uint32_t)a.ly.w[l] + (uint32_t)x;
#pragma unroll
            for (int ci = 0; ci < C; ++ci)
            {
                if (!a.use_environment_map && !saturated) color[ci] = (T * 1.f) * a.background[ci] + color[ci];
                a.out[l][ci * plane + local] = color[ci];
            }
            a.weight[q] = T;
            if (a.out_mask[l]) a.out_mask[l][local] = (T == 0.f) ? a.mask_value : 1.f;
            if (a.out_weight[l]) a.out_weight[l][local] = T;
        }
    }
}

template <int C, bool BILINEAR, bool FUZZY = false>
__global__ void __launch_bounds__(kBlock) bin_build_kernel(BuildPass a)
{
    bin_build<C, BILINEAR, FUZZY>(a);
}

template <int C, bool BILINEAR, bool FUZZY = false>
__global__ void __launch_bounds__(kBlock) bin_build_views_kernel(PerView<BuildPass> views)
{
    bin_build<C, BILINEAR, FUZZY>(views.v[blockIdx.y]);
}

}  // namespace vetrast
