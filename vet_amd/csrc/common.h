// Shared declarations of the gfx950 blending point rasterizer (internal; the public boundary is include/vetrast.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/vetrast.h"

namespace vetrast
{
constexpr int kBlock          = 256;          // threads per workgroup = 4 wave64
constexpr int kWave           = 64;
constexpr uint64_t kInfKey    = ~0ull;        // sorts behind every real (depth bits, point id) key
constexpr int kScanPerThread  = 16;
constexpr int kScanPerBlock   = kBlock * kScanPerThread;  // 4096 counts per workgroup
constexpr int kBlendChunk     = 4;            // fragments a blend / backward thread prefetches at a time
constexpr int kBackgroundRow  = 8;            // floats per workgroup row of background-gradient partial sums
constexpr int kPreparedBackgroundOffset = 16;  // float index inside the flags block: the background as it is blended
constexpr int kPackedFloats   = 8;            // interleaved record: 4 descriptor floats, confidence, 3 pad
constexpr int kPrimaryCap     = 2048;         // fragment records a bin has room for where about a thousand are expected
constexpr int kPrimaryCapSmall = 1024;        // ... and where at most half of that is (a bin built in LDS holds <= 1024)
constexpr int kViewLanes      = 4;            // views of one call that share a launch (each with scratch of its own)
constexpr int kLogSegments    = 256;          // the overflow log is cut into this many segments with a cursor each
constexpr int kLogCursorStride = 16;          // uint32 between two cursors (64 bytes: one cursor per cache line)

// Camera constants of one view, written by prepare_views_kernel and read (uniformly) by every other kernel.
// Counterpart of what the reference pulls per thread out of d_render_params.Pose()/PinholeIntrinsics() and the
// by-value ReducedImageInfo (src/lib/rendering/RenderForward.cu:117-158).
struct DeviceView
{
    float r[9];  // world -> camera rotation, row-major
    float t[3];
    float fx, fy, cx, cy, s;  // K
    float crop[5];            // fx, fy, cx, cy, s of the crop transform
    float rot[4];             // crop rotation r00 r01 r10 r11
    float ccx, ccy;           // (w/2, h/2) with integer halving
    float dist[8];            // k1 k2 k3 k4 k5 k6 p1 p2 of the rational distortion model; read only when has_dist
    uint32_t has_dist;        // some coefficient is not zero and the caller has switched distortion on
    float pad[3];
};
static_assert(sizeof(DeviceView) == 40 * 4, "DeviceView is 40 floats");

// Pixels are numbered tile by tile: every layer is cut into 16x16 pixel tiles (the last column and row of tiles may
// hang over the image), tiles are numbered row-major inside a layer and layer after layer, and pixel (x, y) of layer l is
//   q = 256 * (tile_base[l] + (y / 16) * tiles_x[l] + x / 16) + 16 * (y % 16) + x % 16.
// The 256 pixels of a tile are consecutive, so a tile's fragment lists form one contiguous stretch of the fragment
// buffer and a workgroup that owns a tile reads and writes its per-pixel arrays fully coalesced. Pixels of overhanging
// tiles that lie outside the image exist in the numbering and always have empty lists.
constexpr int kTile       = 16;
constexpr int kTilePixels = kTile * kTile;
struct LayerTable
{
    int L;
    int w[VETRAST_MAX_LAYERS];
    int h[VETRAST_MAX_LAYERS];
    int tiles_x[VETRAST_MAX_LAYERS];
    int tiles_y[VETRAST_MAX_LAYERS];
    uint32_t tile_base[VETRAST_MAX_LAYERS + 1];  // first tile of the layer; [L] = number of tiles
    uint32_t base[VETRAST_MAX_LAYERS + 1];       // first pixel number of the layer = 256 * tile_base
    // Bins of the list-building passes: runs of 2^bin_shift consecutive pixel numbers (256 = a tile, 64 = a 16x4 strip
    // of it, 16 = one row of it, 4), chosen per layer so that a bin is expected to hold about a thousand fragments.
    int bin_shift[VETRAST_MAX_LAYERS];
    uint32_t bin_base[VETRAST_MAX_LAYERS + 1];  // first bin of the layer; [L] = number of bins
    // Every bin owns room for room_cap[l] fragment records (its first arrivals; later ones take the overflow path):
    // the room of bin b of layer l starts at record room_base[l] + (b - bin_base[l]) * room_cap[l].
    uint32_t room_cap[VETRAST_MAX_LAYERS];
    uint32_t room_base[VETRAST_MAX_LAYERS + 1];  // [L] = records in all rooms
};

// First record of the room of `bin`, a bin of layer l.
__host__ __device__ __forceinline__ size_t room_of_bin(const LayerTable& t, int l, uint32_t bin)
{
    return (size_t)t.room_base[l] + (size_t)(bin - t.bin_base[l]) * t.room_cap[l];
}

// Value of lane (lane ^ M) for the xor patterns a 64-wide bitonic network needs. Inside a row of 16 lanes the exchange
// is a DPP move (register to register, a few cycles); only the four patterns that cross rows go through the LDS
// crossbar (ds_swizzle within 32 lanes, ds_bpermute across the halves).
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, false);
}

template <int M>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v, int lane)
{
    if constexpr (M == 1) return dpp_move<0xB1>(v);         // quad_perm [1,0,3,2]
    else if constexpr (M == 2) return dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    else if constexpr (M == 3) return dpp_move<0x1B>(v);    // quad_perm [3,2,1,0]
    else if constexpr (M == 7) return dpp_move<0x141>(v);   // row_half_mirror
    else if constexpr (M == 15) return dpp_move<0x140>(v);  // row_mirror
    else if constexpr (M == 8) return dpp_move<0x128>(v);   // row_ror:8
    else if constexpr (M == 4)
    {
        // banks (groups of 4 lanes) 0 and 2 read lane+4 (row_shl:4), banks 1 and 3 read lane-4 (row_shr:4)
        int t = __builtin_amdgcn_update_dpp((int)v, (int)v, 0x104, 0xF, 0x5, false);
        t     = __builtin_amdgcn_update_dpp(t, (int)v, 0x114, 0xF, 0xA, false);
        return (uint32_t)t;
    }
    else if constexpr (M == 16) return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x401F);  // xor 0x10, and 0x1F
    else if constexpr (M == 31) return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x7C1F);  // xor 0x1F, and 0x1F
    else return (uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ M) << 2, (int)v);               // 32, 63
}

// Inclusive prefix sum over the 64 lanes, all of which must be active: four shift-and-add steps inside every row of 16
// lanes, then the last lane of row 0 (2) is added to row 1 (3) and lane 31 to the upper half; six DPP adds, no LDS
// permute (lanes a shift leaves without a source add zero).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_shifted(uint32_t x)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, ROW_MASK, 0xF, false);
}

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v, int /*lane*/)
{
    v += dpp_shifted<0x111, 0xF>(v);  // row_shr:1
    v += dpp_shifted<0x112, 0xF>(v);  // row_shr:2
    v += dpp_shifted<0x114, 0xF>(v);  // row_shr:4
    v += dpp_shifted<0x118, 0xF>(v);  // row_shr:8
    v += dpp_shifted<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_shifted<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

// Launch descriptor shared by the forward kernels of one view.
// Several views of a call in one launch: the arguments of every view travel side by side as the kernel argument and
// blockIdx.y (blockIdx.z where a kernel uses y itself) picks the view. Small views (training crops) leave most of the
// chip idle on their own and are chains of dependent launches; four of them at a time fill it.
template <class Args>
struct PerView
{
    Args v[kViewLanes];
};

struct ViewPass
{
    const float4* position;
    const int32_t* index;
    const float* confidence;
    const float* dropout;  // already offset to this view, or null
    const DeviceView* view;
    LayerTable ly;
    int N;
    int drop_by_radius;
    float radius_threshold;
    int viewer_only;
    float stability_cutoff;
    int confidence_activation;  // 1: `confidence` holds raw values, the confidence is sigmoid(confidence_scale * raw)
    float confidence_scale;
    float2* projected;  // BILINEAR_BLEND: [N] image position of every visible point at layer 0, written by the scatter pass
    const int32_t* point_order;  // [N] or null: the scatter pass's thread i takes point point_order[i]
};

struct Projected
{
    float ipx, ipy, z, radius;
};

// The 8-coefficient rational distortion model (k1 k2 k3 k4 k5 k6 p1 p2) on a normalised image point, every operation
// rounded on its own so that the CPU check of the same formula agrees bit for bit. The reference calls saiga's
// distortNormalizedPoint here (src/lib/rendering/PointRendererHelper.h:207), which is not in its source tree: this is
// the published model its coefficient layout implies.
__device__ __forceinline__ void distort_point(const float* d, float x, float y, float& xd, float& yd)
{
    const float x2 = x * x, y2 = y * y, r2 = x2 + y2, xy2 = (2.f * x) * y;
    const float u   = 1.f + r2 * (d[0] + r2 * (d[1] + r2 * d[2]));
    const float v   = 1.f + r2 * (d[3] + r2 * (d[4] + r2 * d[5]));
    const float iv  = 1.f / v;
    const float rad = u * iv;
    const float tx = d[6] * xy2 + d[7] * (r2 + 2.f * x2);
    const float ty = d[6] * (r2 + 2.f * y2) + d[7] * xy2;
    xd = x * rad + tx;
    yd = y * rad + ty;
}

// The same with its Jacobians: J = d(xd, yd) / d(x, y) row-major, Jd[2 k], Jd[2 k + 1] = d(xd, yd) / d coefficient k.
__device__ __forceinline__ void distort_point_jacobians(const float* d, float x, float y, float& xd, float& yd,
                                                        float (&J)[4], float (&Jd)[16])
{
    const float x2 = x * x, y2 = y * y, r2 = x2 + y2, xy2 = (2.f * x) * y;
    const float u   = 1.f + r2 * (d[0] + r2 * (d[1] + r2 * d[2]));
    const float v   = 1.f + r2 * (d[3] + r2 * (d[4] + r2 * d[5]));
    const float iv  = 1.f / v;
    const float rad = u * iv;
    const float tx = d[6] * xy2 + d[7] * (r2 + 2.f * x2);
    const float ty = d[6] * (r2 + 2.f * y2) + d[7] * xy2;
    xd = x * rad + tx;
    yd = y * rad + ty;
    const float du   = d[0] + r2 * (2.f * d[1] + (3.f * d[2]) * r2);  // du / d r2
    const float dv   = d[3] + r2 * (2.f * d[4] + (3.f * d[5]) * r2);
    const float drad = (du * v - u * dv) * (iv * iv);                  // d rad / d r2
    const float rx = drad * (2.f * x), ry = drad * (2.f * y);
    J[0] = (rad + x * rx) + ((2.f * d[6]) * y + (6.f * d[7]) * x);
    J[1] = x * ry + ((2.f * d[6]) * x + (2.f * d[7]) * y);
    J[2] = y * rx + ((2.f * d[6]) * x + (2.f * d[7]) * y);
    J[3] = (rad + y * ry) + ((6.f * d[6]) * y + (2.f * d[7]) * x);
    const float r4 = r2 * r2, r6 = r4 * r2;
    const float a = iv, b = -(u * (iv * iv));
    const float c[6] = {a * r2, a * r4, a * r6, b * r2, b * r4, b * r6};
#pragma unroll
    for (int k = 0; k < 6; ++k)
    {
        Jd[2 * k]     = x * c[k];
        Jd[2 * k + 1] = y * c[k];
    }
    Jd[12] = xy2;
    Jd[13] = r2 + 2.f * y2;
    Jd[14] = r2 + 2.f * x2;
    Jd[15] = xy2;
}

// Projection of one point: rigid transform, clamp z, divide, K, crop transform, rotation about the crop centre.
// Follows ProjPoint / ProjectPointPinhole / rotateCropAroundCenter (src/lib/rendering/RenderForward.cu:110-158,
// src/lib/rendering/PointRendererHelper.h:184-218). Every operation is rounded on its own
// (the file is compiled with -ffp-contract=off) so that the CPU check of the same formula agrees bit for bit.
__device__ __forceinline__ bool project_point(const DeviceView& c, const float4 p, Projected& o)
{
    const float vx = ((c.r[0] * p.x + c.r[1] * p.y) + c.r[2] * p.z) + c.t[0];
    const float vy = ((c.r[3] * p.x + c.r[4] * p.y) + c.r[5] * p.z) + c.t[1];
    const float vz = ((c.r[6] * p.x + c.r[7] * p.y) + c.r[8] * p.z) + c.t[2];
    const float z  = fmaxf(vz, 0.f);
    if (!(z > 0.f)) return false;
    float nx = vx / vz;
    float ny = vy / vz;
    if (c.has_dist) distort_point(c.dist, nx, ny, nx, ny);
    const float u   = (c.fx * nx + c.s * ny) + c.cx;
    const float v   = c.fy * ny + c.cy;
    const float ipx = (c.crop[0] * u + c.crop[4] * v) + c.crop[2];
    const float ipy = c.crop[1] * v + c.crop[3];
    const float dx = ipx - c.ccx, dy = ipy - c.ccy;
    const float rx = c.rot[0] * dx + c.rot[1] * dy;
    const float ry = c.rot[2] * dx + c.rot[3] * dy;
    o.ipx          = rx + c.ccx;
    o.ipy          = ry + c.ccy;
    o.z            = z;
    o.radius       = ((c.fx * c.crop[0]) * p.w) / z;
    return true;
}

// Tile and pixel-in-tile of the pixel with (integral) float coordinates (fx, fy) of layer l; false outside the layer.
__device__ __forceinline__ bool tile_of_pixel(const LayerTable& ly, int l, float fx, float fy, uint32_t& tile,
                                              uint32_t& in_tile)
{
    if (!(fx >= 0.f && fx < (float)ly.w[l] && fy >= 0.f && fy < (float)ly.h[l])) return false;
    const uint32_t x = (uint32_t)(int)fx, y = (uint32_t)(int)fy;
    tile    = ly.tile_base[l] + (y / kTile) * (uint32_t)ly.tiles_x[l] + x / kTile;
    in_tile = (y % kTile) * kTile + x % kTile;
    return true;
}

// Pixel a projected point lands in at layer l, as hit number h of HITS. The caller halves ipx/ipy/radius between
// layers (src/lib/rendering/RenderForward.cu:856,888-891).
//   HITS = 1 (FULL_BLEND): the pixel the position rounds to; rintf is round-half-even like __float2int_rn.
//   HITS = 4 (BILINEAR_BLEND): the 2x2 pixels around the position, floor + (h & 1, h >> 1); h is the corner number
//   y_j * 2 + x_i of src/lib/rendering/RenderForward.cu:865-885,1097-1134.
template <int HITS>
__device__ __forceinline__ bool layer_hit(const LayerTable& ly, int l, float ipx, float ipy, int h, uint32_t& tile,
                                          uint32_t& in_tile)
{
    if constexpr (HITS == 1)
        return tile_of_pixel(ly, l, rintf(ipx), rintf(ipy), tile, in_tile);
    else
        return tile_of_pixel(ly, l, floorf(ipx) + (float)(h & 1), floorf(ipy) + (float)(h >> 1), tile, in_tile);
}

// compute_blending_fac (src/lib/rendering/PointBlending.h:12-44): bilinear weight of corner `corner` of a position, and
// optionally its derivative with respect to the position.
__device__ __forceinline__ float bilinear_weight(float u, float v, int corner, float* d_du = nullptr,
                                                 float* d_dv = nullptr)
{
    const float sx = u - floorf(u), sy = v - floorf(v);
    const float wx = (corner & 1) ? sx : 1.f - sx;
    const float wy = (corner & 2) ? sy : 1.f - sy;
    if (d_du)
    {
        // J(0) = (sy - 1, sx - 1), J(1) = (1 - sy, -sx), J(2) = (-sy, 1 - sx), J(3) = (sy, sx)
        const float jx[4] = {sy - 1.f, 1.f - sy, -sy, sy};
        const float jy[4] = {sx - 1.f, -sx, 1.f - sx, sx};
        *d_du = jx[corner];
        *d_dv = jy[corner];
    }
    return wx * wy;
}

// Bin and pixel-in-bin of a pixel given as (tile, pixel in tile) of layer l.
__device__ __forceinline__ void bin_of_pixel(const LayerTable& ly, int l, uint32_t tile, uint32_t in_tile, uint32_t& bin,
                                             uint32_t& in_bin)
{
    const uint32_t in_layer = (tile - ly.tile_base[l]) * kTilePixels + in_tile;
    bin    = ly.bin_base[l] + (in_layer >> ly.bin_shift[l]);
    in_bin = in_layer & ((1u << ly.bin_shift[l]) - 1u);
}

// exp and the logistic function from +, *, rint and one division only, so that the CPU check of the same formulas
// agrees bit for bit (library exp routines differ in the last bits between platforms). Cody-Waite reduction
// x = k ln2 + r, |r| <= ln2 / 2, a degree-7 Taylor polynomial of e^r (relative error about 1e-7), scaling by 2^k through
// the exponent bits.
__host__ __device__ __forceinline__ float exp_canon(float x)
{
    x             = fminf(fmaxf(x, -87.f), 88.f);
    const float k = rintf(x * 1.44269504088896341f);
    float r       = x - k * 0.693145751953125f;
    r             = r - k * 1.42860682030941723e-06f;
    float p       = 1.f / 5040.f;
    p             = p * r + 1.f / 720.f;
    p             = p * r + 1.f / 120.f;
    p             = p * r + 1.f / 24.f;
    p             = p * r + 1.f / 6.f;
    p             = p * r + 0.5f;
    p             = p * r + 1.f;
    p             = p * r + 1.f;
    const int e   = (int)k + 127;  // 40 .. 254
    union
    {
        uint32_t u;
        float f;
    } scale;
    scale.u = (uint32_t)e << 23;
    return p * scale.f;
}

// torch::sigmoid(scale * x) of NeuralPointTextureImpl::PrepareConfidence (src/lib/models/NeuralTexture.h:38-41).
__host__ __device__ __forceinline__ float sigmoid_canon(float x)
{
    return 1.f / (1.f + exp_canon(-x));
}

// Value the other lane of a pair (lane ^ 1) holds: a DPP register move (quad_perm [1,0,3,2]). Every lane of the wave
// must be active. Used to let two neighbouring lanes fetch or store the two 16-byte halves of ONE 32-byte record with
// one instruction: the memory pipeline then sees one 32-byte request per record instead of two 16-byte ones.
__device__ __forceinline__ int pair_other(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false); }
__device__ __forceinline__ float pair_other(float v) { return __int_as_float(pair_other(__float_as_int(v))); }
__device__ __forceinline__ float4 pair_other(float4 v)
{
    return make_float4(pair_other(v.x), pair_other(v.y), pair_other(v.z), pair_other(v.w));
}

// Place of the gradient record of the fragment (layer l, corner h, point id) in the record array of the backward pass
// (hits = 1, or 4 corners in BILINEAR_BLEND). Two layouts, chosen per call on the host. Layer after layer
// ([layer][corner][point]): the per-point kernel, which walks the points in order, reads every layer's records as one
// stream; right for views that see most of the cloud. Point after point ([point][layer][corner]): all records of a
// point are neighbours, one burst for the per-point kernel instead of a 64-byte access per record; right for views that
// see a small part of the cloud (training crops), where the streams of the first layout have turned into scattered
// reads anyway. Measured at 2 M points: full frame 0.313 against 0.336 ms (FULL_BLEND) in favour of the first, batch of
// four 512x512 crops 0.631 against 0.556 ms (BILINEAR_BLEND) in favour of the second.
__device__ __forceinline__ size_t gradient_record(int point_major, int N, int L, int hits, int l, int h, int id)
{
    return point_major ? (size_t)id * (size_t)(L * hits) + (size_t)(l * hits + h)
                       : (size_t)(l * hits + h) * (size_t)N + (size_t)id;
}

// Workgroup -> tile mapping of the per-pixel kernels (blend, backward): a workgroup owns a tile, a wave 16x4 pixels of
// it, because the fragments of neighbouring pixels come from the same few 256-point blocks of the cloud and their
// descriptor records then share cache lines. The same point shows up once per layer, in the tiles that cover the same
// part of the screen, so the tiles are grouped into screen regions: a region is one tile of the coarsest layer plus the
// 4, 16, 64 ... tiles of the finer layers over the same area, and is walked coarsest layer first. Workgroups are dealt
// round-robin to the 8 XCDs (each with its own L2), so workgroup b belongs to XCD b % 8 and takes slot b / 8 of that
// XCD's run of regions (region r goes to XCD r % 8): what one layer's tiles pulled into the XCD's L2 is still there
// when the next layer's tiles of the region ask for the same points.
constexpr int kXcds = 8;
// A layer whose pixels hold long lists is split: a workgroup then owns one 16x4 strip of a tile and each of its waves
// one row of 16 pixels (lanes 16..63 carry no pixel, only fragments), so that such a layer (few pixels, many fragments)
// is spread over four times as many waves, each with a quarter of the rounds to run one after the other.
struct TileMap
{
    int L;
    uint32_t regions_x, regions;     // region grid (regions per row, total)
    uint32_t tiles_per_region;       // (4^L - 1) / 3
    uint32_t regions_per_xcd;        // ceil(regions / 8)
    uint32_t split[VETRAST_MAX_LAYERS];  // workgroups per tile of the layer: 1, or 4 (one per 16x4 strip)
    uint32_t groups_per_region;      // sum over the layers of (tiles of the layer in a region) x split
};

struct TilePixel
{
    bool active;     // the pixel lies inside the layer
    int l, x, y;
    uint32_t q;      // pixel number over all layers
    uint32_t local;  // y * w + x inside the layer: index into the image planes
};

__device__ __forceinline__ TilePixel tile_pixel(const TileMap& tm, const LayerTable& ly)
{
    TilePixel r;
    r.active = false;
    r.l = r.x = r.y = 0;
    r.q = r.local = 0;
    const uint32_t b      = blockIdx.x;
    const uint32_t xcd    = b % kXcds;
    const uint32_t slot   = b / kXcds;
    const uint32_t region = (slot / tm.groups_per_region) * kXcds + xcd;
    uint32_t t            = slot % tm.groups_per_region;  // workgroup inside the region, coarsest layer first
    if (region >= tm.regions) return r;
    // layer L-1 has 1 tile per region, L-2 has 4, L-3 has 16, ...; split[l] workgroups per tile
    int l            = tm.L - 1;
    uint32_t side_log = 0;  // tiles per region side in layer l: 1 << side_log
    while (t >= tm.split[l] << (2 * side_log))
    {
        t -= tm.split[l] << (2 * side_log);
        ++side_log;
        --l;
    }
    // split is 1 or 4 and the side a power of two: shifts and masks instead of divisions by run-time values
    const uint32_t split_log = tm.split[l] == 1 ? 0u : 2u;
    const uint32_t strip     = t & (tm.split[l] - 1u);  // 16x4 strip of the tile, if the layer is split
    t >>= split_log;
    const uint32_t ry = region / tm.regions_x, rx = region - ry * tm.regions_x;
    const uint32_t ty = (ry << side_log) + (t >> side_log), tx = (rx << side_log) + (t & ((1u << side_log) - 1u));
    r.l = l;
    if (tx >= (uint32_t)ly.tiles_x[l] || ty >= (uint32_t)ly.tiles_y[l]) return r;
    uint32_t in_tile = threadIdx.x;  // 16 * (row of the tile) + column
    if (tm.split[l] != 1)
    {
        const uint32_t lane = threadIdx.x & (kWave - 1);
        if (lane >= (uint32_t)kTile) return r;  // this lane carries no pixel
        in_tile = (strip * 4 + threadIdx.x / kWave) * kTile + lane;
    }
    r.x = (int)(tx * kTile + (in_tile & (kTile - 1)));
    r.y = (int)(ty * kTile + (in_tile / kTile));
    r.q = (ly.tile_base[l] + ty * (uint32_t)ly.tiles_x[l] + tx) * kTilePixels + in_tile;
    if (r.x >= ly.w[l] || r.y >= ly.h[l]) return r;
    r.local  = (uint32_t)r.y * (uint32_t)ly.w[l] + (uint32_t)r.x;
    r.active = true;
    return r;
}

}  // namespace vetrast
