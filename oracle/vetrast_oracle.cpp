// CPU oracle of the blending point rasterizer — TEST INFRASTRUCTURE ONLY (see vetrast_oracle.h).
//
// Scalar restatement of the reference's FULL_BLEND and BILINEAR_BLEND paths. Every function names the reference lines it follows
// (paths relative to the reference's src/lib/). Build with -ffp-contract=off: the canonical arithmetic has no
// fused multiply-add, every operation is rounded on its own, in the order written here.
#include "vetrast_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#    include <omp.h>
#endif

namespace
{
struct Prepared
{
    float r[9];  // row-major rotation, world -> camera
    float t[3];
    float fx, fy, cx, cy, s;
    float dist[8];  // k1 k2 k3 k4 k5 k6 p1 p2; used only when has_dist
    bool has_dist;
};

struct Layers
{
    int L;
    int w[VETRAST_MAX_LAYERS], h[VETRAST_MAX_LAYERS];
    int64_t base[VETRAST_MAX_LAYERS + 1];
};

// Layer pyramid: repeated integer halving. rendering/PointRenderer.cu:351-381
Layers make_layers(int w, int h, int L)
{
    Layers ly;
    ly.L       = L;
    ly.base[0] = 0;
    for (int l = 0; l < L; ++l)
    {
        ly.w[l]        = w;
        ly.h[l]        = h;
        ly.base[l + 1] = ly.base[l] + (int64_t)w * h;
        w /= 2;
        h /= 2;
    }
    return ly;
}

// Pose: the reference keeps Sophus::SE3d (unit quaternion x,y,z,w + translation) and casts it to float per use
// (rendering/RenderConstants.h:78, data/NeuralStructure.cpp:15-28). Canon: rotation matrix from the quaternion in
// double (the usual 2xy-2wz form), then one rounding to float.
Prepared prepare(const double* q, const float* intr)
{
    Prepared p;
    const double x = q[0], y = q[1], z = q[2], w = q[3];
    const double tx = 2.0 * x, ty = 2.0 * y, tz = 2.0 * z;
    const double twx = tx * w, twy = ty * w, twz = tz * w;
    const double txx = tx * x, txy = ty * x, txz = tz * x;
    const double tyy = ty * y, tyz = tz * y, tzz = tz * z;
    p.r[0] = (float)(1.0 - (tyy + tzz));
    p.r[1] = (float)(txy - twz);
    p.r[2] = (float)(txz + twy);
    p.r[3] = (float)(txy + twz);
    p.r[4] = (float)(1.0 - (txx + tzz));
    p.r[5] = (float)(tyz - twx);
    p.r[6] = (float)(txz - twy);
    p.r[7] = (float)(tyz + twx);
    p.r[8] = (float)(1.0 - (txx + tyy));
    p.t[0] = (float)q[4];
    p.t[1] = (float)q[5];
    p.t[2] = (float)q[6];
    p.fx   = intr[0];
    p.fy   = intr[1];
    p.cx   = intr[2];
    p.cy   = intr[3];
    p.s    = intr[4];
    p.has_dist = false;
    for (int k = 0; k < 8; ++k)
    {
        p.dist[k] = intr[5 + k];
        if (intr[5 + k] != 0.f) p.has_dist = true;
    }
    return p;
}

// The 8-coefficient rational distortion model (k1 k2 k3 k4 k5 k6 p1 p2) on a normalised image point, every operation
// rounded on its own. The reference calls saiga's distortNormalizedPoint here (rendering/PointRendererHelper.h:207),
// which is not in its source tree: this is the published model its coefficient layout implies, parity unpinned.
// J (optional): d(xd, yd) / d(x, y) row-major; Jd (optional): d(xd, yd) / d coefficient k as Jd[2 k], Jd[2 k + 1].
inline void distort(const float* d, float x, float y, float& xd, float& yd, float* J = nullptr, float* Jd = nullptr)
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
    if (J)
    {
        const float du   = d[0] + r2 * (2.f * d[1] + (3.f * d[2]) * r2);  // du / d r2
        const float dv   = d[3] + r2 * (2.f * d[4] + (3.f * d[5]) * r2);
        const float drad = (du * v - u * dv) * (iv * iv);                  // d rad / d r2
        const float rx = drad * (2.f * x), ry = drad * (2.f * y);          // d rad / dx, dy
        J[0] = (rad + x * rx) + ((2.f * d[6]) * y + (6.f * d[7]) * x);
        J[1] = x * ry + ((2.f * d[6]) * x + (2.f * d[7]) * y);
        J[2] = y * rx + ((2.f * d[6]) * x + (2.f * d[7]) * y);
        J[3] = (rad + y * ry) + ((6.f * d[6]) * y + (2.f * d[7]) * x);
    }
    if (Jd)
    {
        const float r4 = r2 * r2, r6 = r4 * r2;
        const float a = iv, b = -(u * (iv * iv));
        const float c[6] = {a * r2, a * r4, a * r6, b * r2, b * r4, b * r6};
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
}

bool distortion_is_zero(const float* intr)
{
    for (int k = 5; k < 13; ++k)
        if (intr[k] != 0.f) return false;
    return true;
}

struct Projected
{
    float ipx, ipy, z, radius;
};

// ProjPoint + ProjectPointPinhole + rotateCropAroundCenter. rendering/RenderForward.cu:110-158,
// rendering/PointRendererHelper.h:184-218. Zero distortion only, so distortNormalizedPoint is the identity.
// Returns false when the point is rejected (z == 0 after the clamp, RenderForward.cu:852).
bool project(const Prepared& c, const vetrast_view& v, const float* p4, Projected& o)
{
    const float x = p4[0], y = p4[1], zz = p4[2];
    const float vx = ((c.r[0] * x + c.r[1] * y) + c.r[2] * zz) + c.t[0];
    const float vy = ((c.r[3] * x + c.r[4] * y) + c.r[5] * zz) + c.t[1];
    const float vz = ((c.r[6] * x + c.r[7] * y) + c.r[8] * zz) + c.t[2];
    float z        = std::fmax(vz, 0.f);  // PointRendererHelper.h:191-192
    if (!(z > 0.f)) return false;        // z == 0 (also NaN)
    float nx = vx / vz;                   // DivideByZ, PointRendererHelper.h:205
    float ny = vy / vz;
    if (c.has_dist) distort(c.dist, nx, ny, nx, ny);  // distortNormalizedPoint, PointRendererHelper.h:207
    const float u  = (c.fx * nx + c.s * ny) + c.cx;  // K.normalizedToImage, PointRendererHelper.h:214
    const float w  = c.fy * ny + c.cy;
    const float* k = v.crop_transform;
    float ipx      = (k[0] * u + k[4] * w) + k[2];  // crop_transform.normalizedToImage, RenderForward.cu:155
    float ipy      = k[1] * w + k[3];
    const float ccx = (float)(v.w / 2), ccy = (float)(v.h / 2);  // integer halves, RenderForward.cu:156
    const float dx = ipx - ccx, dy = ipy - ccy;
    const float rx = v.crop_rotation[0] * dx + v.crop_rotation[1] * dy;  // RenderForward.cu:110-116
    const float ry = v.crop_rotation[2] * dx + v.crop_rotation[3] * dy;
    o.ipx          = rx + ccx;
    o.ipy          = ry + ccy;
    o.z            = z;
    o.radius       = ((c.fx * k[0]) * p4[3]) / z;  // RenderForward.cu:132
    return true;
}

inline uint32_t float_bits(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}

// Visits the pixel a point lands in, layer by layer. The loop of CountingPrepassMulti / CollectMulti:
// rendering/RenderForward.cu:855-903 and :1075-1096. __float2int_rn = round half to even = rintf in the default mode.
template <class F>
inline void for_each_layer_pixel(const Projected& pr, const Layers& ly, const vetrast_params& prm, F&& fn)
{
    float ipx = pr.ipx, ipy = pr.ipy, radius = pr.radius;
    for (int l = 0; l < ly.L; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
    {
        if (prm.drop_out_points_by_radius && radius < prm.drop_out_radius_threshold) break;
        const float fx = std::rint(ipx), fy = std::rint(ipy);
        // inImage2(y, x): 0 <= x < w and 0 <= y < h
        if (!(fx >= 0.f && fx < (float)ly.w[l] && fy >= 0.f && fy < (float)ly.h[l])) continue;
        fn(l, (int)fx, (int)fy);
    }
}

// BILINEAR_BLEND: visits the up to four pixels around a point, layer by layer, with the corner number
// y_j * 2 + x_i. The loops of CountingPrepassMulti<L,true> / CollectMulti<L,true>:
// rendering/RenderForward.cu:863-885 and :1097-1134. __float2int_rd = floor.
template <class F>
inline void for_each_layer_corner(const Projected& pr, const Layers& ly, const vetrast_params& prm, F&& fn)
{
    float ipx = pr.ipx, ipy = pr.ipy, radius = pr.radius;
    for (int l = 0; l < ly.L; ++l, radius *= 0.5f, ipx *= 0.5f, ipy *= 0.5f)
    {
        if (prm.drop_out_points_by_radius && radius < prm.drop_out_radius_threshold) break;
        const float fx = std::floor(ipx), fy = std::floor(ipy);
        for (int y_j = 0; y_j <= 1; ++y_j)
            for (int x_i = 0; x_i <= 1; ++x_i)
            {
                const float px = fx + (float)x_i, py = fy + (float)y_j;
                if (!(px >= 0.f && px < (float)ly.w[l] && py >= 0.f && py < (float)ly.h[l])) continue;
                fn(l, (int)px, (int)py, y_j * 2 + x_i);
            }
    }
}

// Image position of a projected point at layer l: l exact halvings (RenderForward.cu:856).
inline void layer_position(const Projected& pr, int l, float& ipx, float& ipy)
{
    ipx = pr.ipx;
    ipy = pr.ipy;
    for (int k = 0; k < l; ++k) ipx *= 0.5f, ipy *= 0.5f;
}

// compute_blending_fac, rendering/PointBlending.h:12-44: the four bilinear weights of a position and, optionally, their
// derivatives J[corner][0..1] with respect to (x, y).
inline void blending_fac(float u, float v, float fac[4], float J[4][2])
{
    const float sx = u - std::floor(u), sy = v - std::floor(v);
    fac[0] = (1 - sx) * (1 - sy);
    fac[1] = sx * (1 - sy);
    fac[2] = (1 - sx) * sy;
    fac[3] = sx * sy;
    if (J)
    {
        J[0][0] = sy - 1;
        J[0][1] = sx - 1;
        J[1][0] = 1 - sy;
        J[1][1] = -sx;
        J[2][0] = -sy;
        J[2][1] = 1 - sx;
        J[3][0] = sy;
        J[3][1] = sx;
    }
}

// exp and the logistic function from +, *, rint and one division only (library exp routines differ in the last bits
// between platforms): Cody-Waite reduction x = k ln2 + r, a degree-7 Taylor polynomial of e^r, scaling by 2^k through
// the exponent bits. Canonical arithmetic of the fused confidence activation.
inline float exp_canon(float x)
{
    x             = std::fmin(std::fmax(x, -87.f), 88.f);
    const float k = std::rint(x * 1.44269504088896341f);
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
    const uint32_t bits = (uint32_t)((int)k + 127) << 23;
    float scale;
    std::memcpy(&scale, &bits, 4);
    return p * scale;
}

inline float sigmoid_canon(float x)
{
    return 1.f / (1.f + exp_canon(-x));
}

// The tensors as the rasterizer blends them: NeuralPointTextureImpl::PrepareConfidence / PrepareTexture,
// models/NeuralTexture.h:38-55 (sigmoid((10 + narrowing) * confidence_raw); abs or clone of texture_raw and
// background_color_raw), when those steps are switched on in the params.
struct PreparedInputs
{
    std::vector<float> texture, confidence, background;
    vetrast_forward_args args;  // a copy that points to the prepared tensors, with the switches off
};

inline bool needs_preparation(const vetrast_params& p)
{
    return p.confidence_activation != 0 || p.texture_abs != 0;
}

inline void prepare_inputs(const vetrast_forward_args* a, PreparedInputs& o)
{
    const vetrast_params& p = a->params;
    const size_t N = (size_t)a->num_points, C = (size_t)p.num_texture_channels;
    o.args = *a;
    if (p.confidence_activation)
    {
        o.confidence.resize(N);
        for (size_t i = 0; i < N; ++i) o.confidence[i] = sigmoid_canon(p.confidence_scale * a->confidence[i]);
        o.args.confidence = o.confidence.data();
    }
    if (p.texture_abs)
    {
        o.texture.resize(C * N);
        for (size_t i = 0; i < C * N; ++i) o.texture[i] = std::fabs(a->texture[i]);
        o.background.resize(C);
        for (size_t i = 0; i < C; ++i) o.background[i] = std::fabs(a->background[i]);
        o.args.texture    = o.texture.data();
        o.args.background = o.background.data();
    }
    o.args.params.confidence_activation = 0;
    o.args.params.texture_abs           = 0;
}

inline float sign_of(float x)
{
    return x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f);  // torch's abs backward: grad * sign(x)
}

inline bool is_fuzzy(const vetrast_params& p)
{
    return p.render_mode == VETRAST_RENDER_FUZZY_BLEND;
}

inline bool is_bilinear(const vetrast_params& p)
{
    return p.render_mode == VETRAST_RENDER_BILINEAR_BLEND;
}

struct Scene
{
    const vetrast_forward_args* a;
    Layers ly;
    int64_t P;
    int64_t cap;
    std::vector<Prepared> cams;
};

int validate(const vetrast_forward_args* a)
{
    if (!a || !a->position || !a->texture || !a->confidence || !a->background || !a->poses_se3 || !a->intrinsics ||
        !a->views)
        return VETRAST_ERR_INVALID_ARG;
    const vetrast_params& p = a->params;
    if (a->num_points < 0 || a->num_views < 1) return VETRAST_ERR_INVALID_ARG;
    if (p.num_layers < 1 || p.num_layers > VETRAST_MAX_LAYERS) return VETRAST_ERR_INVALID_ARG;
    if (p.num_texture_channels < 1 || p.num_texture_channels > VETRAST_MAX_CHANNELS) return VETRAST_ERR_INVALID_ARG;
    if (p.check_normal) return VETRAST_ERR_UNSUPPORTED;
    if (p.render_mode != VETRAST_RENDER_FULL_BLEND && !is_bilinear(p) && !is_fuzzy(p))
        return VETRAST_ERR_UNSUPPORTED;
    if (is_bilinear(p) && a->num_points > (1 << 30)) return VETRAST_ERR_INVALID_ARG;  // id and corner share 32 key bits
    for (int b = 0; b < a->num_views; ++b)
    {
        const vetrast_view& v = a->views[b];
        if (v.camera_model_type != VETRAST_CAMERA_PINHOLE_DISTORTION) return VETRAST_ERR_UNSUPPORTED;
        if (v.w != a->views[0].w || v.h != a->views[0].h || v.w < 1 || v.h < 1) return VETRAST_ERR_INVALID_ARG;
        if (v.image_index < 0 || v.image_index >= a->num_poses) return VETRAST_ERR_INVALID_ARG;
        if (v.camera_index < 0 || v.camera_index >= a->num_cameras) return VETRAST_ERR_INVALID_ARG;
        if (!p.allow_distortion && !distortion_is_zero(a->intrinsics + 13 * (size_t)v.camera_index))
            return VETRAST_ERR_BAD_INPUT_DATA;
    }
    return VETRAST_OK;
}

Scene make_scene(const vetrast_forward_args* a)
{
    Scene s;
    s.a   = a;
    s.ly  = make_layers(a->views[0].w, a->views[0].h, a->params.num_layers);
    s.P   = s.ly.base[s.ly.L];
    s.cap = (int64_t)a->num_points * a->params.num_layers * (is_bilinear(a->params) ? 4 : 1);
    for (int b = 0; b < a->num_views; ++b)
    {
        const vetrast_view& v = a->views[b];
        s.cams.push_back(prepare(a->poses_se3 + 8 * (size_t)v.image_index, a->intrinsics + 13 * (size_t)v.camera_index));
    }
    return s;
}

// Point skipping shared by the counting and the collection pass: rendering/RenderForward.cu:829-833,168-176.
inline bool point_skipped(const vetrast_forward_args* a, int b, int i)
{
    if (a->dropout && a->dropout[(size_t)b * a->num_points + i] == 1.f) return true;
    const int ti = a->index ? a->index[i] : i;
    if (a->params.viewer_only && a->confidence[ti] < a->params.stability_cutoff_value) return true;
    return false;
}

// compute_blend / compute_new_alphadest. rendering/PointBlending.h:90-94,116-119
inline float compute_blend(float alpha_dest, float alpha_s, float color, float color_dest)
{
    return alpha_dest * alpha_s * color + color_dest;  // (alpha_dest*alpha_s)*color, then + dest; no contraction
}
inline float compute_new_alphadest(float alphadest_old, float alpha_s)
{
    return (1 - alpha_s) * alphadest_old;
}

inline void atomic_add(float* p, float v, bool parallel)
{
    if (parallel)
    {
#pragma omp atomic
        *p += v;
    }
    else
        *p += v;
}

struct PointGrad
{
    float gp[3];
    double gpose[6];
    float gk[5];
    float gdis[8];
};

// ProjectPointPinholeBackward, rendering/PointRendererHelper.h:317-372 (J_p_dis = I for a camera without distortion), with the
// crop transform scaled by 0.5^layer (all five coefficients, rendering/RenderBackward.cu:1381-1385 and :3100-3106):
// image-space gradient (gxp, gyp) of layer l -> gradients of the point, the pose tangent and fx, fy, cx, cy, s.
// J_point = R, J_p_div = [1/z 0 -x/z^2; 0 1/z -y/z^2].
// with_distortion: the camera model carries the distortion step (vetrast_params.allow_distortion), so its Jacobians
// take part even where every coefficient is zero: d(xd, yd)/d(x, y) is then exactly the identity and the coefficient
// gradients J_dis_dis^T (rendering/PointRendererHelper.h:346-368) are not zero (x r^2 and so on).
inline PointGrad project_point_backward(const Prepared& cam, const vetrast_view& v, int l, const float* p4, float gxp,
                                        float gyp, bool with_distortion)
{
    PointGrad o;
    for (int k = 0; k < 3; ++k) o.gp[k] = 0.f;
    for (int k = 0; k < 6; ++k) o.gpose[k] = 0.0;
    for (int k = 0; k < 5; ++k) o.gk[k] = 0.f;
    for (int k = 0; k < 8; ++k) o.gdis[k] = 0.f;
    const float scale = powf(0.5f, float(l));
    const float cfx = v.crop_transform[0] * scale, cfy = v.crop_transform[1] * scale, cs = v.crop_transform[4] * scale;
    const float px = p4[0], py = p4[1], pz = p4[2];
    const float vx = ((cam.r[0] * px + cam.r[1] * py) + cam.r[2] * pz) + cam.t[0];
    const float vy = ((cam.r[3] * px + cam.r[4] * py) + cam.r[5] * pz) + cam.t[1];
    const float vz = ((cam.r[6] * px + cam.r[7] * py) + cam.r[8] * pz) + cam.t[2];
    if (vz > 0.f)
    {
        const float ar = v.crop_rotation[0] * gxp + v.crop_rotation[2] * gyp;  // J_rot^T grad
        const float br = v.crop_rotation[1] * gxp + v.crop_rotation[3] * gyp;
        const float a2 = cfx * ar;  // J_p_K2^T
        const float b2 = cs * ar + cfy * br;
        float d0 = cam.fx * a2;  // J_p_K1^T
        float d1 = cam.s * a2 + cam.fy * b2;
        float nx = vx / vz, ny = vy / vz;  // the point K is applied to
        if (cam.has_dist || with_distortion)
        {
            // J_dis_dis^T and J_p_dis^T (rendering/PointRendererHelper.h:346-368)
            float J[4], Jd[16], xd, yd;
            distort(cam.dist, nx, ny, xd, yd, J, Jd);
            for (int k = 0; k < 8; ++k) o.gdis[k] = Jd[2 * k] * d0 + Jd[2 * k + 1] * d1;
            const float n0 = J[0] * d0 + J[2] * d1, n1 = J[1] * d0 + J[3] * d1;
            d0 = n0, d1 = n1;
            nx = xd, ny = yd;
        }
        const float iz = 1.f / vz;
        const float e0 = iz * d0, e1 = iz * d1;
        const float e2 = (-vx * iz * iz) * d0 + (-vy * iz * iz) * d1;
        o.gp[0]        = (cam.r[0] * e0 + cam.r[3] * e1) + cam.r[6] * e2;  // R^T
        o.gp[1]        = (cam.r[1] * e0 + cam.r[4] * e1) + cam.r[7] * e2;
        o.gp[2]        = (cam.r[2] * e0 + cam.r[5] * e1) + cam.r[8] * e2;
        // J_pose^T e with J_pose = [I | -[view_p]x]: the tangent (translation, rotation) acts on the left,
        // pose <- exp(tangent) * pose (ApplyTangent, rendering/PointRenderer.cu:1325-1341)
        o.gpose[0] = e0;
        o.gpose[1] = e1;
        o.gpose[2] = e2;
        o.gpose[3] = vy * e2 - vz * e1;  // view_p x e
        o.gpose[4] = vz * e0 - vx * e2;
        o.gpose[5] = vx * e1 - vy * e0;
        // J_k_K1^T grad_p_k2: image = (fx*nx + s*ny + cx, fy*ny + cy), columns fx, fy, cx, cy, s
        o.gk[0] = nx * a2;
        o.gk[1] = ny * b2;
        o.gk[2] = a2;
        o.gk[3] = b2;
        o.gk[4] = ny * a2;
    }
    return o;
}

// The per-fragment scatter of rendering/RenderBackward.cu:1401-1459 (FULL_BLEND) and :3117-3175 (BILINEAR_BLEND); the
// two differ in what they add to the pose count per fragment (1/1024 there, 1 here).
inline void scatter_point_grad(const vetrast_backward_args* g, const vetrast_view& v, int point_id, const PointGrad& pg,
                               float pose_count_step, float k_factor, bool par)
{
    if (g->grad_points)
    {
        for (int k = 0; k < 3; ++k) atomic_add(&g->grad_points[4 * (size_t)point_id + k], pg.gp[k], par);
        atomic_add(&g->grad_point_count[point_id], 1.f, par);
    }
    if (g->grad_pose)
    {
        for (int k = 0; k < 6; ++k)
        {
            double* dst = &g->grad_pose[6 * (size_t)v.image_index + k];
            if (par)
            {
#pragma omp atomic
                *dst += pg.gpose[k];
            }
            else
                *dst += pg.gpose[k];
        }
        atomic_add(&g->grad_pose_count[v.image_index], pose_count_step, par);
    }
    if (g->grad_intrinsics)  // g_k(4) *= 0 removes the skew
    {
        float gk[5] = {pg.gk[0], pg.gk[1], pg.gk[2], pg.gk[3], pg.gk[4]};
        gk[4] *= 0;
        for (int k = 0; k < 5; ++k)
            atomic_add(&g->grad_intrinsics[13 * (size_t)v.camera_index + k], k_factor * gk[k], par);
        // the eight distortion columns, scaled as rendering/RenderBackward.cu:1438-1455 scales them (zero for a camera
        // without distortion)
        if (g->fwd.params.allow_distortion)
        {
            const float w8[8] = {1.f, 1.f, 0.25f, 0.1f, 0.1f, 0.1f, 0.1f, 0.1f};
            for (int k = 0; k < 8; ++k)
                atomic_add(&g->grad_intrinsics[13 * (size_t)v.camera_index + 5 + k],
                           g->fwd.params.distortion_gradient_factor * (pg.gdis[k] * w8[k]), par);
        }
        atomic_add(&g->grad_intrinsics_count[v.camera_index], 1.f / 1024.f, par);
    }
}

// One pixel of BlendBackwardsBilinear<C>, rendering/RenderBackward.cu:2893-3232, followed literally including the
// O(n^2) inner loop. sum_back is the per-fragment gradient_sum_backwards row (indexed by list position).
void bilinear_pixel_backward(const vetrast_backward_args* g, const Scene& s, int b, int l, int gx, int gy,
                             uint32_t offset, int size_of_chunk, const uint64_t* frag, const float* G, float* sum_back,
                             bool need_point_gradients, bool par)
{
    const vetrast_forward_args* a = &g->fwd;
    const vetrast_params& pr      = a->params;
    const Prepared& cam           = s.cams[b];
    const vetrast_view& v         = a->views[b];
    const int N = a->num_points, C = pr.num_texture_channels;
    const int lw = s.ly.w[l], lh = s.ly.h[l];
    const size_t plane = (size_t)lw * lh;
    auto get_point_id      = [&](uint32_t pos) { return (int)((uint32_t)frag[pos] >> 2); };
    auto sample_texture_id = [&](uint32_t pos) {
        const int id = get_point_id(pos);
        return a->index ? a->index[id] : id;
    };
    // per_point_data of the fragment: (uv, corner); uv is the projection of the point at this layer again
    auto get_uv = [&](uint32_t pos, float& u, float& w2) {
        Projected pp;
        project(cam, v, a->position + 4 * (size_t)get_point_id(pos), pp);
        layer_position(pp, l, u, w2);
    };
    auto get_subpixel_weight = [&](uint32_t pos) {
        float u, w2, fac[4];
        get_uv(pos, u, w2);
        blending_fac(u, w2, fac, nullptr);
        return fac[(uint32_t)frag[pos] & 3u];
    };
    {
        float alpha_dest    = 1.f;
        const int list_size = pr.use_environment_map ? size_of_chunk : size_of_chunk + 1;
        for (int i = 0; i < list_size; ++i)
        {
            const bool is_foreground       = i != size_of_chunk;
            const uint32_t full_buffer_pos = offset + (uint32_t)i;
            int texture_index              = 0;
            if (is_foreground) texture_index = sample_texture_id(full_buffer_pos);
            float alpha_val = 1.f;
            if (is_foreground) alpha_val = get_subpixel_weight(full_buffer_pos) * a->confidence[texture_index];
            float colors[VETRAST_MAX_CHANNELS], grad_in[VETRAST_MAX_CHANNELS];
            for (int ci = 0; ci < C; ++ci)
                colors[ci] = is_foreground ? a->texture[(size_t)ci * N + texture_index] : a->background[ci];
            float g_alpha = 0;
            for (int ci = 0; ci < C; ++ci)
            {
                grad_in[ci]   = G[ci * plane + (size_t)gy * lw + gx];
                float g_col   = alpha_dest * alpha_val * grad_in[ci];
                float* target = is_foreground ? &g->grad_texture[(size_t)ci * N + texture_index] : &g->grad_background[ci];
                atomic_add(target, g_col, par);
                g_alpha += colors[ci] * grad_in[ci];
            }
            g_alpha *= alpha_dest;
            if (is_foreground) sum_back[full_buffer_pos] += g_alpha;  // :2987 (guarded here, unlike FULL_BLEND)
            for (int j = 0; j < i; ++j)
            {
                const uint32_t pos_iter    = offset + (uint32_t)j;
                const int texture_iter     = sample_texture_id(pos_iter);
                const float alpha_val_iter = get_subpixel_weight(pos_iter) * a->confidence[texture_iter];
                float g_iter               = 0;
                for (int ci = 0; ci < C; ++ci)
                {
                    const float epsilon = 1e-9;
                    float g_alpha_iter  = (grad_in[ci] * colors[ci] * alpha_dest * alpha_val / (1 - alpha_val_iter + epsilon));
                    g_iter -= g_alpha_iter;
                }
                sum_back[pos_iter] += g_iter;
            }
            alpha_dest = compute_new_alphadest(alpha_dest, alpha_val);
            if (alpha_dest < 0.001)  // :3014-3019: later fragments took no part in the forward blend either
            {
                if (is_foreground) size_of_chunk = i + 1;
                break;
            }
        }
    }
    // confidence and position gradients, only for pixels more than 2 away from the border (:3044)
    const int edge = std::min(std::min(gx, gy), std::min(lw - 1 - gx, lh - 1 - gy));
    if (!(edge > 2)) return;
    for (int i = 0; i < size_of_chunk; ++i)
    {
        const uint32_t full_buffer_pos = offset + (uint32_t)i;
        const int texture_index        = sample_texture_id(full_buffer_pos);
        float u, w2, fac[4], J[4][2];
        get_uv(full_buffer_pos, u, w2);
        const int blend_index  = (int)((uint32_t)frag[full_buffer_pos] & 3u);
        const float grad_alpha = sum_back[full_buffer_pos];
        blending_fac(u, w2, fac, J);
        atomic_add(&g->grad_confidence[texture_index], fac[blend_index] * grad_alpha, par);  // dA/dc = blend factor
        if (!need_point_gradients) continue;
        const float grad_blend_single = a->confidence[texture_index] * grad_alpha;  // dA/db = confidence
        // dR_dp = J_uv_b^T * grad_blending, grad_blending zero but for this corner (:3083-3088)
        const float gxp    = J[blend_index][0] * grad_blend_single;
        const float gyp    = J[blend_index][1] * grad_blend_single;
        const int point_id = get_point_id(full_buffer_pos);
        const PointGrad pg = project_point_backward(cam, v, l, a->position + 4 * (size_t)point_id, gxp, gyp, a->params.allow_distortion != 0);
        scatter_point_grad(g, v, point_id, pg, 1.f, pr.K_gradient_factor, par);  // pose count +1 here (:3146)
    }
}

// Value gradients of one pixel in FUZZY_BLEND: the first half of BlendBackwardsFuzzy<C>,
// rendering/RenderBackward.cu:570-727, literally. Unlike the forward kernel this one starts every new bucket at the
// depth of its first fragment (:712), so buckets form all along the list, the background (depth MAX_DEPTH_CONST = 1e5)
// closes the last one and is a bucket of its own. A bucket's gradient is shared out evenly among its elements; every
// element in front of a bucket receives the bucket's whole transmittance term divided by (1 - mean confidence of the
// element's own bucket) (:654-672, the mean confidences are the values the kernel parks in gradient_sum_backwards).
// The position part of that kernel (:729-1080) computes the same heuristic as BlendBackwards2, so the caller shares it.
void fuzzy_pixel_value_gradients(const vetrast_backward_args* g, int N, int C, const float* G, size_t plane,
                                 size_t pixel, uint32_t offset, int size_of_chunk, const uint64_t* frag, bool par)
{
    const vetrast_forward_args* a = &g->fwd;
    const vetrast_params& pr      = a->params;
    const float MAX_DEPTH_CONST   = 100000.f;  // rendering/RenderConstants.h:30
    auto texture_index_at         = [&](int pos) {
        const int id = (int)(uint32_t)frag[pos];
        return a->index ? a->index[id] : id;
    };
    auto depth_at = [&](int pos) {
        const uint32_t bits = (uint32_t)(frag[pos] >> 32);
        float d;
        std::memcpy(&d, &bits, 4);
        return d;
    };
    std::vector<float> saved_confidence((size_t)size_of_chunk + 1, 0.f);  // gradient_sum_backwards row C of this pixel
    float accumulation_last_min_d = 0.f;
    float accumulation_desc[VETRAST_MAX_CHANNELS];
    float accumulation_conf_val = 0.f;
    int accumulation_num_elems  = 0;
    int accum_start_index       = 0;
    float alpha_dest            = 1.f;
    for (int ci = 0; ci < C; ++ci) accumulation_desc[ci] = 0.f;

    auto accumulateCollectedBackwards = [&]() {
        const float inv_weight     = 1.f / float(accumulation_num_elems);
        const float confidence_val = accumulation_conf_val * inv_weight;
        float colors[VETRAST_MAX_CHANNELS], grad_in[VETRAST_MAX_CHANNELS], g_colors[VETRAST_MAX_CHANNELS];
        float g_alpha = 0;
        for (int ci = 0; ci < C; ++ci)
        {
            colors[ci]   = accumulation_desc[ci] * inv_weight;
            grad_in[ci]  = G[ci * plane + pixel];
            g_colors[ci] = alpha_dest * confidence_val * grad_in[ci];
            g_alpha += colors[ci] * grad_in[ci];
        }
        g_alpha *= alpha_dest;
        for (int t = accum_start_index; t < accum_start_index + accumulation_num_elems; ++t)
        {
            const bool is_foreground = t != size_of_chunk;
            const int texture_index  = is_foreground ? texture_index_at((int)offset + t) : 0;
            for (int ci = 0; ci < C; ++ci)
            {
                float* target = is_foreground ? &g->grad_texture[(size_t)ci * N + texture_index] : &g->grad_background[ci];
                atomic_add(target, g_colors[ci] * inv_weight, par);
            }
            if (is_foreground)
            {
                atomic_add(&g->grad_confidence[texture_index], g_alpha * inv_weight, par);
                saved_confidence[(size_t)t] = confidence_val;
            }
        }
        for (int j = 0; j < accum_start_index; ++j)
        {
            const int texture_index_iter    = texture_index_at((int)offset + j);
            const float confidence_val_iter = saved_confidence[(size_t)j];
            float g_iter                    = 0;
            for (int ci = 0; ci < C; ++ci)
            {
                const float epsilon = 1e-9;
                float g_alpha_iter =
                    (grad_in[ci] * colors[ci] * alpha_dest * confidence_val / (1 - confidence_val_iter + epsilon));
                g_iter -= g_alpha_iter;
            }
            atomic_add(&g->grad_confidence[texture_index_iter], g_iter, par);
        }
        alpha_dest = compute_new_alphadest(alpha_dest, confidence_val);
    };

    const int list_size = pr.use_environment_map ? size_of_chunk : size_of_chunk + 1;
    for (int i = 0; i < list_size; ++i)
    {
        const bool is_foreground = i != size_of_chunk;
        const float d            = is_foreground ? depth_at((int)offset + i) : MAX_DEPTH_CONST;
        if (!(d - accumulation_last_min_d < pr.depth_accept_blend))
        {
            if (i != 0) accumulateCollectedBackwards();
            accumulation_conf_val  = 0.f;
            accumulation_num_elems = 0;
            for (int ci = 0; ci < C; ++ci) accumulation_desc[ci] = 0.f;
            accumulation_last_min_d = d;
            accum_start_index       = i;
        }
        const int texture_index = is_foreground ? texture_index_at((int)offset + i) : 0;
        accumulation_conf_val += is_foreground ? a->confidence[texture_index] : 1.f;
        for (int ci = 0; ci < C; ++ci)
            accumulation_desc[ci] += is_foreground ? a->texture[(size_t)ci * N + texture_index] : a->background[ci];
        ++accumulation_num_elems;
    }
    if (accumulation_num_elems > 0) accumulateCollectedBackwards();
}

}  // namespace

// out26: rotation rows with the translation in the fourth column (12), fx fy cx cy s (5), the eight distortion
// coefficients, and 1 if any of them is not zero
extern "C" int vetref_prepare_view(const double* pose8, const float* intrinsics13, float* out17)
{
    Prepared p = prepare(pose8, intrinsics13);
    for (int k = 0; k < 8; ++k) out17[17 + k] = p.dist[k];
    out17[25] = p.has_dist ? 1.f : 0.f;
    for (int r = 0; r < 3; ++r)
    {
        for (int c = 0; c < 3; ++c) out17[4 * r + c] = p.r[3 * r + c];
        out17[4 * r + 3] = p.t[r];
    }
    out17[12] = p.fx;
    out17[13] = p.fy;
    out17[14] = p.cx;
    out17[15] = p.cy;
    out17[16] = p.s;
    return 0;
}

extern "C" int vetref_project_point(const float* m, const vetrast_view* view, const float* position4, float* ip_z_r)
{
    Prepared p;
    for (int r = 0; r < 3; ++r)
    {
        for (int c = 0; c < 3; ++c) p.r[3 * r + c] = m[4 * r + c];
        p.t[r] = m[4 * r + 3];
    }
    p.fx = m[12];
    p.fy = m[13];
    p.cx = m[14];
    p.cy = m[15];
    p.s  = m[16];
    for (int k = 0; k < 8; ++k) p.dist[k] = m[17 + k];
    p.has_dist = m[25] != 0.f;
    Projected o;
    if (!project(p, *view, position4, o)) return 0;
    ip_z_r[0] = o.ipx;
    ip_z_r[1] = o.ipy;
    ip_z_r[2] = o.z;
    ip_z_r[3] = o.radius;
    return 1;
}

// Forward pass. Host sequence of BlendPointCloudForward, rendering/PointRenderer.cu:768-899:
// counting pass, exclusive scan, collection pass, per-pixel sort, blend.
extern "C" int vetref_forward(const vetrast_forward_args* a, uint32_t* offsets, uint64_t* fragments,
                              float* transmittance, float* weight, uint32_t* kept, int num_threads)
{
    int st = validate(a);
    if (st != VETRAST_OK) return st;
    if (needs_preparation(a->params))
    {
        PreparedInputs prep;
        prepare_inputs(a, prep);
        return vetref_forward(&prep.args, offsets, fragments, transmittance, weight, kept, num_threads);
    }
    if (!offsets || !fragments || !weight) return VETRAST_ERR_INVALID_ARG;
    for (int l = 0; l < a->params.num_layers; ++l)
        if (!a->out[l]) return VETRAST_ERR_INVALID_ARG;
    Scene s                  = make_scene(a);
    const int N              = a->num_points;
    const int C              = a->params.num_texture_channels;
    const int K              = a->params.debug_max_list_length;
    const vetrast_params& pr = a->params;
    const bool par           = num_threads > 1;
    const bool bilinear      = is_bilinear(pr);
    const bool fuzzy         = is_fuzzy(pr);
#ifdef _OPENMP
    omp_set_num_threads(num_threads > 0 ? num_threads : 1);
#endif

    for (int b = 0; b < a->num_views; ++b)
    {
        const Prepared& cam   = s.cams[b];
        const vetrast_view& v = a->views[b];
        uint32_t* off         = offsets + (size_t)b * (s.P + 1);
        uint64_t* frag        = fragments + (size_t)b * s.cap;
        float* wgt            = weight + (size_t)b * s.P;
        uint32_t* kept_b      = kept ? kept + (size_t)b * s.P : nullptr;
        std::vector<uint32_t> count((size_t)s.P, 0u), cursor((size_t)s.P, 0u);

        // CountingPrepassMulti<L,false>, rendering/RenderForward.cu:806-905 (the depth atomicMin image is not
        // read by FULL_BLEND and is not produced here).
#pragma omp parallel for schedule(static) if (par)
        for (int i = 0; i < N; ++i)
        {
            if (point_skipped(a, b, i)) continue;
            Projected p;
            if (!project(cam, v, a->position + 4 * (size_t)i, p)) continue;
            auto hit = [&](int l, int x, int y) {
                uint32_t* c = &count[(size_t)(s.ly.base[l] + (int64_t)y * s.ly.w[l] + x)];
                if (par)
                    __atomic_fetch_add(c, 1u, __ATOMIC_RELAXED);
                else
                    ++*c;
            };
            if (bilinear)
                for_each_layer_corner(p, s.ly, pr, [&](int l, int x, int y, int) { hit(l, x, y); });
            else
                for_each_layer_pixel(p, s.ly, pr, hit);
        }

        // thrust::exclusive_scan per layer, rendering/PointRenderer.cu:799-813. The layers are concatenated here,
        // so a layer's list positions are shifted by the fragments of the finer layers; list contents are the same.
        uint32_t run = 0;
        for (int64_t q = 0; q < s.P; ++q)
        {
            off[q] = run;
            run += count[(size_t)q];
        }
        off[s.P] = run;

        // CollectMulti<L,false>, rendering/RenderForward.cu:1011-1096: slot = scan[pixel] + atomicAdd(counter, 1),
        // record = (depth bits, point id).
#pragma omp parallel for schedule(static) if (par)
        for (int i = 0; i < N; ++i)
        {
            if (point_skipped(a, b, i)) continue;
            Projected p;
            if (!project(cam, v, a->position + 4 * (size_t)i, p)) continue;
            // Record: depth bits above the point id. In BILINEAR_BLEND the reference keeps (id, ip, corner) in a side
            // table addressed through the record (RenderForward.cu:1112-1128); here the corner rides in the two low
            // key bits next to the id, and ip is the (deterministic) projection of that point again.
            auto put = [&](int l, int x, int y, uint32_t low) {
                const size_t q = (size_t)(s.ly.base[l] + (int64_t)y * s.ly.w[l] + x);
                uint32_t slot;
                if (par)
                    slot = __atomic_fetch_add(&cursor[q], 1u, __ATOMIC_RELAXED);
                else
                    slot = cursor[q]++;
                frag[off[q] + slot] = ((uint64_t)float_bits(p.z) << 32) | low;
            };
            if (bilinear)
                for_each_layer_corner(p, s.ly, pr,
                                      [&](int l, int x, int y, int corner) { put(l, x, y, ((uint32_t)i << 2) | (uint32_t)corner); });
            else
                for_each_layer_pixel(p, s.ly, pr, [&](int l, int x, int y) { put(l, x, y, (uint32_t)i); });
        }

        // SortMulti, rendering/RenderForward.cu:1277-1300 and rendering/AlphaListSort.cu:23-32: ascending depth per
        // pixel list. The reference leaves equal depths in arrival order; the point id in the low key bits makes
        // the order total. BlendMulti, rendering/RenderForward.cu:1303-1357.
        for (int l = 0; l < s.ly.L; ++l)
        {
            const int lw = s.ly.w[l], lh = s.ly.h[l];
            float* out = a->out[l] + (size_t)b * C * lw * lh;
#pragma omp parallel for schedule(dynamic, 8) if (par)
            for (int y = 0; y < lh; ++y)
                for (int x = 0; x < lw; ++x)
                {
                    const size_t q   = (size_t)(s.ly.base[l] + (int64_t)y * lw + x);
                    const uint32_t o = off[q];
                    const int n      = (int)(off[q + 1] - o);
                    std::sort(frag + o, frag + o + n);
                    int size_of_chunk = n;
                    if (K > 0) size_of_chunk = std::min(K, size_of_chunk);  // RenderForward.cu:1317-1318
                    float alpha_dest = 1.f;
                    float color_out[VETRAST_MAX_CHANNELS];
                    for (int ci = 0; ci < C; ++ci) color_out[ci] = 0.f;
                    int blended = 0;  // fragments that took part
                    if (fuzzy)
                    {
                        // BlendMultiFuzzy, rendering/RenderForward.cu:1393-1503: fragments are collected while their
                        // depth stays within depth_accept_blend of the first one of the bucket, the bucket is blended
                        // as one fragment with the mean confidence and the mean descriptor. After the first bucket
                        // the reference resets its reference depth to -100000 (:1468), not to the next depth, so
                        // every later fragment closes the bucket before it: only the nearest bucket averages.
                        float accumulation_last_min_d = 0.f;
                        float accumulation_desc[VETRAST_MAX_CHANNELS];
                        float accumulation_conf_val = 0.f;
                        int accumulation_num_elems  = 0;
                        for (int ci = 0; ci < C; ++ci) accumulation_desc[ci] = 0.f;
                        auto accumulateCollected = [&]() {
                            const float confidence_val = accumulation_conf_val / float(accumulation_num_elems);
                            for (int ci = 0; ci < C; ++ci)
                            {
                                const float color = accumulation_desc[ci] / float(accumulation_num_elems);
                                color_out[ci]     = compute_blend(alpha_dest, confidence_val, color, color_out[ci]);
                            }
                            alpha_dest = compute_new_alphadest(alpha_dest, confidence_val);
                        };
                        for (int i = 0; i < size_of_chunk; ++i)
                        {
                            const int point_id      = (int)(uint32_t)frag[o + i];
                            const int texture_index = a->index ? a->index[point_id] : point_id;
                            const uint32_t dbits    = (uint32_t)(frag[o + i] >> 32);
                            float d;
                            std::memcpy(&d, &dbits, 4);
                            if (accumulation_last_min_d == 0.f) accumulation_last_min_d = d;
                            if (!(d - accumulation_last_min_d < pr.depth_accept_blend))
                            {
                                accumulateCollected();
                                accumulation_last_min_d = -100000.f;
                                accumulation_conf_val   = 0.f;
                                accumulation_num_elems  = 0;
                                for (int ci = 0; ci < C; ++ci) accumulation_desc[ci] = 0.f;
                            }
                            // saved for inspection only (the fuzzy backward pass recomputes its own chain): the
                            // transmittance in front of the bucket the fragment joins
                            if (transmittance) transmittance[(size_t)b * s.cap + o + i] = alpha_dest;
                            accumulation_conf_val += a->confidence[texture_index];
                            for (int ci = 0; ci < C; ++ci)
                                accumulation_desc[ci] += a->texture[(size_t)ci * N + texture_index];
                            ++accumulation_num_elems;
                            ++blended;
                        }
                        if (accumulation_num_elems > 0) accumulateCollected();
                    }
                    for (int i = 0; i < size_of_chunk && !fuzzy; ++i)
                    {
                        const uint32_t low      = (uint32_t)frag[o + i];
                        const int point_id      = bilinear ? (int)(low >> 2) : (int)low;
                        const int texture_index = a->index ? a->index[point_id] : point_id;
                        float conf              = a->confidence[texture_index];
                        if (bilinear)
                        {
                            // BlendMultiBilinear, rendering/RenderForward.cu:1539-1644: alpha = bilinear weight of
                            // this pixel's corner x confidence
                            Projected pp;
                            project(cam, v, a->position + 4 * (size_t)point_id, pp);
                            float u, w2, fac[4];
                            layer_position(pp, l, u, w2);
                            blending_fac(u, w2, fac, nullptr);
                            conf = fac[low & 3u] * conf;
                        }
                        if (transmittance) transmittance[(size_t)b * s.cap + o + i] = alpha_dest;
                        for (int ci = 0; ci < C; ++ci)
                        {
                            const float color = a->texture[(size_t)ci * N + texture_index];
                            color_out[ci]     = compute_blend(alpha_dest, conf, color, color_out[ci]);
                        }
                        alpha_dest = compute_new_alphadest(alpha_dest, conf);
                        ++blended;
                        if (bilinear && alpha_dest < 0.001) break;  // RenderForward.cu:1626 (compared as double)
                    }
                    if (kept_b) kept_b[q] = (uint32_t)blended;
                    for (int ci = 0; ci < C; ++ci)
                    {
                        if (!pr.use_environment_map && (!bilinear || alpha_dest >= 0.001))  // :1633-1636
                            color_out[ci] = compute_blend(alpha_dest, 1.f, a->background[ci], color_out[ci]);
                        out[((size_t)ci * lh + y) * lw + x] = color_out[ci];
                    }
                    wgt[q] = alpha_dest;  // atomicAdd onto a zeroed image, RenderForward.cu:1355-1356
                    // CreateMask, rendering/PointRenderer.cu:216-235
                    if (pr.output_background_mask && a->out_mask[l])
                        a->out_mask[l][((size_t)b * lh + y) * lw + x] =
                            (alpha_dest == 0.f) ? pr.output_background_mask_value : 1.f;
                }
        }
    }
    return VETRAST_OK;
}

// Backward pass. BlendBackwards2<C>, rendering/RenderBackward.cu:1083-1513, followed literally including the O(n^2)
// inner loop; host part rendering/PointRenderer.cu:1111-1323 (zeroed gradient buffers, NormalizeGradient).
extern "C" int vetref_backward(const vetrast_backward_args* g, const uint32_t* offsets, const uint64_t* fragments,
                               int num_threads)
{
    const vetrast_forward_args* a = &g->fwd;
    int st                        = validate(a);
    if (st != VETRAST_OK) return st;
    if (!g->grad_texture || !g->grad_confidence || !g->grad_background) return VETRAST_ERR_INVALID_ARG;
    if (needs_preparation(a->params))
    {
        // gradients of the prepared tensors first, then the chain rule of the preparation steps (what autograd does
        // with torch::sigmoid and torch::abs in the reference)
        PreparedInputs prep;
        prepare_inputs(a, prep);
        vetrast_backward_args g2 = *g;
        g2.fwd                   = prep.args;
        st                       = vetref_backward(&g2, offsets, fragments, num_threads);
        if (st != VETRAST_OK) return st;
        const vetrast_params& p = a->params;
        const size_t N = (size_t)a->num_points, C = (size_t)p.num_texture_channels;
        if (p.confidence_activation)
            for (size_t i = 0; i < N; ++i)
            {
                const float sgm = prep.confidence[i];
                g->grad_confidence[i] = g->grad_confidence[i] * ((p.confidence_scale * sgm) * (1.f - sgm));
            }
        if (p.texture_abs)
        {
            for (size_t i = 0; i < C * N; ++i) g->grad_texture[i] = g->grad_texture[i] * sign_of(a->texture[i]);
            for (size_t i = 0; i < C; ++i) g->grad_background[i] = g->grad_background[i] * sign_of(a->background[i]);
        }
        return VETRAST_OK;
    }
    if (g->grad_points && !g->grad_point_count) return VETRAST_ERR_INVALID_ARG;
    if (g->grad_pose && !g->grad_pose_count) return VETRAST_ERR_INVALID_ARG;
    if (g->grad_intrinsics && !g->grad_intrinsics_count) return VETRAST_ERR_INVALID_ARG;
    Scene s                  = make_scene(a);
    const int N              = a->num_points;
    const int C              = a->params.num_texture_channels;
    const int K              = a->params.debug_max_list_length;
    const vetrast_params& pr = a->params;
    const bool par           = num_threads > 1;
#ifdef _OPENMP
    omp_set_num_threads(num_threads > 0 ? num_threads : 1);
#endif
    if (g->grad_pose)
    {
        std::fill(g->grad_pose, g->grad_pose + (size_t)6 * a->num_poses, 0.0);
        std::fill(g->grad_pose_count, g->grad_pose_count + a->num_poses, 0.f);
    }
    if (g->grad_intrinsics)
    {
        std::fill(g->grad_intrinsics, g->grad_intrinsics + (size_t)13 * a->num_cameras, 0.f);
        std::fill(g->grad_intrinsics_count, g->grad_intrinsics_count + a->num_cameras, 0.f);
    }
    // zeros_like of every gradient tensor, rendering/PointRenderer.cu:267-277
    std::fill(g->grad_texture, g->grad_texture + (size_t)C * N, 0.f);
    std::fill(g->grad_confidence, g->grad_confidence + N, 0.f);
    std::fill(g->grad_background, g->grad_background + C, 0.f);
    if (g->grad_points)
    {
        std::fill(g->grad_points, g->grad_points + (size_t)4 * N, 0.f);
        std::fill(g->grad_point_count, g->grad_point_count + N, 0.f);
    }
    const bool need_point_gradients = pr.need_point_gradient && (g->grad_points || g->grad_pose || g->grad_intrinsics);

    const bool bilinear = is_bilinear(pr);
    const bool fuzzy    = is_fuzzy(pr);
    // gradient_sum_backwards: one zeroed float per fragment, rendering/PointRenderer.cu:1186-1200
    std::vector<float> sum_back(bilinear ? (size_t)s.cap : 0, 0.f);
    for (int b = 0; b < a->num_views; ++b)
    {
        const Prepared& cam   = s.cams[b];
        const vetrast_view& v = a->views[b];
        const uint32_t* off   = offsets + (size_t)b * (s.P + 1);
        const uint64_t* frag  = fragments + (size_t)b * s.cap;
        std::fill(sum_back.begin(), sum_back.end(), 0.f);
        for (int l = 0; l < s.ly.L; ++l)
        {
            const int lw = s.ly.w[l], lh = s.ly.h[l];
            const size_t plane = (size_t)lw * lh;
            const float* G     = g->grad_out[l] + (size_t)b * C * plane;
            const float* I     = a->out[l] + (size_t)b * C * plane;
#pragma omp parallel for schedule(dynamic, 8) if (par)
            for (int gy = 0; gy < lh; ++gy)
                for (int gx = 0; gx < lw; ++gx)
                {
                    const size_t q             = (size_t)(s.ly.base[l] + (int64_t)gy * lw + gx);
                    const uint32_t offset      = off[q];
                    int size_of_chunk          = (int)(off[q + 1] - offset);
                    if (K > 0) size_of_chunk   = std::min(K, size_of_chunk);  // RenderBackward.cu:1098-1100
                    if (bilinear)
                    {
                        bilinear_pixel_backward(g, s, b, l, gx, gy, offset, size_of_chunk, frag, G, sum_back.data() + 0,
                                                need_point_gradients, par);
                        continue;
                    }
                    auto sample_point_id       = [&](int pos) { return (int)(uint32_t)frag[pos]; };
                    auto sample_texture_index  = [&](int pos) {
                        const int id = sample_point_id(pos);
                        return a->index ? a->index[id] : id;
                    };
                    if (fuzzy)
                        fuzzy_pixel_value_gradients(g, N, C, G, plane, (size_t)gy * lw + gx, offset, size_of_chunk, frag, par);
                    // ---- value gradients, RenderBackward.cu:1118-1181
                    if (!fuzzy)
                    {
                        float alpha_dest = 1.f;
                        const int list_size = pr.use_environment_map ? size_of_chunk : size_of_chunk + 1;
                        for (int i = 0; i < list_size; ++i)
                        {
                            const bool is_foreground = i != size_of_chunk;
                            int texture_index        = 0;
                            if (is_foreground) texture_index = sample_texture_index(offset + i);
                            float confidence_val = 1.f;
                            if (is_foreground) confidence_val = a->confidence[texture_index];
                            float colors[VETRAST_MAX_CHANNELS], grad_in[VETRAST_MAX_CHANNELS];
                            for (int ci = 0; ci < C; ++ci)
                                colors[ci] = is_foreground ? a->texture[(size_t)ci * N + texture_index]
                                                           : a->background[ci];
                            float g_alpha = 0;
                            for (int ci = 0; ci < C; ++ci)
                            {
                                grad_in[ci]   = G[ci * plane + (size_t)gy * lw + gx];
                                float g_col   = alpha_dest * confidence_val * grad_in[ci];
                                float* target = is_foreground ? &g->grad_texture[(size_t)ci * N + texture_index]
                                                              : &g->grad_background[ci];
                                atomic_add(target, g_col, par);
                                g_alpha += colors[ci] * grad_in[ci];
                            }
                            g_alpha *= alpha_dest;
                            // The reference adds this unguarded, so the background element leaks into index 0
                            // (RenderBackward.cu:1130-1131,1157); kept behind a switch.
                            if (is_foreground || pr.quirk_background_confidence_leak)
                                atomic_add(&g->grad_confidence[texture_index], g_alpha, par);
                            for (int j = 0; j < i; ++j)
                            {
                                const int texture_index_iter    = sample_texture_index(offset + j);
                                const float confidence_val_iter = a->confidence[texture_index_iter];
                                float g_iter                    = 0;
                                for (int ci = 0; ci < C; ++ci)
                                {
                                    const float epsilon = 1e-9;
                                    float g_alpha_iter  = (grad_in[ci] * colors[ci] * alpha_dest * confidence_val /
                                                          (1 - confidence_val_iter + epsilon));
                                    g_iter -= g_alpha_iter;
                                }
                                atomic_add(&g->grad_confidence[texture_index_iter], g_iter, par);
                            }
                            alpha_dest = compute_new_alphadest(alpha_dest, confidence_val);
                        }
                    }
                    if (!need_point_gradients) continue;
                    // ---- position gradient heuristic, RenderBackward.cu:1185-1408
                    // distanceFromEdge(y, x) = min(x, y, w-1-x, h-1-y)
                    const int edge = std::min(std::min(gx, gy), std::min(lw - 1 - gx, lh - 1 - gy));
                    if (!(edge > 2)) continue;
                    for (int i = 0; i < size_of_chunk; ++i)
                    {
                        const int point_id      = sample_point_id(offset + i);
                        const int texture_index = a->index ? a->index[point_id] : point_id;
                        float dR_dpx = 0, dR_dpy = 0;
                        for (int ci = 0; ci < C; ++ci)
                        {
                            const float T_p   = a->texture[(size_t)ci * N + texture_index];
                            const float* Ic   = I + ci * plane;
                            const float* Gc   = G + ci * plane;
                            const size_t ctr  = (size_t)gy * lw + gx;
                            const float I_px0 = Ic[ctr - 1], I_px1 = Ic[ctr + 1];
                            const float I_py0 = Ic[ctr - lw], I_py1 = Ic[ctr + lw];
                            const float G_px0 = Gc[ctr - 1], G_px1 = Gc[ctr + 1];
                            const float G_py0 = Gc[ctr - lw], G_py1 = Gc[ctr + lw];
                            float dI_dp_at_px0 = -(T_p - I_px0) * G_px0;  // RenderBackward.cu:1364-1371
                            float dI_dp_at_px1 = (T_p - I_px1) * G_px1;
                            float dI_dp_at_py0 = -(T_p - I_py0) * G_py0;
                            float dI_dp_at_py1 = (T_p - I_py1) * G_py1;
                            dR_dpx += 0.5f * (dI_dp_at_px0 + dI_dp_at_px1);
                            dR_dpy += 0.5f * (dI_dp_at_py0 + dI_dp_at_py1);
                        }
                        const float gxp = dR_dpx / float(C), gyp = dR_dpy / float(C);  // :1374
                        const PointGrad pg =
                            project_point_backward(cam, v, l, a->position + 4 * (size_t)point_id, gxp, gyp, a->params.allow_distortion != 0);
                        scatter_point_grad(g, v, point_id, pg, 1.f / 1024.f, pr.K_gradient_factor, par);
                    }
                }
        }
    }

    // NormalizeGradientDevTensor<double,6> and NormalizeGradient<float,13>, rendering/PointRenderer.cu:1253-1308
    if (pr.camera_gradient_normalization)
    {
        if (g->grad_pose)
            for (int i = 0; i < a->num_poses; ++i)
            {
                const float c = g->grad_pose_count[i];
                if (c > 0)
                    for (int k = 0; k < 6; ++k) g->grad_pose[6 * (size_t)i + k] /= c;
            }
        if (g->grad_intrinsics)
            for (int i = 0; i < a->num_cameras; ++i)
            {
                const float c = g->grad_intrinsics_count[i];
                if (c > 0)
                    for (int k = 0; k < 13; ++k) g->grad_intrinsics[13 * (size_t)i + k] /= c;
            }
    }

    // NormalizeGradient<float,3>, rendering/PointRenderer.cu:1072-1090,1273-1280
    if (g->grad_points && pr.point_gradient_normalization == 1)
    {
        for (int i = 0; i < N; ++i)
        {
            const float c = g->grad_point_count[i];
            if (c > 0)
                for (int k = 0; k < 3; ++k) g->grad_points[4 * (size_t)i + k] /= c;
        }
    }
    else if (g->grad_points && pr.point_gradient_normalization == 2)
    {
        // literal: the [N,4] buffer is addressed as N vec3, so flat elements 3i..3i+2 are divided by count[i]
        for (int i = 0; i < N; ++i)
        {
            const float c = g->grad_point_count[i];
            if (c > 0)
                for (int k = 0; k < 3; ++k) g->grad_points[3 * (size_t)i + k] /= c;
        }
    }
    return VETRAST_OK;
}

// torch::sigmoid(scale * x) in the canonical arithmetic (exposed so that tests can pin it against a float64 logistic).
extern "C" int vetref_struct_sizes(uint64_t sizes[4])
{
    sizes[0] = sizeof(vetrast_forward_args);
    sizes[1] = sizeof(vetrast_backward_args);
    sizes[2] = sizeof(vetrast_adam_args);
    sizes[3] = sizeof(vetrast_lift_args);
    return 0;
}

extern "C" int vetref_sigmoid(const float* x, float* y, int64_t n, float scale)
{
    for (int64_t i = 0; i < n; ++i) y[i] = sigmoid_canon(scale * x[i]);
    return VETRAST_OK;
}

// One Adam step: MyAdam::step, models/my_adam.cpp:66-101 (torch's Adam without amsgrad), every operation rounded on its
// own in the order of the tensor ops there; bias corrections in double as at :72-73.
extern "C" int vetref_adam_step(const vetrast_adam_args* a)
{
    if (!a || a->n < 0 || a->step < 1) return VETRAST_ERR_INVALID_ARG;
    const double bc1 = 1.0 - std::pow(a->beta1, (double)a->step);
    const double bc2 = 1.0 - std::pow(a->beta2, (double)a->step);
    const float sqrt_bc2 = (float)std::sqrt(bc2), step_size = (float)(a->lr / bc1);
    const float omb1 = (float)(1.0 - a->beta1), omb2 = (float)(1.0 - a->beta2);
    const float beta1 = (float)a->beta1, beta2 = (float)a->beta2, eps = (float)a->eps, wd = (float)a->weight_decay;
    for (int64_t i = 0; i < a->n; ++i)
    {
        const float p = a->param[i];
        float gr      = a->grad[i];
        if (wd != 0.f) gr = gr + wd * p;
        const float m     = a->exp_avg[i] * beta1 + omb1 * gr;
        const float v     = a->exp_avg_sq[i] * beta2 + (omb2 * gr) * gr;
        const float denom = std::sqrt(v) / sqrt_bc2 + eps;
        a->exp_avg[i]     = m;
        a->exp_avg_sq[i]  = v;
        a->param[i]       = p + (-step_size) * (m / denom);
        if (a->zero_grad) a->grad[i] = 0.f;
    }
    return VETRAST_OK;
}

// sign() and PointInTriangle(), rendering/RenderForward.cu:605-625.
static inline float lift_sign(const float* p1, const float* p2, const float* p3)
{
    return (p1[0] - p3[0]) * (p2[1] - p3[1]) - (p2[0] - p3[0]) * (p1[1] - p3[1]);
}

static inline bool lift_point_in_triangle(const float* pt, const float* v1, const float* v2, const float* v3)
{
    const float d1 = lift_sign(pt, v1, v2), d2 = lift_sign(pt, v2, v3), d3 = lift_sign(pt, v3, v1);
    const bool has_neg = (d1 < 0) || (d2 < 0) || (d3 < 0);
    const bool has_pos = (d1 > 0) || (d2 > 0) || (d3 > 0);
    return !(has_neg && has_pos);
}

// Error lifting: FillSceneGridWithLossRasterize, rendering/RenderForward.cu:639-761, one cell after the other and the
// pixels of a cell in the order of the reference's xy_c counter. The reference leaves a cell when min_depths is set,
// which a lane may read before the lanes that project have written it (no __syncwarp, :704-705); the oracle takes the
// evident intent: a cell with any corner at z <= 0 is skipped. The float terms of a cell are summed in double and added
// to cell_value with one rounding (the reference's atomicAdd order is unspecified).
extern "C" int vetref_lift_error(const vetrast_lift_args* a, int num_threads)
{
    if (!a || a->num_cells < 0 || a->channels < 1 || a->height < 1 || a->width < 1) return VETRAST_ERR_INVALID_ARG;
    const vetrast_view& v = a->view;
    if (v.image_index < 0 || v.image_index >= a->num_poses || v.camera_index < 0 || v.camera_index >= a->num_cameras)
        return VETRAST_ERR_INVALID_ARG;
    const Prepared cam = prepare(a->poses_se3 + 8 * (size_t)v.image_index, a->intrinsics + 13 * (size_t)v.camera_index);
    const int border   = a->border_pixels;
    const int W = a->width, H = a->height;
    static const int tris[12][3]    = {{0, 1, 4}, {0, 4, 2}, {1, 5, 7}, {1, 7, 4}, {5, 3, 6}, {5, 6, 7},
                                       {3, 0, 6}, {0, 6, 2}, {3, 0, 5}, {0, 5, 1}, {2, 4, 6}, {4, 6, 7}};
    static const float bb_facs[8][3] = {{0, 0, 0}, {1, 0, 0}, {0, 1, 0}, {0, 0, 1}, {1, 1, 0}, {1, 0, 1}, {0, 1, 1}, {1, 1, 1}};
    omp_set_num_threads(num_threads > 0 ? num_threads : 1);
#pragma omp parallel for schedule(dynamic, 16) if (num_threads > 1)
    for (int64_t cell = 0; cell < a->num_cells; ++cell)
    {
        float proj[8][2];
        bool behind = false;
        for (int i = 0; i < 8; ++i)
        {
            float p4[4];
            for (int k = 0; k < 3; ++k) p4[k] = a->cell_bb_min[3 * cell + k] + a->cell_bb_length[3 * cell + k] * bb_facs[i][k];
            p4[3] = 0.f;
            Projected o;
            if (!project(cam, v, p4, o))  // z <= 0 (:694)
            {
                behind = true;
                break;
            }
            proj[i][0] = o.ipx;
            proj[i][1] = o.ipy;
        }
        if (behind) continue;
        float max_x = -10000000.f, max_y = -10000000.f, min_x = 10000000.f, min_y = 10000000.f;
        for (int i = 0; i < 8; ++i)
        {
            max_x = std::fmax(proj[i][0], max_x);
            max_y = std::fmax(proj[i][1], max_y);
            min_x = std::fmin(proj[i][0], min_x);
            min_y = std::fmin(proj[i][1], min_y);
        }
        if (max_x < border || min_x >= W - border || max_y < border || min_y >= H - border) continue;
        min_x = std::fmax(min_x, (float)border);
        min_y = std::fmax(min_y, (float)border);
        max_x = std::fmin(max_x, (float)(W - border));
        max_y = std::fmin(max_y, (float)(H - border));
        const int y_size = int(max_y - min_y);
        const int x_size = int(max_x - min_x);
        double sum = 0.0;
        int count  = 0;
        for (int xy_c = 0; xy_c < y_size * x_size; ++xy_c)
        {
            const int x_c     = (int)((float)(xy_c % x_size) + min_x);
            const int y_c     = (int)((float)(xy_c / x_size) + min_y);
            const float pt[2] = {(float)x_c, (float)y_c};
            bool is_in        = false;
            for (int t = 0; t < 12; ++t)
                if (lift_point_in_triangle(pt, proj[tris[t][0]], proj[tris[t][1]], proj[tris[t][2]])) is_in = true;
            if (!is_in) continue;
            if (x_c < 0 || x_c >= W || y_c < 0 || y_c >= H) continue;  // cannot happen with border >= 0
            float grad = 0.f;
            for (int i = 0; i < a->channels; ++i) grad += std::fabs(a->loss_image[((size_t)i * H + y_c) * W + x_c]);
            sum += (double)grad;
            count += 1;
        }
        if (count > 0)
        {
            a->cell_value[cell]        = (float)((double)a->cell_value[cell] + sum);
            a->cell_access_count[cell] = a->cell_access_count[cell] + count;
        }
    }
    return VETRAST_OK;
}
