/*
 * CPU oracle of the blending point rasterizer — TEST INFRASTRUCTURE ONLY.
 *
 * A plain scalar restatement of the reference's FULL_BLEND path, of its BILINEAR_BLEND path (params.render_mode = 3)
 * and of its FUZZY_BLEND path (params.render_mode = 2) (lfranke/VET, src/lib/rendering). It exists to
 * check the GPU library and to be timed as the CPU baseline; nothing that ships may call it. Only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg load this library.
 *
 * Argument structs are the PODs of include/vetrast.h, with every `device` pointer replaced by a host pointer and
 * the workspace ignored; saved state goes to explicit caller-allocated arrays instead:
 *   offsets       uint32 [B][P+1]   exclusive scan of per-pixel counts, pixels of all layers concatenated
 *   fragments     uint64 [B][N*L]   (depth_bits << 32) | point_id; every pixel list fully sorted ascending
 *                                   (BILINEAR_BLEND: [B][4*N*L], low word = point_id << 2 | corner, corner = 2*dy + dx)
 *   transmittance float  [B][N*L]   transmittance in front of fragment i for every fragment that took part in the blend
 *   weight        float  [B][P]     final transmittance per pixel
 *
 * Parity status of the pieces (what pins each is in tests/test_oracle_*.py):
 *   projection        pinned by the reference's own host restatements of the pinhole model
 *                     (src/lib/data/SceneData.cpp:28-36,1020-1049) for zero distortion and by brute-force checks;
 *                     the bit pattern of saiga's TransformPoint / DivideByZ is PARITY UNPINNED (saiga is not vendored)
 *   lens distortion   (params.allow_distortion) PARITY UNPINNED: the reference calls saiga's distortNormalizedPoint
 *                     (rendering/PointRendererHelper.h:207,348), whose source is not in its tree, and holds no vector
 *                     for it. The oracle states the published 8-coefficient rational model the coefficient layout
 *                     implies; what pins THAT (a float64 statement, closed forms, central differences of every
 *                     gradient) is in tests/test_oracle_distortion.py. dist_cutoff is not applied.
 *   count/scan/fill   pinned by brute force and by the reference's own invariant counters == counts
 *   sort              pinned against a generic sort of (depth, id) pairs; the id tie-break refines the reference's
 *                     depth-only order
 *   blend             pinned by closed forms (empty pixel, one fragment, n equal fragments, partition of unity)
 *   value gradients   pinned by double-precision central differences of an independent numpy blend
 *   position gradient literal restatement; the heuristic is checked on hand-computed cases, the projection Jacobian
 *                     by finite differences; saiga's operator order inside the Jacobians is PARITY UNPINNED
 *   bilinear mode     splat weights pinned by closed forms (weights of a point sum to 1 over its 2x2 pixels, a point on
 *                     a pixel centre lands in one pixel), the blend and its early exit by an independent numpy blend,
 *                     value and position gradients by double-precision central differences of that blend (the
 *                     position gradient is analytic in this mode, so finite differences do pin it)
 *   fuzzy mode        (render_mode 2) pinned by: a vanishing depth range is FULL_BLEND; on scenes whose buckets are fixed
 *                     by construction (points on depth levels) an independent float64 model gives the forward image
 *                     (nearest level averaged only), the descriptor/background gradients (central differences) and the
 *                     confidence gradient (own bucket's term + bucket size x later buckets' terms)
 *   fused preparation confidence = sigmoid(scale * raw) pinned against a float64 logistic (<= 4e-7 relative: the exact bits of
 *                     torch::sigmoid are PARITY UNPINNED), |texture| / |background| and the chain rule of both by
 *                     comparing with the unfused path fed the prepared tensors and torch autograd
 *   Adam step         pinned against torch.optim.Adam on the CPU over several steps with and without weight decay
 *   error lifting     literal restatement; pinned by an independent numpy rasterization (the union of the 12 projected
 *                     face triangles is the convex hull of the 8 projected corners, tested with half-plane checks of a
 *                     hull built by scipy, away from the hull's boundary), by closed forms (an axis-aligned cell seen
 *                     head-on covers a known pixel rectangle, a constant error image gives value = channels * count)
 *                     and by the skip rules (corner behind the camera, box outside the border). The reference kernel
 *                     is compiled with nvcc's default fused multiply-add; which side of a triangle edge a pixel
 *                     exactly on it falls under that contraction is PARITY UNPINNED
 *   distortion != 0, check_normal, OCam, spherical: not implemented (rejected), PARITY UNPINNED
 */
#ifndef VETRAST_ORACLE_H
#define VETRAST_ORACLE_H

#include "../include/vetrast.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Prepared per-view camera constants: 12 floats world->camera (R row-major | t as 4th column per row),
 * then fx,fy,cx,cy,s. Exposed so that tests can pin the quaternion conversion. */
int vetref_prepare_view(const double* pose8, const float* intrinsics13, float* out17);

/* Project one point for one prepared view; returns 0 if rejected (z == 0). ip_z_r = {ip.x, ip.y, z, radius_px}. */
int vetref_project_point(const float* prepared17, const vetrast_view* view, const float* position4, float* ip_z_r);

/* kept (optional): uint32 [B][P], the number of fragments of every pixel that took part in the blend: min(count, K), and
 * in BILINEAR_BLEND also cut where the transmittance fell below 0.001. */
int vetref_forward(const vetrast_forward_args* args, uint32_t* offsets, uint64_t* fragments, float* transmittance,
                   float* weight, uint32_t* kept, int num_threads);

int vetref_backward(const vetrast_backward_args* args, const uint32_t* offsets, const uint64_t* fragments,
                    int num_threads);

/* sigmoid(scale * x) in the canonical arithmetic of the fused confidence activation (params.confidence_activation). */
int vetref_sigmoid(const float* x, float* y, int64_t n, float scale);

/* One Adam step on host arrays (MyAdam::step). */
int vetref_adam_step(const vetrast_adam_args* args);

/* Error lifting on host arrays (FillSceneGridWithLossRasterize); the workspace is ignored. */
int vetref_lift_error(const vetrast_lift_args* args, int num_threads);

/* Sizes of the argument structs this library was compiled with (forward, backward, adam, lift arguments): lets a
 * caller that mirrors them notice a library built from an older header instead of reading past a struct. */
int vetref_struct_sizes(uint64_t sizes[4]);

#ifdef __cplusplus
}
#endif
#endif
