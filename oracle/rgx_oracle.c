/*
 * rgx_oracle.c -- CPU restatement of the RayGaussX differentiable Gaussian
 * ray-marching path.  TEST INFRASTRUCTURE ONLY: this file is the checker the
 * HIP kernels are compared against.  Only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load it; the product never routes through it.
 *
 * Every function cites the reference file:line it restates (paths relative to
 * the reference tree).  The reference's arithmetic lives in OptiX device
 * programs; OptiX itself (closed source, v7.6) only supplies BVH culling, whose
 * functional result for custom primitives is "the set of primitives whose
 * intersection program reports a hit in [tmin,tmax]".  That set is computed
 * here by brute force over all primitives.
 *
 * Canonical arithmetic (shared contract with the HIP kernels so that hit sets
 * are bit-identical): IEEE binary32 throughout, no contraction (build with
 * -ffp-contract=off), fmaf exactly where the reference writes fmaf, dot(a,b)
 * = (a.x*b.x + a.y*b.y) + a.z*b.z, normalize(v) = v * (1/sqrt(dot(v,v))),
 * __frcp_rn(x) = 1.0f/x, __fdividef(a,b) = a/b, logf(x) = (float)log((double)x)
 * (so both sides round the same way), rsqrtf(x) = 1.0f/sqrtf(x).  expf/cbrtf
 * are the C library's; they only reach colours and gradients, which are gated
 * by tolerance, not bit-exactness.
 *
 * Pinning status (what independent check holds each function; see tests/):
 *   orc_aabb            closed form k*sqrt(diag(R S^2 R^T)) + surface sampling
 *   orc_pack_prims      closed form rho*exp(-k^2/2) = sigma_threshold
 *   orc_sh_forward      textbook real SH (scipy) + degree-0 special case
 *   orc_sh_backward     torch.autograd of the forward + the one documented
 *                       deviation of the reference (sh_utils.cu:367, see below)
 *   orc_ray_dirs        pinhole model K^-1 [u,v,1] rotated by c2w
 *   line/segment hit    float64 closed-form ray/ellipsoid roots, equivariance
 *   orc_first_hit / orc_trace_segments   numpy brute force in float64
 *   orc_march_forward   analytic optical depth (erf) of one isotropic Gaussian,
 *                       empty scene, compositing identity, float64 numpy march;
 *                       its dynamic_sampling branch: a float64 march that recomputes
 *                       every step from its own transmittance (same slab sequence,
 *                       steps and hit sets on every ray away from a decision edge),
 *                       and closed forms on one Gaussian (T = 1: the distance term
 *                       exactly; T(t) through erf; the 4 dt0 cap exactly)
 *   orc_march_backward  torch.autograd through a float64 torch forward with
 *                       frozen hit sets and cut-off masks + central differences;
 *                       its dynamic_sampling branch: autograd is fed the forward's
 *                       (pinned) slab sequence, so a backward that stepped
 *                       differently would miss its gradients
 *   orc_march_backward_in_cut / orc_set_backward_mask_form (probes of the backward's
 *                       cut-off decisions): the count against a float64 count over the same
 *                       slabs on every ray with no sample within rounding of a cut-off; the
 *                       forward's form of the decision leaves every Gaussian alone that no
 *                       disagreeing ray touches
 *   orc_cull_build      brute force (same candidates, bit for bit)
 *   orc_march_gui       float64 quadrature of int t sigma exp(-tau) dt for one Gaussian,
 *                       depth / (1 - T) inside the scene box, known quantisation values
 *   orc_morton_codes    naive per-bit loop
 *   orc_dist2_knn3      scipy.spatial.cKDTree (k = 4 with the point itself) in float64
 * The reference ships no tests, golden vectors or fixtures for this path, and
 * cannot be built or imported without OptiX/CuPy/an NVIDIA GPU, so there is no
 * oracle/_ref build.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define BUFFER_SIZE 32 /* cuda_train/forward/gaussians_aabb.h:2 */
#define CHUNK_SIZE 16  /* cuda_train/forward/gaussians_aabb.h:3 */

typedef struct { float x, y, z; } f3;

typedef struct {
    float eye[3];
    float u[3], v[3], w[3]; /* world_view_transform[:3,0..2], optix_utils.py:261-263 */
    float tan_x, tan_y, px, py; /* cam_intr, optix_utils.py:266 */
    int width, height;          /* already multiplied by supersampling */
} OrcCamera;

typedef struct {
    float dt_step;
    int dynamic_sampling;
    int max_prim_slice;
    int white_background;
    float t_eps; /* TRANSMITTANCE_EPSILON, gaussians_aabb.h:4 (0.001f) */
} OrcMarch;

typedef struct {
    int64_t hit_pairs;     /* sum over marched slabs of hit-list length */
    int64_t slabs;         /* slabs that were blended */
    int64_t empty_slabs;   /* collect queries that returned nothing */
    int64_t overflow_rays; /* collect queries truncated at max_prim_slice */
    int64_t rays_hit;      /* rays whose first-hit query found something */
} OrcStats;

static inline f3 mk3(float x, float y, float z) { f3 r = {x, y, z}; return r; }
static inline f3 add3(f3 a, f3 b) { return mk3(a.x + b.x, a.y + b.y, a.z + b.z); }
static inline f3 sub3(f3 a, f3 b) { return mk3(a.x - b.x, a.y - b.y, a.z - b.z); }
static inline f3 mul3(f3 a, f3 b) { return mk3(a.x * b.x, a.y * b.y, a.z * b.z); }
static inline f3 scl3(f3 a, float s) { return mk3(a.x * s, a.y * s, a.z * s); }
/* vec_math.h dot(float3,float3): a.x*b.x + a.y*b.y + a.z*b.z, left to right */
static inline float dot3(f3 a, f3 b) { return (a.x * b.x + a.y * b.y) + a.z * b.z; }
/* vec_math.h:554-558 normalize: v * (1/sqrtf(dot(v,v))) */
static inline f3 normalize3(f3 v) { float inv = 1.0f / sqrtf(dot3(v, v)); return scl3(v, inv); }
static inline float canon_logf(float x) { return (float)log((double)x); }
static float g_step_scale = 1.0f; /* see orc_set_step_scale() */
static int g_mask_form = 0;       /* see orc_set_backward_mask_form() */

/* cuda_train/forward/gaussians_aabb.cu:7-17 quaternion_to_matrix (columns of R) */
static inline void quat_to_cols(const float *q, f3 *c0, f3 *c1, f3 *c2)
{
    const float r = q[0], i = q[1], j = q[2], k = q[3];
    const float ii = i + i, jj = j + j, kk = k + k;
    const float ri = r * ii, rj = r * jj, rk = r * kk;
    const float ii2 = i * ii, jj2 = j * jj, kk2 = k * kk;
    const float ij = i * jj, ik = i * kk, jk = j * kk;
    *c0 = mk3(1.f - (jj2 + kk2), ij + rk, ik - rj);
    *c1 = mk3(ij - rk, 1.f - (ii2 + kk2), jk + ri);
    *c2 = mk3(ik + rj, jk - ri, 1.f - (ii2 + jj2));
}

/* gaussians_aabb.cu:19-30 apply_Sinv_Rt */
static inline f3 apply_sinv_rt(f3 x, f3 U, f3 V, f3 W, f3 inv_s)
{
    const float rx = fmaf(U.x, x.x, fmaf(U.y, x.y, U.z * x.z));
    const float ry = fmaf(V.x, x.x, fmaf(V.y, x.y, V.z * x.z));
    const float rz = fmaf(W.x, x.x, fmaf(W.y, x.y, W.z * x.z));
    return mk3(rx * inv_s.x, ry * inv_s.y, rz * inv_s.z);
}

/* ------------------------------------------------------------------------- */
/* a2: optix_utils.py:36-109 (_ELLIPSOID_BBOX + scene bbox reductions)        */
void orc_aabb(int64_t N, const float *pos, const float *scale, const float *quat,
              const float *dens, float sigma_thr, float *bboxes, float *bb_min, float *bb_max)
{
    float mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
    for (int64_t n = 0; n < N; ++n) {
        float t = dens[n] / sigma_thr;
        float d = canon_logf(t * t);
        if (!(d > 0.0f)) d = 0.0f;
        d = sqrtf(d);
        float W = quat[4 * n], X = quat[4 * n + 1], Y = quat[4 * n + 2], Z = quat[4 * n + 3];
        float nn = ((W * W + X * X) + Y * Y) + Z * Z;
        float invn = 1.0f / sqrtf(nn + 1e-20f);
        W *= invn; X *= invn; Y *= invn; Z *= invn;
        float L1x = 1.f - 2.f * (Y * Y + Z * Z), L1y = 2.f * (X * Y - W * Z), L1z = 2.f * (X * Z + W * Y);
        float L2x = 2.f * (X * Y + W * Z), L2y = 1.f - 2.f * (X * X + Z * Z), L2z = 2.f * (Y * Z - W * X);
        float L3x = 2.f * (X * Z - W * Y), L3y = 2.f * (Y * Z + W * X), L3z = 1.f - 2.f * (X * X + Y * Y);
        float s0 = scale[3 * n], s1 = scale[3 * n + 1], s2 = scale[3 * n + 2];
        float hx = d * sqrtf(((s0 * L1x) * (s0 * L1x) + (s1 * L1y) * (s1 * L1y)) + (s2 * L1z) * (s2 * L1z));
        float hy = d * sqrtf(((s0 * L2x) * (s0 * L2x) + (s1 * L2y) * (s1 * L2y)) + (s2 * L2z) * (s2 * L2z));
        float hz = d * sqrtf(((s0 * L3x) * (s0 * L3x) + (s1 * L3y) * (s1 * L3y)) + (s2 * L3z) * (s2 * L3z));
        float c0 = pos[3 * n], c1 = pos[3 * n + 1], c2 = pos[3 * n + 2];
        float b[6] = {c0 - hx, c1 - hy, c2 - hz, c0 + hx, c1 + hy, c2 + hz};
        for (int a = 0; a < 6; ++a) bboxes[6 * n + a] = b[a];
        for (int a = 0; a < 3; ++a) {
            if (b[a] < mn[a]) mn[a] = b[a];
            if (b[a + 3] > mx[a]) mx[a] = b[a + 3];
        }
    }
    for (int a = 0; a < 3; ++a) { bb_min[a] = mn[a]; bb_max[a] = mx[a]; }
}

/* a4: optix_utils.py:268-304 prim packing into the 64-byte PrimData record   */
/* (gaussians_aabb.h:7-12): pos4, inv_inter4, quat4, rgba4                    */
void orc_pack_prims(int64_t N, const float *eye, const float *pos, const float *scale,
                    const float *quat, const float *dens, const float *rgb, float sigma_thr,
                    float *prims)
{
    for (int64_t n = 0; n < N; ++n) {
        float *p = prims + 16 * n;
        const float rho = dens[n];
        for (int a = 0; a < 3; ++a) p[a] = eye[a] - pos[3 * n + a];
        p[3] = 0.0f;
        const float k = sqrtf(2.0f * canon_logf(rho / sigma_thr)); /* optix_utils.py:288 */
        for (int a = 0; a < 3; ++a) p[4 + a] = (1.0f / scale[3 * n + a]) / k;
        p[7] = k;
        for (int a = 0; a < 4; ++a) p[8 + a] = quat[4 * n + a];
        for (int a = 0; a < 3; ++a) p[12 + a] = rgb[3 * n + a] * rho;
        p[15] = rho;
    }
}

/* ------------------------------------------------------------------------- */
/* a6: utils/sh_utils.cu:6-23 constants, 122-216 forward_sh                   */
static const float SH_C0 = 0.28209479177387814f;
static const float SH_C1 = 0.4886025119029199f;
static const float SH_C2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                               -1.0925484305920792f, 0.5462742152960396f};
static const float SH_C3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                               0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                               -0.5900435899266435f};

/* basis_j(dir) for j < (degree+1)^2, in the order forward_sh multiplies sh[j] */
static void sh_basis(int degree, float x, float y, float z, float *b)
{
    b[0] = SH_C0;
    if (degree > 0) {
        b[1] = -SH_C1 * y; b[2] = SH_C1 * z; b[3] = -SH_C1 * x;
        if (degree > 1) {
            float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
            b[4] = SH_C2[0] * xy; b[5] = SH_C2[1] * yz; b[6] = SH_C2[2] * (2.0f * zz - xx - yy);
            b[7] = SH_C2[3] * xz; b[8] = SH_C2[4] * (xx - yy);
            if (degree > 2) {
                b[9] = SH_C3[0] * y * (3.0f * xx - yy);
                b[10] = SH_C3[1] * xy * z;
                b[11] = SH_C3[2] * y * (4.0f * zz - xx - yy);
                b[12] = SH_C3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy);
                b[13] = SH_C3[4] * x * (4.0f * zz - xx - yy);
                b[14] = SH_C3[5] * z * (xx - yy);
                b[15] = SH_C3[6] * x * (xx - 3.0f * yy);
            }
        }
    }
}

void orc_sh_forward(int64_t N, const float *eye, const float *pos, const float *sh,
                    const float *sg, const float *sharp, const float *axis, int G, int degree,
                    float *rgb)
{
    const int K = (degree + 1) * (degree + 1);
    for (int64_t n = 0; n < N; ++n) {
        f3 d0 = mk3(pos[3 * n] - eye[0], pos[3 * n + 1] - eye[1], pos[3 * n + 2] - eye[2]);
        float len = sqrtf(dot3(d0, d0)); /* sh_utils.cu:130 dir_orig / length(dir_orig) */
        f3 d = mk3(d0.x / len, d0.y / len, d0.z / len);
        float res[3] = {0.f, 0.f, 0.f};
        for (int l = 0; l < G; ++l) { /* sh_utils.cu:140-151 spherical Gaussians */
            f3 ax = mk3(axis[(n * G + l) * 3], axis[(n * G + l) * 3 + 1], axis[(n * G + l) * 3 + 2]);
            float g = expf(sharp[n * G + l] * (dot3(d, ax) - 1.0f));
            for (int c = 0; c < 3; ++c) res[c] += sg[n * G * 3 + c * G + l] * g;
        }
        float b[16];
        sh_basis(degree, d.x, d.y, d.z, b);
        for (int c = 0; c < 3; ++c) {
            const float *s = sh + (n * 3 + c) * K; /* channel-major (N,3,K), sh_utils.cu:154-156 */
            float r = res[c];
            for (int j = 0; j < K; ++j) r += b[j] * s[j];
            rgb[3 * n + c] = r + 0.5f; /* sh_utils.cu:213-215, no clamp */
        }
    }
}

/* a17: utils/sh_utils.cu:218-412 backward_sh.  NOTE sh_utils.cu:367: the      */
/* reference's d/dy of basis 9 is written (3xx - yy) where calculus gives      */
/* 3(xx - yy) (its own comment, line 360, has the latter).  A drop-in returns  */
/* the reference's gradients, so the restatement keeps the reference's term;   */
/* `exact_dy9` != 0 switches to the calculus value (used by the autograd test  */
/* to show this is the ONLY deviation).                                        */
void orc_sh_backward(int64_t N, const float *eye, const float *pos, const float *sh,
                     const float *sg, const float *sharp, const float *axis, int G, int degree,
                     const float *drgb, int exact_dy9, float *dsh, float *dpos, float *dsg,
                     float *dsharp, float *daxis)
{
    const int K = (degree + 1) * (degree + 1);
    for (int64_t n = 0; n < N; ++n) {
        const float gr[3] = {drgb[3 * n], drgb[3 * n + 1], drgb[3 * n + 2]};
        float *o_sh = dsh + n * 3 * K;
        float *o_pos = dpos + 3 * n;
        for (int j = 0; j < 3 * K; ++j) o_sh[j] = 0.f;
        o_pos[0] = o_pos[1] = o_pos[2] = 0.f;
        for (int l = 0; l < G; ++l) {
            for (int c = 0; c < 3; ++c) { dsg[n * G * 3 + c * G + l] = 0.f; daxis[(n * G + l) * 3 + c] = 0.f; }
            dsharp[n * G + l] = 0.f;
        }
        if (gr[0] == 0.f && gr[1] == 0.f && gr[2] == 0.f) continue; /* sh_utils.cu:226 */
        f3 v = mk3(pos[3 * n] - eye[0], pos[3 * n + 1] - eye[1], pos[3 * n + 2] - eye[2]);
        float len = sqrtf(dot3(v, v));
        const float x = v.x / len, y = v.y / len, z = v.z / len;
        float b[16];
        sh_basis(degree, x, y, z, b);
        for (int c = 0; c < 3; ++c)
            for (int j = 0; j < K; ++j) o_sh[c * K + j] = b[j] * gr[c]; /* sh_utils.cu:250-347 */
        /* dRGB/d(dir) per channel, sh_utils.cu:271-376 */
        float dx[3] = {0, 0, 0}, dy[3] = {0, 0, 0}, dz[3] = {0, 0, 0};
        if (degree > 0) {
            float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
            for (int c = 0; c < 3; ++c) {
                const float *s = sh + (n * 3 + c) * K;
                dx[c] = -SH_C1 * s[3]; dy[c] = -SH_C1 * s[1]; dz[c] = SH_C1 * s[2];
                if (degree > 1) {
                    dx[c] += SH_C2[0] * y * s[4] + SH_C2[2] * 2.0f * -x * s[6] + SH_C2[3] * z * s[7] + SH_C2[4] * 2.0f * x * s[8];
                    dy[c] += SH_C2[0] * x * s[4] + SH_C2[1] * z * s[5] + SH_C2[2] * 2.0f * -y * s[6] + SH_C2[4] * 2.0f * -y * s[8];
                    dz[c] += SH_C2[1] * y * s[5] + SH_C2[2] * 2.0f * 2.0f * z * s[6] + SH_C2[3] * x * s[7];
                    if (degree > 2) {
                        float dy9 = exact_dy9 ? 3.0f * (xx - yy) : (3.0f * xx - yy);
                        dx[c] += SH_C3[0] * s[9] * 3.0f * 2.0f * xy + SH_C3[1] * s[10] * yz + SH_C3[2] * s[11] * -2.0f * xy +
                                 SH_C3[3] * s[12] * -3.0f * 2.0f * xz + SH_C3[4] * s[13] * (-3.0f * xx + 4.0f * zz - yy) +
                                 SH_C3[5] * s[14] * 2.0f * xz + SH_C3[6] * s[15] * 3.0f * (xx - yy);
                        dy[c] += SH_C3[0] * s[9] * dy9 + SH_C3[1] * s[10] * xz + SH_C3[2] * s[11] * (-3.0f * yy + 4.0f * zz - xx) +
                                 SH_C3[3] * s[12] * -3.0f * 2.0f * yz + SH_C3[4] * s[13] * -2.0f * xy + SH_C3[5] * s[14] * -2.0f * yz +
                                 SH_C3[6] * s[15] * -3.0f * 2.0f * xy;
                        dz[c] += SH_C3[1] * s[10] * xy + SH_C3[2] * s[11] * 4.0f * 2.0f * yz + SH_C3[3] * s[12] * 3.0f * (2.0f * zz - xx - yy) +
                                 SH_C3[4] * s[13] * 4.0f * 2.0f * xz + SH_C3[5] * s[14] * (xx - yy);
                    }
                }
            }
        }
        f3 ddir = mk3((gr[0] * dx[0] + gr[1] * dx[1]) + gr[2] * dx[2],
                      (gr[0] * dy[0] + gr[1] * dy[1]) + gr[2] * dy[2],
                      (gr[0] * dz[0] + gr[1] * dz[1]) + gr[2] * dz[2]); /* sh_utils.cu:382 */
        for (int l = 0; l < G; ++l) { /* sh_utils.cu:385-405 */
            f3 feat = mk3(sg[n * G * 3 + l], sg[n * G * 3 + G + l], sg[n * G * 3 + 2 * G + l]);
            f3 ax = mk3(axis[(n * G + l) * 3], axis[(n * G + l) * 3 + 1], axis[(n * G + l) * 3 + 2]);
            float sp = sharp[n * G + l];
            float dm1 = dot3(mk3(x, y, z), ax) - 1.0f;
            float wgt = expf(dm1 * sp);
            for (int c = 0; c < 3; ++c) dsg[n * G * 3 + c * G + l] = gr[c] * wgt;
            float dwgt = dot3(mk3(gr[0], gr[1], gr[2]), feat);
            daxis[(n * G + l) * 3 + 0] = dwgt * sp * x * wgt;
            daxis[(n * G + l) * 3 + 1] = dwgt * sp * y * wgt;
            daxis[(n * G + l) * 3 + 2] = dwgt * sp * z * wgt;
            dsharp[n * G + l] = dwgt * dm1 * wgt;
            ddir = add3(ddir, scl3(ax, dwgt * sp * wgt));
        }
        float sum2 = dot3(v, v);                          /* sh_utils.cu:406-410 */
        float inv32 = 1.0f / sqrtf(sum2 * sum2 * sum2);
        o_pos[0] = ((sum2 - v.x * v.x) * ddir.x - v.y * v.x * ddir.y - v.z * v.x * ddir.z) * inv32;
        o_pos[1] = (-v.x * v.y * ddir.x + (sum2 - v.y * v.y) * ddir.y - v.z * v.y * ddir.z) * inv32;
        o_pos[2] = (-v.x * v.z * ddir.x - v.y * v.z * ddir.y + (sum2 - v.z * v.z) * ddir.z) * inv32;
    }
}

/* ------------------------------------------------------------------------- */
/* a7: gaussians_aabb.cu:95-110 computeRay                                    */
static inline f3 compute_ray(const OrcCamera *c, unsigned ix, unsigned iy)
{
    const float idx_x = ((float)ix + 0.5f) / (float)(unsigned)c->width;
    const float idx_y = ((float)iy + 0.5f) / (float)(unsigned)c->height;
    const float px = 2.0f * (idx_x - c->px), py = 2.0f * (idx_y - c->py);
    const float dx = px * c->tan_x, dy = py * c->tan_y;
    f3 d = mk3((dx * c->u[0] + dy * c->v[0]) + c->w[0],
               (dx * c->u[1] + dy * c->v[1]) + c->w[1],
               (dx * c->u[2] + dy * c->v[2]) + c->w[2]);
    return normalize3(d);
}

void orc_ray_dirs(const OrcCamera *cam, int64_t n, const int64_t *ray_ids, float *dirs)
{
    for (int64_t r = 0; r < n; ++r) {
        int64_t id = ray_ids ? ray_ids[r] : r;
        f3 d = compute_ray(cam, (unsigned)(id % cam->width), (unsigned)(id / cam->width));
        dirs[3 * r] = d.x; dirs[3 * r + 1] = d.y; dirs[3 * r + 2] = d.z;
    }
}

/* a9: gaussians_aabb.cu:36-92 __intersection__gaussian.  The part that does   */
/* not depend on [ray_tmin, ray_tmax] (lines 43-82: disc test and the two      */
/* roots) is evaluated once per (ray, prim) here; the interval part (84-89)    */
/* is segment_hit() below.  Splitting changes no operation or rounding.        */
typedef struct { int32_t id; float r1, r2; } Cand;

static inline int line_roots(const float *p, f3 dir, float *r1, float *r2)
{
    const f3 inv_scales = mk3(p[4], p[5], p[6]);
    const f3 O = mk3(p[0], p[1], p[2]);
    f3 U, V, W;
    quat_to_cols(p + 8, &U, &V, &W);
    const f3 Oe = apply_sinv_rt(O, U, V, W, inv_scales);
    const f3 De = apply_sinv_rt(dir, U, V, W, inv_scales);
    const float a = fmaf(De.x, De.x, fmaf(De.y, De.y, De.z * De.z));
    const float b = -fmaf(Oe.x, De.x, fmaf(Oe.y, De.y, Oe.z * De.z));
    const float c = fmaf(Oe.x, Oe.x, fmaf(Oe.y, Oe.y, fmaf(Oe.z, Oe.z, -1.0f)));
    const float inv_a = 1.0f / a;
    const float b_inv_a = b * inv_a;
    const f3 P = mk3(fmaf(b_inv_a, De.x, Oe.x), fmaf(b_inv_a, De.y, Oe.y), fmaf(b_inv_a, De.z, Oe.z));
    const float d2 = fmaf(P.x, P.x, fmaf(P.y, P.y, P.z * P.z));
    const float disc = 1.0f - d2;
    if (disc > 1e-7f) {
        const float sdisc = sqrtf(disc * a);
        const float q = b + copysignf(sdisc, b);
        *r1 = c / q;
        *r2 = q * inv_a;
        return 1;
    }
    return 0;
}

/* gaussians_aabb.cu:84-89: hit iff max(tmin,root1) <= min(tmax,root2); t = the max */
static inline int segment_hit(float r1, float r2, float tmin, float tmax, float *t)
{
    const float min_t = fmaxf(tmin, r1);
    const float max_t = fminf(tmax, r2);
    if (min_t <= max_t) { *t = min_t; return 1; }
    return 0;
}

typedef struct { Cand *c; int64_t n, cap; } CandList;

static inline void cands_push(CandList *L, int32_t id, float r1, float r2)
{
    if (L->n == L->cap) {
        L->cap = L->cap ? 2 * L->cap : 1024;
        L->c = (Cand *)realloc(L->c, (size_t)L->cap * sizeof(Cand));
    }
    L->c[L->n].id = id; L->c[L->n].r1 = r1; L->c[L->n].r2 = r2;
    L->n++;
}

/* ------------------------------------------------------------------------- */
/* Optional culling for the timed CPU baseline.  The brute-force loop below    */
/* is the oracle proper: it evaluates the reference's predicate on every       */
/* primitive.  With orc_cull_build() a bounding-volume tree over the           */
/* primitives' k-sigma boxes (eye-relative, as the packed records are) feeds   */
/* the same predicate only the primitives whose padded box the ray's line      */
/* meets, and the survivors are put back into ascending index order, so the    */
/* candidate lists -- and with them every result -- are those of the brute     */
/* force (tests/test_oracle_geometry.py holds the two to each other).  The     */
/* boxes are padded by 1e-5 of their distance from the eye, a hundred times    */
/* what rounding lets the fp32 predicate accept outside the exact ellipsoid.   */
typedef struct { float lo[3], hi[3]; int32_t a, b; } CullNode; /* inner: children a, b; leaf: a = first, b = -count */
static struct { CullNode *nodes; int32_t *perm; int32_t n_nodes; const float *prims; int64_t N; } g_cull;

static int cull_cmp(const void *x, const void *y)
{
    const uint64_t a = *(const uint64_t *)x, b = *(const uint64_t *)y;
    return a < b ? -1 : a > b;
}

static int32_t cull_make(int32_t lo, int32_t hi, const float *boxes)
{
    const int32_t me = g_cull.n_nodes++;
    CullNode *nd = &g_cull.nodes[me];
    if (hi - lo <= 4) {
        nd->a = lo; nd->b = -(hi - lo);
        for (int c = 0; c < 3; ++c) { nd->lo[c] = INFINITY; nd->hi[c] = -INFINITY; }
        for (int32_t j = lo; j < hi; ++j) {
            const float *bx = boxes + 6 * (int64_t)g_cull.perm[j];
            for (int c = 0; c < 3; ++c) { nd->lo[c] = fminf(nd->lo[c], bx[c]); nd->hi[c] = fmaxf(nd->hi[c], bx[3 + c]); }
        }
        return me;
    }
    const int32_t mid = lo + (hi - lo) / 2;
    const int32_t a = cull_make(lo, mid, boxes), b = cull_make(mid, hi, boxes);
    nd = &g_cull.nodes[me];
    nd->a = a; nd->b = b;
    for (int c = 0; c < 3; ++c) {
        nd->lo[c] = fminf(g_cull.nodes[a].lo[c], g_cull.nodes[b].lo[c]);
        nd->hi[c] = fmaxf(g_cull.nodes[a].hi[c], g_cull.nodes[b].hi[c]);
    }
    return me;
}

void orc_cull_free(void)
{
    free(g_cull.nodes); free(g_cull.perm);
    memset(&g_cull, 0, sizeof g_cull);
}

/* Builds the tree for this primitive block; candidate searches on exactly this block (same   */
/* pointer, same N) use it until orc_cull_free().                                             */
void orc_cull_build(int64_t N, const float *prims)
{
    orc_cull_free();
    if (N <= 0) return;
    float *boxes = (float *)malloc(sizeof(float) * 6 * (size_t)N);
    uint64_t *keys = (uint64_t *)malloc(sizeof(uint64_t) * (size_t)N);
    float mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
    int64_t live = 0;
    for (int64_t i = 0; i < N; ++i) {
        const float *p = prims + 16 * i;
        if (!(p[7] == p[7])) continue; /* k is NaN below the density threshold: can never be hit */
        f3 U, V, W;
        quat_to_cols(p + 8, &U, &V, &W);
        const float ax = 1.0f / p[4], ay = 1.0f / p[5], az = 1.0f / p[6]; /* k * scale */
        const float h[3] = {sqrtf(U.x * U.x * ax * ax + V.x * V.x * ay * ay + W.x * W.x * az * az),
                            sqrtf(U.y * U.y * ax * ax + V.y * V.y * ay * ay + W.y * W.y * az * az),
                            sqrtf(U.z * U.z * ax * ax + V.z * V.z * ay * ay + W.z * W.z * az * az)};
        const float c[3] = {-p[0], -p[1], -p[2]}; /* centre - eye */
        const float pad = 1e-5f * (sqrtf(c[0] * c[0] + c[1] * c[1] + c[2] * c[2]) + fmaxf(h[0], fmaxf(h[1], h[2])) + 1.0f);
        float *bx = boxes + 6 * i;
        for (int a = 0; a < 3; ++a) {
            bx[a] = c[a] - h[a] * 1.001f - pad; bx[3 + a] = c[a] + h[a] * 1.001f + pad;
            mn[a] = fminf(mn[a], c[a]); mx[a] = fmaxf(mx[a], c[a]);
        }
        keys[live++] = (uint64_t)i; /* the code goes into the upper bits below */
    }
    for (int64_t j = 0; j < live; ++j) {
        const int64_t i = (int64_t)keys[j];
        const float *p = prims + 16 * i;
        uint64_t code = 0;
        const float c[3] = {-p[0], -p[1], -p[2]};
        uint32_t q[3];
        for (int a = 0; a < 3; ++a) {
            const float u = (c[a] - mn[a]) / fmaxf(mx[a] - mn[a], 1e-30f);
            q[a] = (uint32_t)fminf(fmaxf(u * 1023.0f, 0.0f), 1023.0f);
        }
        for (int b = 0; b < 10; ++b)
            for (int a = 0; a < 3; ++a) code |= (uint64_t)((q[a] >> b) & 1u) << (3 * b + a);
        keys[j] = code << 32 | (uint64_t)i;
    }
    qsort(keys, (size_t)live, sizeof(uint64_t), cull_cmp);
    g_cull.perm = (int32_t *)malloc(sizeof(int32_t) * (size_t)(live > 0 ? live : 1));
    for (int64_t j = 0; j < live; ++j) g_cull.perm[j] = (int32_t)(keys[j] & 0xffffffffu);
    g_cull.nodes = (CullNode *)malloc(sizeof(CullNode) * (size_t)(live > 0 ? live : 1));
    g_cull.n_nodes = 0;
    if (live > 0) cull_make(0, (int32_t)live, boxes);
    g_cull.prims = prims; g_cull.N = N;
    free(boxes); free(keys);
}

static int cand_cmp(const void *x, const void *y) { return ((const Cand *)x)->id - ((const Cand *)y)->id; }

static void cands_build_culled(CandList *L, const float *prims, f3 dir)
{
    int32_t stack[128];
    int sp = 0;
    if (g_cull.n_nodes > 0) stack[sp++] = 0;
    const float d[3] = {dir.x, dir.y, dir.z};
    while (sp > 0) {
        const CullNode *nd = &g_cull.nodes[stack[--sp]];
        float tn = -INFINITY, tf = INFINITY; /* the whole line: the predicate's roots do not depend on the interval */
        int miss = 0;
        for (int a = 0; a < 3 && !miss; ++a) {
            if (d[a] == 0.0f) { miss = nd->lo[a] > 0.0f || nd->hi[a] < 0.0f; continue; }
            const float inv = 1.0f / d[a];
            const float t0 = nd->lo[a] * inv, t1 = nd->hi[a] * inv;
            tn = fmaxf(tn, fminf(t0, t1)); tf = fminf(tf, fmaxf(t0, t1));
        }
        if (miss || tn > tf) continue;
        if (nd->b < 0) {
            for (int32_t j = nd->a; j < nd->a - nd->b; ++j) {
                const int32_t i = g_cull.perm[j];
                float r1, r2;
                if (line_roots(prims + 16 * (int64_t)i, dir, &r1, &r2)) cands_push(L, i, r1, r2);
            }
        } else if (sp + 2 <= 128) { /* depth <= log2(N) + 1 */
            stack[sp++] = nd->a; stack[sp++] = nd->b;
        }
    }
    qsort(L->c, (size_t)L->n, sizeof(Cand), cand_cmp); /* ascending index, as the brute force lists them */
}

static void cands_build(CandList *L, int64_t N, const float *prims, f3 dir)
{
    L->n = 0;
    if (g_cull.nodes && g_cull.prims == prims && g_cull.N == N) { cands_build_culled(L, prims, dir); return; }
    for (int64_t i = 0; i < N; ++i) {
        float r1, r2;
        if (line_roots(prims + 16 * i, dir, &r1, &r2)) cands_push(L, (int32_t)i, r1, r2);
    }
}

/* a10: first-hit query (optixTrace SBT 0 + __closesthit__ch 376-380 +         */
/* __miss__ms_ch 370-373): smallest reported t over prims hit in [tlo,thi],    */
/* -1.0f if none.  OptiX shrinks tmax as closer hits are accepted; the result  */
/* is the minimum either way.                                                  */
static float first_hit(const CandList *L, float tlo, float thi)
{
    float best = -1.0f; int found = 0;
    for (int64_t i = 0; i < L->n; ++i) {
        float t;
        if (segment_hit(L->c[i].r1, L->c[i].r2, tlo, thi, &t)) {
            if (!found || t < best) { best = t; found = 1; }
        }
    }
    return best;
}

/* a11: collect query (optixTrace SBT 1 + __anyhit__ah 349-367).  Order here   */
/* is ascending primitive index (OptiX's is unspecified).  Stops at cap        */
/* (optixTerminateRay at max_prim_slice) and reports the truncation.           */
static int collect(const CandList *L, float tlo, float thi, int cap, int32_t *ids, int *overflow)
{
    int p0 = 0; *overflow = 0;
    for (int64_t i = 0; i < L->n; ++i) {
        float t;
        if (segment_hit(L->c[i].r1, L->c[i].r2, tlo, thi, &t)) {
            if (p0 >= cap) { *overflow = 1; break; }
            ids[p0++] = L->c[i].id;
        }
    }
    return p0;
}

void orc_first_hit(int64_t N, const float *prims, int64_t n, const float *dirs, const float *tlo,
                   const float *thi, float *out_t)
{
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < n; ++r) {
            cands_build(&L, N, prims, mk3(dirs[3 * r], dirs[3 * r + 1], dirs[3 * r + 2]));
            out_t[r] = first_hit(&L, tlo[r], thi[r]);
        }
        free(L.c);
    }
}

/* per segment: count of hits and up to `cap` ids in ascending order */
void orc_trace_segments(int64_t N, const float *prims, int64_t n, const float *dirs,
                        const float *tlo, const float *thi, int cap, int32_t *counts, int32_t *ids)
{
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < n; ++r) {
            cands_build(&L, N, prims, mk3(dirs[3 * r], dirs[3 * r + 1], dirs[3 * r + 2]));
            int ov;
            int c = collect(&L, tlo[r], thi[r], cap, ids + (int64_t)r * cap, &ov);
            counts[r] = ov ? -c : c;
        }
        free(L.c);
    }
}

/* a13: gaussians_aabb.cu:112-180 accumulateChunk<16>.  buf[i] = (sigma, r, g, b) */
static void accumulate_chunk(const float *prims, const int32_t *ids, int p0, float tbuffer, f3 dir,
                             float dt, int i_begin, float buf[CHUNK_SIZE][4])
{
    memset(buf, 0, sizeof(float) * CHUNK_SIZE * 4);
    const float t_mid = fmaf(dt, (float)i_begin + 0.5f, tbuffer);
    const f3 ray_dir_tbuff = scl3(dir, t_mid);
    for (int h = 0; h < p0; ++h) {
        const float *p = prims + 16 * (int64_t)ids[h];
        const f3 pos_rel = mk3(p[0], p[1], p[2]);
        const float k = p[7];
        const f3 inv_scales = mk3(p[4] * k, p[5] * k, p[6] * k);
        const float power_cut = k * k;
        f3 U, V, W;
        quat_to_cols(p + 8, &U, &V, &W);
        const f3 xhit = add3(pos_rel, ray_dir_tbuff);
        const f3 Mx0 = apply_sinv_rt(xhit, U, V, W, inv_scales);
        const f3 Md = apply_sinv_rt(dir, U, V, W, inv_scales);
        const float Md2 = dot3(Md, Md);
        const float Md_dt_2 = (dt * dt) * Md2;
        float power = dot3(Mx0, Mx0);
        float inc = Md_dt_2 + 2.0f * dot3(Mx0, Md) * dt;
        const float inc_st = 2.0f * Md_dt_2;
        for (int i = 0; i < CHUNK_SIZE; ++i) {
            if (power < power_cut) {
                const float gw = expf(-0.5f * power);
                buf[i][0] += p[15] * gw;
                buf[i][1] += p[12] * gw;
                buf[i][2] += p[13] * gw;
                buf[i][3] += p[14] * gw;
            }
            power += inc;
            inc += inc_st;
        }
    }
}

/* scene-bbox slab test.  fwd: gaussians_aabb.cu:212-224 (multiply by the      */
/* reciprocal); bwd: backward/gaussians_aabb.cu:222-228 (divide).              */
static void bbox_interval(f3 o, f3 d, const float *bmin, const float *bmax, int divide,
                          float *tenter, float *texit)
{
    float t0[3], t1[3];
    const float oo[3] = {o.x, o.y, o.z}, dd[3] = {d.x, d.y, d.z};
    for (int a = 0; a < 3; ++a) {
        if (divide) { t0[a] = (bmin[a] - oo[a]) / dd[a]; t1[a] = (bmax[a] - oo[a]) / dd[a]; }
        else { float inv = 1.0f / dd[a]; t0[a] = (bmin[a] - oo[a]) * inv; t1[a] = (bmax[a] - oo[a]) * inv; }
    }
    float mn[3], mx[3];
    for (int a = 0; a < 3; ++a) { mn[a] = fminf(t0[a], t1[a]); mx[a] = fmaxf(t0[a], t1[a]); }
    *tenter = fmaxf(0.0f, fmaxf(mn[0], fmaxf(mn[1], mn[2])));
    *texit = fminf(mx[0], fminf(mx[1], mx[2]));
}

/* Optional per-ray slab trace, for the hit-set parity gate. */
typedef struct {
    int max_slabs, max_ids;
    int n_slabs, n_ids;
    float *slab_t;     /* (max_slabs,4): tbuffer, dt, t_min_slab, t_max_slab */
    int32_t *slab_off; /* (max_slabs+1) offsets into ids */
    int32_t *ids;
} Trace;

/* a12 + a14: gaussians_aabb.cu:205-340 __raygen__rg and 182-203 colorBlendingT_chunked */
static void march_forward_ray(const OrcCamera *cam, const OrcMarch *m, const float *bmin,
                              const float *bmax, int64_t N, const float *prims, int64_t ray,
                              CandList *L, int32_t *ids, float *out_rgb, OrcStats *st, Trace *tr,
                              float *out_depth)
{
    /* out_depth (optional): the viewer's expected depth, sum of T (1 - w) t over the samples
     * (cuda_gui/gaussians_aabb.cu:189-202) */
    float depth = 0.0f;
    if (out_depth) *out_depth = 0.0f;
    const unsigned ix = (unsigned)(ray % cam->width), iy = (unsigned)(ray / cam->width);
    const f3 o = mk3(cam->eye[0], cam->eye[1], cam->eye[2]);
    const f3 dir = compute_ray(cam, ix, iy);
    float tenter, texit;
    bbox_interval(o, dir, bmin, bmax, 0, &tenter, &texit);
    const float dt_base = m->dt_step;
    float dt = dt_base, slab_spacing = dt * BUFFER_SIZE;
    float T = 1.0f;
    f3 C = mk3(0, 0, 0);
    const float bg = m->white_background ? 1.0f : 0.0f;
    cands_build(L, N, prims, dir);
    const float fh = first_hit(L, tenter, texit);
    if (fh == -1.0f) { out_rgb[0] = out_rgb[1] = out_rgb[2] = bg; return; }
    st->rays_hit++;
    tenter = fh;
    if (!(tenter < texit)) { out_rgb[0] = out_rgb[1] = out_rgb[2] = bg; return; }
    float tbuffer = tenter;
    while (tbuffer < texit && T > m->t_eps) {
        if (m->dynamic_sampling) { /* gaussians_aabb.cu:267-272 */
            float dt_dist = fmaxf(tbuffer / 1024.0f, dt_base);
            float coeff = (1.0f / cbrtf(T)) * g_step_scale;
            dt = fminf(dt_dist * coeff, 4.0f * dt_base);
            slab_spacing = dt * BUFFER_SIZE;
        }
        const float t_min_slab = fmaxf(tenter, tbuffer);
        const float t_max_slab = fminf(texit, tbuffer + slab_spacing);
        if (t_max_slab > tenter) {
            int ov;
            const int p0 = collect(L, t_min_slab, t_max_slab, m->max_prim_slice, ids, &ov);
            if (ov) st->overflow_rays++;
            if (tr && tr->n_slabs < tr->max_slabs && tr->n_ids + p0 <= tr->max_ids) {
                float *s = tr->slab_t + 4 * tr->n_slabs;
                s[0] = tbuffer; s[1] = dt; s[2] = t_min_slab; s[3] = t_max_slab;
                tr->slab_off[tr->n_slabs] = tr->n_ids;
                memcpy(tr->ids + tr->n_ids, ids, sizeof(int32_t) * (size_t)p0);
                tr->n_ids += p0; tr->n_slabs++;
                tr->slab_off[tr->n_slabs] = tr->n_ids;
            }
            if (p0 == 0) {
                st->empty_slabs++;
                tbuffer += slab_spacing;
                const float nt = first_hit(L, tbuffer, texit);
                if (nt == -1.0f) break;
                tbuffer = nt;
                continue;
            }
            st->slabs++;
            st->hit_pairs += p0;
            float t_sample = tbuffer + 0.5f * dt; /* cuda_gui/gaussians_aabb.cu:189 */
            for (int base = 0; base < BUFFER_SIZE && T > m->t_eps; base += CHUNK_SIZE) {
                float local[CHUNK_SIZE][4];
                accumulate_chunk(prims, ids, p0, tbuffer, dir, dt, base, local);
                for (int i = 0; i < CHUNK_SIZE; ++i) { /* gaussians_aabb.cu:195-201 */
                    const float x = local[i][0] * dt;
                    const float w = expf(-x);
                    const float s = dt * ((1.0f - w) / fmaxf(x, 1e-6f));
                    const float ts = T * s;
                    C = add3(C, mk3(ts * local[i][1], ts * local[i][2], ts * local[i][3]));
                    depth += T * (1.0f - w) * t_sample;
                    T *= w;
                    t_sample += dt;
                }
            }
        }
        tbuffer += slab_spacing;
    }
    out_rgb[0] = C.x + T * bg; out_rgb[1] = C.y + T * bg; out_rgb[2] = C.z + T * bg;
    if (out_depth) *out_depth = depth;
}

static void stats_add(OrcStats *a, const OrcStats *b)
{
    a->hit_pairs += b->hit_pairs; a->slabs += b->slabs; a->empty_slabs += b->empty_slabs;
    a->overflow_rays += b->overflow_rays; a->rays_hit += b->rays_hit;
}

/* ray_colors is the full (W*H,3) image; ray_ids (n) selects the rays to march
 * (NULL = all W*H rays). */
void orc_march_forward(const OrcCamera *cam, const OrcMarch *m, const float *bmin, const float *bmax,
                       int64_t N, const float *prims, int64_t n, const int64_t *ray_ids,
                       float *ray_colors, OrcStats *stats)
{
    OrcStats total; memset(&total, 0, sizeof total);
    if (!ray_ids) n = (int64_t)cam->width * cam->height;
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
        int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(m->max_prim_slice > 0 ? m->max_prim_slice : 1));
        OrcStats st; memset(&st, 0, sizeof st);
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < n; ++r) {
            int64_t ray = ray_ids ? ray_ids[r] : r;
            march_forward_ray(cam, m, bmin, bmax, N, prims, ray, &L, ids, ray_colors + 3 * ray, &st, NULL, NULL);
        }
#pragma omp critical
        stats_add(&total, &st);
        free(ids); free(L.c);
    }
    if (stats) *stats = total;
}

/* orc_march_forward with the march counters kept per ray: counts (n,2) = slabs blended and the
 * sum of their hit-list lengths, for the n rays of ray_ids (NULL = all).  Tells a test which rays
 * marched the same slab sequence on both sides when the adaptive step makes that depend on the
 * last bit of cbrt / exp. */
void orc_march_forward_counts(const OrcCamera *cam, const OrcMarch *m, const float *bmin, const float *bmax,
                              int64_t N, const float *prims, int64_t n, const int64_t *ray_ids,
                              float *ray_colors, int64_t *counts)
{
    if (!ray_ids) n = (int64_t)cam->width * cam->height;
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
        int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(m->max_prim_slice > 0 ? m->max_prim_slice : 1));
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < n; ++r) {
            int64_t ray = ray_ids ? ray_ids[r] : r;
            OrcStats st; memset(&st, 0, sizeof st);
            march_forward_ray(cam, m, bmin, bmax, N, prims, ray, &L, ids, ray_colors + 3 * ray, &st, NULL, NULL);
            counts[2 * r] = st.slabs;
            counts[2 * r + 1] = st.hit_pairs;
        }
        free(ids); free(L.c);
    }
}

/* cuda_gui/helpers.h:45-59: clamp to [0,1], then min(uint(x * 256), 255) */
static unsigned char quantize8(float x)
{
    x = fminf(fmaxf(x, 0.0f), 1.0f);
    const unsigned v = (unsigned)(x * 256.0f);
    return (unsigned char)(v < 255u ? v : 255u);
}

/* The viewer's launch (cuda_gui/gaussians_aabb.cu __raygen__rg): the forward march on a black
 * background, colours quantised to uchar4 (alpha 255), expected depth per ray.  `colors` (W*H,3)
 * receives the unquantised colours as well. */
void orc_march_gui(const OrcCamera *cam, const OrcMarch *m, const float *bmin, const float *bmax,
                   int64_t N, const float *prims, unsigned char *frame, float *depth, float *colors)
{
    OrcMarch mm = *m;
    mm.white_background = 0;
    const int64_t n = (int64_t)cam->width * cam->height;
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
        int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(mm.max_prim_slice > 0 ? mm.max_prim_slice : 1));
        OrcStats st; memset(&st, 0, sizeof st);
#pragma omp for schedule(dynamic, 16)
        for (int64_t ray = 0; ray < n; ++ray) {
            float rgb[3];
            march_forward_ray(cam, &mm, bmin, bmax, N, prims, ray, &L, ids, rgb, &st, NULL, depth + ray);
            for (int c = 0; c < 3; ++c) { frame[4 * ray + c] = quantize8(rgb[c]); colors[3 * ray + c] = rgb[c]; }
            frame[4 * ray + 3] = 255;
        }
        free(ids); free(L.c);
    }
}

/* One ray with its slab-by-slab hit lists recorded.  Returns the number of
 * slabs recorded (collect queries, including empty ones). */
int orc_march_trace(const OrcCamera *cam, const OrcMarch *m, const float *bmin, const float *bmax,
                    int64_t N, const float *prims, int64_t ray, int max_slabs, int max_ids,
                    float *slab_t, int32_t *slab_off, int32_t *ids_out, float *rgb_out)
{
    CandList L = {0, 0, 0};
    int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(m->max_prim_slice > 0 ? m->max_prim_slice : 1));
    OrcStats st; memset(&st, 0, sizeof st);
    Trace tr = {max_slabs, max_ids, 0, 0, slab_t, slab_off, ids_out};
    slab_off[0] = 0;
    march_forward_ray(cam, m, bmin, bmax, N, prims, ray, &L, ids, rgb_out, &st, &tr, NULL);
    free(ids); free(L.c);
    return tr.n_slabs;
}

/* ------------------------------------------------------------------------- */
/* a15: backward/gaussians_aabb.cu:113-184 accumulateChunk_backw               */
static void accumulate_chunk_backw(const float *prims, const int32_t *ids, int p0, float tbuffer,
                                   f3 dir, float dt, int i_begin, f3 diff, float buf[CHUNK_SIZE][2])
{
    memset(buf, 0, sizeof(float) * CHUNK_SIZE * 2);
    const float t_mid = fmaf(dt, (float)i_begin + 0.5f, tbuffer);
    const f3 ray_dir_tbuff = scl3(dir, t_mid);
    for (int h = 0; h < p0; ++h) {
        const float *p = prims + 16 * (int64_t)ids[h];
        const f3 pos_rel = mk3(p[0], p[1], p[2]);
        const float k = p[7];
        const f3 inv_scales = mk3(p[4] * k, p[5] * k, p[6] * k);
        const float power_cut = k * k;
        const float ddc = dot3(diff, mk3(p[12], p[13], p[14]));
        f3 U, V, W;
        quat_to_cols(p + 8, &U, &V, &W);
        const f3 xhit = add3(pos_rel, ray_dir_tbuff);
        const f3 Mx0 = apply_sinv_rt(xhit, U, V, W, inv_scales);
        const f3 Md = apply_sinv_rt(dir, U, V, W, inv_scales);
        const float Md2 = dot3(Md, Md);
        const float Md_dt_2 = (dt * dt) * Md2;
        float power = dot3(Mx0, Mx0);
        float inc = Md_dt_2 + 2.0f * dot3(Mx0, Md) * dt;
        const float inc_st = 2.0f * Md_dt_2;
        for (int i = 0; i < CHUNK_SIZE; ++i) {
            if (power < power_cut) {
                const float gw = expf(-0.5f * power);
                buf[i][0] += p[15] * gw;
                buf[i][1] += ddc * gw;
            }
            power += inc;
            inc += inc_st;
        }
    }
}

typedef struct { double *ddens, *drgb, *dpos, *dscale, *dquat; } GradAcc;

static inline void acc_add(double *p, float v)
{
#pragma omp atomic
    *p += (double)v;
}

/* a15: backward/gaussians_aabb.cu:209-497 __raygen__rg (replay + gradients).  */
/* Per-(ray,slab,hit) contributions are formed in fp32 exactly as written;     */
/* the reference adds them into 4 replica buffers with fp32 atomicAdd and sums */
/* the replicas afterwards (optix_utils.py:325-361) -- the cross-ray sum is    */
/* order-free, and is carried in double here.                                  */
static void march_backward_ray(const OrcCamera *cam, const OrcMarch *m, const float *bmin,
                               const float *bmax, int64_t N, const float *prims, int64_t ray,
                               const float *ray_color, const float *dloss, CandList *L,
                               int32_t *ids, GradAcc *g, OrcStats *st, int64_t *in_cut)
{
    const unsigned ix = (unsigned)(ray % cam->width), iy = (unsigned)(ray / cam->width);
    const f3 o = mk3(cam->eye[0], cam->eye[1], cam->eye[2]);
    const f3 dir = compute_ray(cam, ix, iy);
    float tenter, texit;
    bbox_interval(o, dir, bmin, bmax, 1, &tenter, &texit);
    const float dt_base = m->dt_step;
    float dt = dt_base, slab_spacing = dt * BUFFER_SIZE;
    cands_build(L, N, prims, dir);
    const float fh = first_hit(L, tenter, texit);
    if (fh == -1.0f) return;
    tenter = fh;
    if (!(tenter < texit)) return;
    float tbuffer = tenter;
    float T = 1.0f;
    const f3 diff = mk3(dloss[0], dloss[1], dloss[2]);
    float D = dot3(diff, mk3(ray_color[0], ray_color[1], ray_color[2]));
    while (tbuffer < texit && T > m->t_eps) {
        if (m->dynamic_sampling) {
            float dt_dist = fmaxf(tbuffer / 1024.0f, dt_base);
            float coeff = (1.0f / cbrtf(T)) * g_step_scale;
            dt = fminf(dt_dist * coeff, 4.0f * dt_base);
            slab_spacing = dt * BUFFER_SIZE;
        }
        const float t_min_slab = tbuffer; /* unclipped: backward/gaussians_aabb.cu:279-280 */
        const float t_max_slab = tbuffer + slab_spacing;
        if (t_max_slab > tenter) {
            int ov;
            const int p0 = collect(L, t_min_slab, t_max_slab, m->max_prim_slice, ids, &ov);
            if (ov) st->overflow_rays++;
            if (p0 == 0) {
                tbuffer += slab_spacing;
                const float nt = first_hit(L, tbuffer, texit);
                if (nt == -1.0f) break;
                tbuffer = nt;
                continue;
            }
            st->slabs++;
            st->hit_pairs += p0;
            float buffers[2][CHUNK_SIZE][2];
            for (int b = 0; b < 2; ++b)
                accumulate_chunk_backw(prims, ids, p0, tbuffer, dir, dt, b * CHUNK_SIZE, diff, buffers[b]);
            /* backward/gaussians_aabb.cu:330-352 prefix loop */
            float T_after = T, D_after = D;
            for (int b = 0; b < 2; ++b)
                for (int i = 0; i < CHUNK_SIZE; ++i) {
                    const float sd = buffers[b][i][0];
                    float e = buffers[b][i][1];
                    const float inv_d = (sd > 0.0f) ? 1.0f / sd : 0.0f;
                    e *= inv_d;
                    const float w = expf(-sd * dt);
                    buffers[b][i][1] = e;
                    D_after -= T_after * (1.0f - w) * e;
                    T_after *= w;
                }
            /* backward/gaussians_aabb.cu:353-490 per-hit gradient loop */
            for (int h = 0; h < p0; ++h) {
                const int32_t id = ids[h];
                const float *p = prims + 16 * (int64_t)id;
                float Dt = D, Tt = T;
                float grad_color = 0.f, dsig = 0.f;
                f3 dscale = mk3(0, 0, 0), dpos = mk3(0, 0, 0);
                f3 dr1 = mk3(0, 0, 0), dr2 = mk3(0, 0, 0), dr3 = mk3(0, 0, 0);
                const f3 pos_rel = mk3(p[0], p[1], p[2]);
                const float k = p[7];
                const f3 inv_s = mk3(p[4] * k, p[5] * k, p[6] * k);
                const float power_cut = k * k;
                f3 U, V, W;
                quat_to_cols(p + 8, &U, &V, &W);
                /* the same power by the forward's arrangement (gaussians_aabb.cu:135-164: t_mid by fmaf, the   */
                /* dot-product form of S^-1 R^T), its recurrence carried over the slab's 32 samples: see          */
                /* orc_set_backward_mask_form()                                                                  */
                const f3 fx0 = apply_sinv_rt(add3(pos_rel, scl3(dir, fmaf(dt, 0.5f, tbuffer))), U, V, W, inv_s);
                const f3 fMd = apply_sinv_rt(dir, U, V, W, inv_s);
                const float fMd_dt_2 = (dt * dt) * dot3(fMd, fMd);
                float fpower = dot3(fx0, fx0);
                float finc = fMd_dt_2 + 2.0f * dot3(fx0, fMd) * dt;
                const float finc_st = 2.0f * fMd_dt_2;
                U = scl3(U, inv_s.x); V = scl3(V, inv_s.y); W = scl3(W, inv_s.z);
                const f3 M1 = mk3(U.x, V.x, W.x), M2 = mk3(U.y, V.y, W.y), M3 = mk3(U.z, V.z, W.z);
                const float gd = p[15];
                const float dcg = dot3(mk3(p[12], p[13], p[14]), diff) / p[15];
                const float t0 = tbuffer + 0.5f * dt;
                f3 x = add3(pos_rel, scl3(dir, t0));
                f3 Mx = add3(add3(scl3(M1, x.x), scl3(M2, x.y)), scl3(M3, x.z));
                const f3 Md = add3(add3(scl3(M1, dir.x), scl3(M2, dir.y)), scl3(M3, dir.z));
                const float Md2 = dot3(Md, Md);
                const float Md_dt_2 = (dt * dt) * Md2;
                float power = dot3(Mx, Mx);
                float inc = Md_dt_2 + 2.0f * dot3(Mx, Md) * dt;
                const float inc_st = 2.0f * Md_dt_2;
                for (int base = 0; base < BUFFER_SIZE && Tt > m->t_eps; base += CHUNK_SIZE) {
                    const int b = base / CHUNK_SIZE;
                    for (int i = 0; i < CHUNK_SIZE; ++i) {
                        const float sigma = buffers[b][i][0];
                        const float w = expf(-sigma * dt);
                        const float e = buffers[b][i][1];
                        const int in_b = power < power_cut, in_f = fpower < power_cut;
                        if (in_cut) { in_cut[0] += in_b; in_cut[1] += in_b != in_f; }
                        if (g_mask_form ? in_f : in_b) {
                            const float aT = Tt * (1.0f - w) * ((sigma > 0.0f) ? 1.0f / sigma : 0.0f);
                            const float wd = expf(-0.5f * power);
                            const float sw = wd * gd;
                            grad_color += sw * aT;
                            const float aux = (Tt * e - Dt) * dt;
                            dsig += aux * wd;
                            float dW = aux * gd;
                            dW += aT * gd * (dcg - e);
                            dsig += aT * wd * (dcg - e);
                            dscale.x += dW * wd * (Mx.x * Mx.x) * inv_s.x;
                            dscale.y += dW * wd * (Mx.y * Mx.y) * inv_s.y;
                            dscale.z += dW * wd * (Mx.z * Mx.z) * inv_s.z;
                            dpos.x += dW * wd * dot3(M1, Mx);
                            dpos.y += dW * wd * dot3(M2, Mx);
                            dpos.z += dW * wd * dot3(M3, Mx);
                            dr1 = sub3(dr1, scl3(scl3(x, dW * wd), Mx.x * inv_s.x));
                            dr2 = sub3(dr2, scl3(scl3(x, dW * wd), Mx.y * inv_s.y));
                            dr3 = sub3(dr3, scl3(scl3(x, dW * wd), Mx.z * inv_s.z));
                        }
                        x = add3(x, scl3(dir, dt));
                        Mx = add3(Mx, scl3(Md, dt));
                        power += inc;
                        inc += inc_st;
                        fpower += finc;
                        finc += finc_st;
                        Dt -= Tt * (1.0f - w) * e;
                        Tt *= w;
                    }
                }
                acc_add(&g->drgb[3 * id + 0], diff.x * grad_color);
                acc_add(&g->drgb[3 * id + 1], diff.y * grad_color);
                acc_add(&g->drgb[3 * id + 2], diff.z * grad_color);
                acc_add(&g->ddens[id], dsig);
                acc_add(&g->dscale[3 * id + 0], dscale.x);
                acc_add(&g->dscale[3 * id + 1], dscale.y);
                acc_add(&g->dscale[3 * id + 2], dscale.z);
                acc_add(&g->dpos[3 * id + 0], dpos.x);
                acc_add(&g->dpos[3 * id + 1], dpos.y);
                acc_add(&g->dpos[3 * id + 2], dpos.z);
                /* backward/gaussians_aabb.cu:469-481, q = (x,y,z,w) = (r,i,j,k) */
                const float qx = p[8], qy = p[9], qz = p[10], qw = p[11];
                const float gqx = (2 * qw * dr1.y - 2 * qz * dr1.z - 2 * qw * dr2.x + 2 * qy * dr2.z + 2 * qz * dr3.x - 2 * qy * dr3.y);
                const float gqy = (2 * qz * dr1.y + 2 * qw * dr1.z + 2 * qz * dr2.x - 4 * qy * dr2.y + 2 * qx * dr2.z + 2 * qw * dr3.x - 2 * qx * dr3.y - 4 * qy * dr3.z);
                const float gqz = (-4 * qz * dr1.x + 2 * qy * dr1.y - 2 * qx * dr1.z + 2 * qy * dr2.x + 2 * qw * dr2.z + 2 * qx * dr3.x + 2 * qw * dr3.y - 4 * qz * dr3.z);
                const float gqw = (-4 * qw * dr1.x + 2 * qx * dr1.y + 2 * qy * dr1.z - 2 * qx * dr2.x - 4 * qw * dr2.y + 2 * qz * dr2.z + 2 * qy * dr3.x + 2 * qz * dr3.y);
                acc_add(&g->dquat[4 * id + 0], gqx);
                acc_add(&g->dquat[4 * id + 1], gqy);
                acc_add(&g->dquat[4 * id + 2], gqz);
                acc_add(&g->dquat[4 * id + 3], gqw);
            }
            D = D_after;
            T = T_after;
        }
        tbuffer += slab_spacing;
    }
}

/* ray_colors / dloss are full (W*H,3) images; gradients are returned w.r.t.
 * density, rgb (the SH output colour), position, scale, quaternion. */
void orc_march_backward(const OrcCamera *cam, const OrcMarch *m, const float *bmin, const float *bmax,
                        int64_t N, const float *prims, int64_t n, const int64_t *ray_ids,
                        const float *ray_colors, const float *dloss, float *ddens, float *drgb,
                        float *dpos, float *dscale, float *dquat, OrcStats *stats)
{
    GradAcc g;
    g.ddens = (double *)calloc((size_t)N, sizeof(double));
    g.drgb = (double *)calloc((size_t)N * 3, sizeof(double));
    g.dpos = (double *)calloc((size_t)N * 3, sizeof(double));
    g.dscale = (double *)calloc((size_t)N * 3, sizeof(double));
    g.dquat = (double *)calloc((size_t)N * 4, sizeof(double));
    OrcStats total; memset(&total, 0, sizeof total);
    if (!ray_ids) n = (int64_t)cam->width * cam->height;
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
        int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(m->max_prim_slice > 0 ? m->max_prim_slice : 1));
        OrcStats st; memset(&st, 0, sizeof st);
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < n; ++r) {
            int64_t ray = ray_ids ? ray_ids[r] : r;
            march_backward_ray(cam, m, bmin, bmax, N, prims, ray, ray_colors + 3 * ray, dloss + 3 * ray,
                               &L, ids, &g, &st, NULL);
        }
#pragma omp critical
        stats_add(&total, &st);
        free(ids); free(L.c);
    }
    for (int64_t i = 0; i < N; ++i) ddens[i] = (float)g.ddens[i];
    for (int64_t i = 0; i < 3 * N; ++i) { drgb[i] = (float)g.drgb[i]; dpos[i] = (float)g.dpos[i]; dscale[i] = (float)g.dscale[i]; }
    for (int64_t i = 0; i < 4 * N; ++i) dquat[i] = (float)g.dquat[i];
    free(g.ddens); free(g.drgb); free(g.dpos); free(g.dscale); free(g.dquat);
    if (stats) *stats = total;
}

/* ------------------------------------------------------------------------- */
/* a19: utils/reordering_utils.py:55-104 quantify_pos_min_max + morton_code    */
/* scale = 1023 / (max - min + 1e-9) evaluated in fp32 as torch does, the      */
/* product truncated toward zero to int32; bits x->3i, y->3i+1, z->3i+2.       */
void orc_morton_codes(int64_t N, const float *pos, int64_t *codes)
{
    float mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
    for (int64_t n = 0; n < N; ++n)
        for (int a = 0; a < 3; ++a) {
            float v = pos[3 * n + a];
            if (v < mn[a]) mn[a] = v;
            if (v > mx[a]) mx[a] = v;
        }
    float scale[3];
    for (int a = 0; a < 3; ++a) scale[a] = 1023.0f / ((mx[a] - mn[a]) + 1e-9f);
    for (int64_t n = 0; n < N; ++n) {
        int32_t q[3];
        for (int a = 0; a < 3; ++a) q[a] = (int32_t)((pos[3 * n + a] - mn[a]) * scale[a]);
        int64_t code = 0;
        for (int i = 0; i < 10; ++i) {
            code |= (int64_t)((q[0] >> i) & 1) << (3 * i);
            code |= (int64_t)((q[1] >> i) & 1) << (3 * i + 1);
            code |= (int64_t)((q[2] >> i) & 1) << (3 * i + 2);
        }
        codes[n] = code;
    }
}

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Sensitivity probe for the tests: scales the adaptive step's coefficient (1.0f: exactly the
 * reference's arithmetic; 1 + 2^-23: as if cbrtf had rounded the other way). */
void orc_set_step_scale(float s) { g_step_scale = s; }

/* Probes of the backward's cut-off decisions (tests only).  The gradient loop of the backward
 * (backward/gaussians_aabb.cu:375-396) decides `power < k^2` per sample from its own arrangement of
 * the arithmetic -- the sample point by t0 = tbuffer + 0.5 dt and a 3x3 matrix product -- which is not
 * the forward's (112-180: t_mid by fmaf, S^-1 R^T by dot products).  For a thin Gaussian one ulp of t
 * moves the power by 1e-4 of its value, so the reference's own two passes disagree on samples that sit
 * within that of k^2, and a sample flipped is, for a few hundred rays, 1e-3 of the whole gradient.
 * orc_march_backward_in_cut returns per ray {samples the gradient loop took as inside a cut-off, samples on
 * which the two arrangements disagree}; orc_set_backward_mask_form(1) makes the loop decide by the forward's
 * arrangement (its set-up at the slab's first sample, the recurrence carried over all 32 samples), everything
 * else as the reference has it; 0 is the reference. */
void orc_set_backward_mask_form(int forward_form) { g_mask_form = forward_form; }

void orc_march_backward_in_cut(const OrcCamera *cam, const OrcMarch *m, const float *bmin, const float *bmax,
                               int64_t N, const float *prims, int64_t n, const int64_t *ray_ids,
                               const float *ray_colors, int64_t *in_cut)
{
    GradAcc g;
    g.ddens = (double *)calloc((size_t)N, sizeof(double));
    g.drgb = (double *)calloc((size_t)N * 3, sizeof(double));
    g.dpos = (double *)calloc((size_t)N * 3, sizeof(double));
    g.dscale = (double *)calloc((size_t)N * 3, sizeof(double));
    g.dquat = (double *)calloc((size_t)N * 4, sizeof(double));
    if (!ray_ids) n = (int64_t)cam->width * cam->height;
    const float zero[3] = {0.f, 0.f, 0.f};
#pragma omp parallel
    {
        CandList L = {0, 0, 0};
        int32_t *ids = (int32_t *)malloc(sizeof(int32_t) * (size_t)(m->max_prim_slice > 0 ? m->max_prim_slice : 1));
        OrcStats st; memset(&st, 0, sizeof st);
#pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < n; ++r) {
            int64_t ray = ray_ids ? ray_ids[r] : r;
            in_cut[2 * r] = in_cut[2 * r + 1] = 0;
            march_backward_ray(cam, m, bmin, bmax, N, prims, ray, ray_colors + 3 * ray, zero, &L, ids, &g, &st, in_cut + 2 * r);
        }
        free(ids); free(L.c);
    }
    free(g.ddens); free(g.drgb); free(g.dpos); free(g.dscale); free(g.dquat);
}

void orc_set_num_threads(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------------- */
/* distCUDA2 (submodules/simple-knn/simple_knn.cu:137-184): mean of the squared
 * distances to the three nearest other points.  The reference prunes with Morton-sorted boxes;
 * its pruning is exact, so brute force gives the same three distances.  updateKBest<3> is kept
 * as written (insertion into a sorted triple); dist = (dx*dx + dy*dy) + dz*dz. */
void orc_dist2_knn3(int64_t n, const float *pos, float *out)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t i = 0; i < n; ++i) {
        float best[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
        for (int64_t j = 0; j < n; ++j) {
            if (j == i) continue;
            const float dx = pos[3 * j] - pos[3 * i], dy = pos[3 * j + 1] - pos[3 * i + 1], dz = pos[3 * j + 2] - pos[3 * i + 2];
            float dist = (dx * dx + dy * dy) + dz * dz;
            for (int k = 0; k < 3; ++k)
                if (best[k] > dist) { const float t = best[k]; best[k] = dist; dist = t; }
        }
        out[i] = ((best[0] + best[1]) + best[2]) / 3.0f;
    }
}
