// Shared device-side definitions of librgx: canonical fp32 arithmetic of the
// hit predicate, BVH node layout, skip-link traversal, workspace layout.
//
// Canonical arithmetic (what makes per-segment hit sets reproducible bit for
// bit against a CPU evaluation of the same formulas): IEEE binary32, the
// translation units are compiled with -ffp-contract=off so a*b+c stays two
// roundings unless written as fmaf, fmaf exactly where the reference's
// intersection program writes fmaf, dot = (x*x' + y*y') + z*z',
// reciprocal and division correctly rounded, logf(x) := (float)log((double)x).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/rgx.h"

#define RGX_BUFFER_SIZE 32 // samples per slab   (cuda_train/forward/gaussians_aabb.h:2)
#define RGX_CHUNK_SIZE 16  // samples per chunk  (cuda_train/forward/gaussians_aabb.h:3)

struct f3 {
    float x, y, z;
};
__device__ __forceinline__ f3 mk3(float x, float y, float z) { return f3{x, y, z}; }
__device__ __forceinline__ f3 operator+(f3 a, f3 b) { return mk3(a.x + b.x, a.y + b.y, a.z + b.z); }
__device__ __forceinline__ f3 operator-(f3 a, f3 b) { return mk3(a.x - b.x, a.y - b.y, a.z - b.z); }
__device__ __forceinline__ f3 operator*(f3 a, float s) { return mk3(a.x * s, a.y * s, a.z * s); }
__device__ __forceinline__ float dot3(f3 a, f3 b) { return (a.x * b.x + a.y * b.y) + a.z * b.z; }
__device__ __forceinline__ float canon_logf(float x) { return (float)log((double)x); }

// Columns of the rotation matrix of quaternion (r,i,j,k)
// (cuda_train/forward/gaussians_aabb.cu:7-17).
__device__ __forceinline__ void quat_to_cols(float4 q, f3 &c0, f3 &c1, f3 &c2)
{
    const float r = q.x, i = q.y, j = q.z, k = q.w;
    const float ii = i + i, jj = j + j, kk = k + k;
    const float ri = r * ii, rj = r * jj, rk = r * kk;
    const float ii2 = i * ii, jj2 = j * jj, kk2 = k * kk;
    const float ij = i * jj, ik = i * kk, jk = j * kk;
    c0 = mk3(1.f - (jj2 + kk2), ij + rk, ik - rj);
    c1 = mk3(ij - rk, 1.f - (ii2 + kk2), jk + ri);
    c2 = mk3(ik + rj, jk - ri, 1.f - (ii2 + jj2));
}

// S^-1 R^T x (cuda_train/forward/gaussians_aabb.cu:19-30).
__device__ __forceinline__ f3 apply_sinv_rt(f3 x, f3 U, f3 V, f3 W, f3 inv_s)
{
    const float rx = fmaf(U.x, x.x, fmaf(U.y, x.y, U.z * x.z));
    const float ry = fmaf(V.x, x.x, fmaf(V.y, x.y, V.z * x.z));
    const float rz = fmaf(W.x, x.x, fmaf(W.y, x.y, W.z * x.z));
    return mk3(rx * inv_s.x, ry * inv_s.y, rz * inv_s.z);
}

// 64-byte primitive record (cuda_train/forward/gaussians_aabb.h:7-12).
struct __align__(16) Prim {
    float4 pos4;       // eye - centre, 0
    float4 inv_inter4; // (1/scale)/k, k
    float4 quat4;      // w,x,y,z
    float4 rgba4;      // rgb*density, density
};

// The part of __intersection__gaussian (gaussians_aabb.cu:43-82) that does not
// depend on the ray interval: true when the line meets the k-sigma ellipsoid,
// with the two roots.
__device__ __forceinline__ bool line_roots(float4 pos4, float4 inv4, float4 quat, f3 dir, float &r1, float &r2)
{
    const f3 inv_scales = mk3(inv4.x, inv4.y, inv4.z);
    const f3 O = mk3(pos4.x, pos4.y, pos4.z);
    f3 U, V, W;
    quat_to_cols(quat, U, V, W);
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
        r1 = c / q;
        r2 = q * inv_a;
        return true;
    }
    return false;
}

// Interval part (gaussians_aabb.cu:84-89).
__device__ __forceinline__ bool segment_hit(float r1, float r2, float tmin, float tmax, float &t)
{
    const float min_t = fmaxf(tmin, r1);
    const float max_t = fminf(tmax, r2);
    t = min_t;
    return min_t <= max_t;
}

// ---------------------------------------------------------------------------
// BVH: binary radix tree with skip links ("ropes"), 32 bytes per node.
// Internal nodes are [0, n-1), leaf j (j-th Gaussian in Morton order) is node
// n-1+j.  Traversal needs no stack: on a box hit go to `left` (internal) or
// test the primitive (leaf) and follow `skip`; on a miss follow `skip`.
struct __align__(16) Node {
    float lo[3];
    int32_t left; // internal: index of the left child; leaf: ~(sorted primitive index)
    float hi[3];
    int32_t skip; // next node when this subtree is done or culled; -1 = end
};

struct __align__(16) WsHeader {
    float bb_min[3];
    float bb_max[3];
    int32_t bb_min_enc[3]; // order-preserving int encodings used by the atomic reduction
    int32_t bb_max_enc[3];
    int64_t n;
    int32_t root;
    int32_t built;
    int32_t refit_ok; // set by a refit's first kernel: the workspace held a finished tree over the same number of boxes
    int32_t pad_[3];
};

struct WsLayout {
    size_t header, aabb, keys0, keys1, vals0, vals1, nodes, parent, right, flags, hist, total;
};

#define RGX_RS_THREADS 256
#ifndef RGX_RS_ITEMS
#define RGX_RS_ITEMS 8
#endif
#define RGX_RS_TILE (RGX_RS_THREADS * RGX_RS_ITEMS)

static inline size_t rgx_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

static inline WsLayout rgx_ws_layout(int64_t n)
{
    WsLayout L;
    const size_t nn = (size_t)(n > 0 ? n : 1);
    const size_t nblocks = (nn + RGX_RS_TILE - 1) / RGX_RS_TILE;
    size_t off = 0;
    L.header = off; off = rgx_align_up(off + sizeof(WsHeader), 256);
    L.aabb = off;   off = rgx_align_up(off + nn * 6 * sizeof(float), 256);
    L.keys0 = off;  off = rgx_align_up(off + nn * sizeof(uint64_t), 256);
    L.keys1 = off;  off = rgx_align_up(off + nn * sizeof(uint64_t), 256);
    L.vals0 = off;  off = rgx_align_up(off + nn * sizeof(uint32_t), 256); // after the build: sorted position -> input index
    L.vals1 = off;  off = rgx_align_up(off + nn * sizeof(uint32_t), 256); // after the build: input index -> sorted position
    L.nodes = off;  off = rgx_align_up(off + (2 * nn) * sizeof(Node), 256);
    L.parent = off; off = rgx_align_up(off + (2 * nn) * sizeof(int32_t), 256);
    L.right = off;  off = rgx_align_up(off + nn * sizeof(int32_t), 256);
    L.flags = off;  off = rgx_align_up(off + nn * sizeof(int32_t), 256);
    L.hist = off;   off = rgx_align_up(off + 256 * (nblocks + 1) * sizeof(uint32_t), 256);
    L.total = off;
    return L;
}

// Pointers into a built workspace, as the march kernels see it.
struct BvhView {
    const Node *nodes;
    const uint32_t *order; // sorted position -> input index
    const WsHeader *hdr;
    int32_t root;
    int64_t n;
};

// Per-ray constants of the conservative node test.  Node boxes are unions of
// the fp32 k-sigma AABBs; the hit predicate above is evaluated in fp32 on
// quantities of magnitude |eye - centre| / scale, so it can accept a ray that
// misses the exact ellipsoid by a few ulp of the distance travelled.  The node
// test therefore widens every slab by pad = RGX_PAD_REL * max(t_hi, 1) world
// units, far more than that rounding and far less than any Gaussian.
#define RGX_PAD_REL 8e-6f

struct RayBox {
    f3 o, inv, pad; // pad.x = world pad * |inv.x| : the pad expressed in t along each axis
};

__device__ __forceinline__ float clamp_inv(float d)
{
    float inv = 1.0f / d;
    // axis-parallel rays: keep the slab arithmetic finite (the pad then accepts
    // every box on that axis, which is conservative)
    if (!(fabsf(inv) < 1e30f)) inv = copysignf(1e30f, d);
    return inv;
}

__device__ __forceinline__ RayBox make_raybox(f3 o, f3 dir, float thi)
{
    RayBox rb;
    rb.o = o;
    rb.inv = mk3(clamp_inv(dir.x), clamp_inv(dir.y), clamp_inv(dir.z));
    const float pad = RGX_PAD_REL * fmaxf(fabsf(thi), 1.0f);
    rb.pad = mk3(pad * fabsf(rb.inv.x), pad * fabsf(rb.inv.y), pad * fabsf(rb.inv.z));
    return rb;
}

__device__ __forceinline__ bool box_overlaps(const RayBox &rb, float4 a, float4 b, float tlo, float thi)
{
    const float x0 = (a.x - rb.o.x) * rb.inv.x, x1 = (b.x - rb.o.x) * rb.inv.x;
    const float y0 = (a.y - rb.o.y) * rb.inv.y, y1 = (b.y - rb.o.y) * rb.inv.y;
    const float z0 = (a.z - rb.o.z) * rb.inv.z, z1 = (b.z - rb.o.z) * rb.inv.z;
    const float tn = fmaxf(fmaxf(fminf(x0, x1) - rb.pad.x, fminf(y0, y1) - rb.pad.y),
                           fmaxf(fminf(z0, z1) - rb.pad.z, tlo));
    const float tf = fminf(fminf(fmaxf(x0, x1) + rb.pad.x, fmaxf(y0, y1) + rb.pad.y),
                           fminf(fmaxf(z0, z1) + rb.pad.z, thi));
    return tn <= tf;
}

// Pixel -> ray (cuda_train/forward/gaussians_aabb.cu:95-110 computeRay).
__device__ __forceinline__ f3 compute_ray(const RgxCamera &c, unsigned ix, unsigned iy)
{
    const float idx_x = ((float)ix + 0.5f) / (float)(unsigned)c.width;
    const float idx_y = ((float)iy + 0.5f) / (float)(unsigned)c.height;
    const float px = 2.0f * (idx_x - c.principal_x), py = 2.0f * (idx_y - c.principal_y);
    const float dx = px * c.tan_half_fov_x, dy = py * c.tan_half_fov_y;
    const f3 d = mk3((dx * c.u[0] + dy * c.v[0]) + c.w[0], (dx * c.u[1] + dy * c.v[1]) + c.w[1],
                     (dx * c.u[2] + dy * c.v[2]) + c.w[2]);
    const float inv = 1.0f / sqrtf(dot3(d, d)); // vec_math.h:554-558 normalize
    return d * inv;
}

// Host-side helpers shared by the translation units.
int rgx_set_hip_error(hipError_t e);
#define RGX_HIP(call)                                      \
    do {                                                   \
        hipError_t e_ = (call);                            \
        if (e_ != hipSuccess) return rgx_set_hip_error(e_); \
    } while (0)
#define RGX_LAUNCH_CHECK() RGX_HIP(hipGetLastError())

// Makes the device that owns device pointer `p` current for the scope of an entry point and restores
// the caller's device afterwards (callers on another thread, e.g. the autograd engine's, may have a
// different current device).  A pointer the runtime does not know leaves the device as it is.
struct DeviceScope {
    int prev = -1;
    explicit DeviceScope(const void *p);
    ~DeviceScope();
    DeviceScope(const DeviceScope &) = delete;
    DeviceScope &operator=(const DeviceScope &) = delete;
};

// Event-timed spans (rgx_timing_* in the C ABI).  begin returns NULL when timing is off.
enum {
    RGX_T_BUILD = 0, RGX_T_SH_FWD, RGX_T_PACK, RGX_T_MARCH_FWD, RGX_T_MARCH_BWD, RGX_T_UNPERMUTE, RGX_T_SH_BWD,
    RGX_T_COUNT
};
void *rgx_span_begin(int id, hipStream_t s);
void rgx_span_end(void *span, hipStream_t s);
