// Ray-march kernels: forward compositing and the replaying backward pass.
// Replace the OptiX programs of optix_raycasting/cuda_train/forward/gaussians_aabb.cu
// (also cuda_test/, byte-identical) and cuda_train/backward/gaussians_aabb.cu, and
// their launchers (optix_raycasting/optix_utils.py:222-322, 363-500, 503-601).
//
// One lane per ray, one 64-lane wavefront per 8x8 pixel tile.  Each ray walks
// the skip-link BVH once per query (first-hit or collect); a slab's hit list
// lives in LDS (lane-interleaved, RGX_LDS_HITS entries per ray) and overflows
// into a global spill area up to max_prim_slice entries.
#include "rgx_device.h"

#define RGX_LDS_HITS 32

struct MarchParams {
    RgxCamera cam;
    RgxMarch m;
    const Node *nodes;
    const uint32_t *order;
    const WsHeader *hdr;
    const Prim *prims;
    int64_t n;
    float *ray_colors;       // fwd: output
    const float *fwd_colors; // bwd: forward output (C + T*bg)
    const float *dloss;      // bwd
    float *gbuf;             // bwd: (n,16) gradient block in Morton order
    int32_t *spill;
    int32_t spill_cap; // entries per ray beyond RGX_LDS_HITS
    RgxStats *stats;
    int32_t tiles_x, tiles_y;
};

struct HitList {
    int32_t *lds;   // &hits[0][lane]
    int32_t *spill; // this ray's spill row (may be null when spill_cap == 0)
    __device__ __forceinline__ void put(int j, int32_t v) const
    {
        if (j < RGX_LDS_HITS) lds[j * 64] = v;
        else spill[j - RGX_LDS_HITS] = v;
    }
    __device__ __forceinline__ int32_t get(int j) const { return j < RGX_LDS_HITS ? lds[j * 64] : spill[j - RGX_LDS_HITS]; }
};

struct Counters {
    unsigned hit_pairs = 0, slabs = 0, empty = 0, overflow = 0, rays_hit = 0;
    unsigned long long nodes = 0;
};

// First-hit query: optixTrace with SBT offset 0 (gaussians_aabb.cu:234-247, 300-313),
// __closesthit__ch / __miss__ms_ch (370-380).  Smallest reported t, or -1.
__device__ float first_hit(const MarchParams &P, f3 o, f3 dir, float tlo, float thi, Counters &cn)
{
    const RayBox rb = make_raybox(o, dir, thi);
    float best = -1.0f;
    int32_t node = P.n > 0 ? 0 : -1;
    const float4 *nodes4 = (const float4 *)P.nodes;
    // a sound tree is walked in < 2n steps and never leaves [0, 2n-1); both bounds are enforced
    // so that a corrupted workspace ends the query instead of hanging or faulting the GPU
    const uint32_t n_nodes = (uint32_t)(2 * P.n - 1);
    uint32_t steps = 0;
    while ((uint32_t)node < n_nodes && steps++ < n_nodes) {
        const float4 a = nodes4[2 * node], b = nodes4[2 * node + 1];
        cn.nodes++;
        int32_t next = __float_as_int(b.w);
        if (box_overlaps(rb, a, b, tlo, thi)) {
            const int32_t left = __float_as_int(a.w);
            if (left < 0) {
                const Prim *p = P.prims + (~left);
                float r1, r2, t;
                if (line_roots(p->pos4, p->inv_inter4, p->quat4, dir, r1, r2) && segment_hit(r1, r2, tlo, thi, t)) {
                    thi = t; // OptiX shrinks the interval to the closest accepted hit
                    best = t;
                }
            } else {
                next = left;
            }
        }
        node = next;
    }
    return best;
}

// Collect query: optixTrace with SBT offset 1 + __anyhit__ah (gaussians_aabb.cu:282-295,
// 349-367).  Appends every Gaussian hit in [tlo, thi] (sorted index) until `cap`.
__device__ int collect(const MarchParams &P, f3 o, f3 dir, float tlo, float thi, int cap, const HitList &hl, bool &overflow,
                       Counters &cn)
{
    const RayBox rb = make_raybox(o, dir, thi);
    int p0 = 0;
    overflow = false;
    int32_t node = P.n > 0 ? 0 : -1;
    const float4 *nodes4 = (const float4 *)P.nodes;
    const uint32_t n_nodes = (uint32_t)(2 * P.n - 1);
    uint32_t steps = 0;
    while ((uint32_t)node < n_nodes && steps++ < n_nodes) {
        const float4 a = nodes4[2 * node], b = nodes4[2 * node + 1];
        cn.nodes++;
        int32_t next = __float_as_int(b.w);
        if (box_overlaps(rb, a, b, tlo, thi)) {
            const int32_t left = __float_as_int(a.w);
            if (left < 0) {
                const Prim *p = P.prims + (~left);
                float r1, r2, t;
                if (line_roots(p->pos4, p->inv_inter4, p->quat4, dir, r1, r2) && segment_hit(r1, r2, tlo, thi, t)) {
                    if (p0 >= cap) { // optixTerminateRay at max_prim_slice (gaussians_aabb.cu:352-356)
                        overflow = true;
                        next = -1;
                    } else {
                        hl.put(p0++, ~left);
                    }
                }
            } else {
                next = left;
            }
        }
        node = next;
    }
    return p0;
}

// Per-hit constants of the sample recurrence (gaussians_aabb.cu:135-164).
struct HitSetup {
    float power, inc, inc_st, cut;
};
__device__ __forceinline__ HitSetup hit_setup(const Prim &p, f3 dir, f3 ray_dir_tmid, float dt)
{
    const float k = p.inv_inter4.w;
    const f3 inv_s = mk3(p.inv_inter4.x * k, p.inv_inter4.y * k, p.inv_inter4.z * k);
    f3 U, V, W;
    quat_to_cols(p.quat4, U, V, W);
    const f3 xhit = mk3(p.pos4.x, p.pos4.y, p.pos4.z) + ray_dir_tmid;
    const f3 Mx0 = apply_sinv_rt(xhit, U, V, W, inv_s);
    const f3 Md = apply_sinv_rt(dir, U, V, W, inv_s);
    const float Md2 = dot3(Md, Md);
    const float Md_dt_2 = (dt * dt) * Md2;
    HitSetup h;
    h.power = dot3(Mx0, Mx0);
    h.inc = Md_dt_2 + 2.0f * dot3(Mx0, Md) * dt;
    h.inc_st = 2.0f * Md_dt_2;
    h.cut = k * k;
    return h;
}

__device__ __forceinline__ void tile_pixel(const MarchParams &P, int &px, int &py, bool &valid)
{
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD one contiguous
    // band of tiles so its L2 sees one region of the scene.
    const int ntiles = P.tiles_x * P.tiles_y;
    const int per = (gridDim.x + 7) >> 3;
    const int tile = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    const int lane = threadIdx.x;
    const int tx = tile % P.tiles_x, ty = tile / P.tiles_x;
    px = tx * 8 + (lane & 7);
    py = ty * 8 + (lane >> 3);
    valid = tile < ntiles && px < P.cam.width && py < P.cam.height;
}

__device__ __forceinline__ void flush_stats(RgxStats *st, const Counters &c)
{
    if (!st) return;
    unsigned long long v[6] = {c.hit_pairs, c.slabs, c.empty, c.overflow, c.rays_hit, c.nodes};
    for (int k = 0; k < 6; ++k) {
        unsigned long long x = v[k];
        for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
        v[k] = x;
    }
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&st->hit_pairs, v[0]); atomicAdd(&st->slabs, v[1]); atomicAdd(&st->empty_slabs, v[2]);
        atomicAdd(&st->overflow_rays, v[3]); atomicAdd(&st->rays_hit, v[4]); atomicAdd(&st->nodes_visited, v[5]);
    }
}

// ---------------------------------------------------------------------------
// Forward: __raygen__rg (gaussians_aabb.cu:205-340), accumulateChunk (112-180),
// colorBlendingT_chunked (182-203).
__global__ __launch_bounds__(64) void k_march_fwd(const MarchParams P)
{
    __shared__ int32_t hits[RGX_LDS_HITS][64];
    int px, py;
    bool valid;
    tile_pixel(P, px, py, valid);
    Counters cn;
    if (valid) {
        const int64_t ray = (int64_t)py * P.cam.width + px;
        const f3 o = mk3(P.cam.eye[0], P.cam.eye[1], P.cam.eye[2]);
        const f3 dir = compute_ray(P.cam, (unsigned)px, (unsigned)py);
        const HitList hl = {&hits[0][threadIdx.x], P.spill ? P.spill + ray * P.spill_cap : nullptr};
        const float bg = P.m.white_background ? 1.0f : 0.0f;
        float out_r = bg, out_g = bg, out_b = bg;
        // scene-bbox slab test (gaussians_aabb.cu:212-224)
        const f3 inv = mk3(1.0f / dir.x, 1.0f / dir.y, 1.0f / dir.z);
        const float *bmn = P.hdr->bb_min, *bmx = P.hdr->bb_max;
        const float t0x = (bmn[0] - o.x) * inv.x, t1x = (bmx[0] - o.x) * inv.x;
        const float t0y = (bmn[1] - o.y) * inv.y, t1y = (bmx[1] - o.y) * inv.y;
        const float t0z = (bmn[2] - o.z) * inv.z, t1z = (bmx[2] - o.z) * inv.z;
        float tenter = fmaxf(0.0f, fmaxf(fminf(t0x, t1x), fmaxf(fminf(t0y, t1y), fminf(t0z, t1z))));
        const float texit = fminf(fmaxf(t0x, t1x), fminf(fmaxf(t0y, t1y), fmaxf(t0z, t1z)));
        const float dt_base = P.m.dt_step;
        float dt = dt_base, slab_spacing = dt * RGX_BUFFER_SIZE;
        const float fh = first_hit(P, o, dir, tenter, texit, cn);
        if (fh != -1.0f) {
            cn.rays_hit++;
            tenter = fh;
            if (tenter < texit) {
                float T = 1.0f, Cr = 0.f, Cg = 0.f, Cb = 0.f;
                float tbuffer = tenter;
                while (tbuffer < texit && T > P.m.t_eps) {
                    if (!(tbuffer + slab_spacing > tbuffer)) break; // step below one ulp of t: no progress possible
                    if (P.m.dynamic_sampling) { // gaussians_aabb.cu:267-272
                        const float dt_dist = fmaxf(tbuffer / 1024.0f, dt_base);
                        const float coeff = rcbrtf(T);
                        dt = fminf(dt_dist * coeff, 4.0f * dt_base);
                        slab_spacing = dt * RGX_BUFFER_SIZE;
                    }
                    const float t_min_slab = fmaxf(tenter, tbuffer);
                    const float t_max_slab = fminf(texit, tbuffer + slab_spacing);
                    if (t_max_slab > tenter) {
                        bool ov;
                        const int p0 = collect(P, o, dir, t_min_slab, t_max_slab, P.m.max_prim_slice, hl, ov, cn);
                        if (ov) cn.overflow++;
                        if (p0 == 0) {
                            cn.empty++;
                            tbuffer += slab_spacing;
                            const float nt = first_hit(P, o, dir, tbuffer, texit, cn);
                            if (nt == -1.0f) break;
                            tbuffer = nt;
                            continue;
                        }
                        cn.slabs++;
                        cn.hit_pairs += p0;
                        for (int base = 0; base < RGX_BUFFER_SIZE && T > P.m.t_eps; base += RGX_CHUNK_SIZE) {
                            float sg[RGX_CHUNK_SIZE], cr[RGX_CHUNK_SIZE], cg[RGX_CHUNK_SIZE], cb[RGX_CHUNK_SIZE];
#pragma unroll
                            for (int i = 0; i < RGX_CHUNK_SIZE; ++i) sg[i] = cr[i] = cg[i] = cb[i] = 0.f;
                            const float t_mid = fmaf(dt, (float)base + 0.5f, tbuffer);
                            const f3 rdt = dir * t_mid;
                            for (int h = 0; h < p0; ++h) {
                                const Prim p = P.prims[hl.get(h)];
                                HitSetup hs = hit_setup(p, dir, rdt, dt);
#pragma unroll
                                for (int i = 0; i < RGX_CHUNK_SIZE; ++i) {
                                    const float gw = hs.power < hs.cut ? __expf(-0.5f * hs.power) : 0.0f;
                                    sg[i] = fmaf(p.rgba4.w, gw, sg[i]);
                                    cr[i] = fmaf(p.rgba4.x, gw, cr[i]);
                                    cg[i] = fmaf(p.rgba4.y, gw, cg[i]);
                                    cb[i] = fmaf(p.rgba4.z, gw, cb[i]);
                                    hs.power += hs.inc;
                                    hs.inc += hs.inc_st;
                                }
                            }
#pragma unroll
                            for (int i = 0; i < RGX_CHUNK_SIZE; ++i) { // gaussians_aabb.cu:195-201
                                const float x = sg[i] * dt;
                                const float w = __expf(-x);
                                const float s = dt * ((1.0f - w) / fmaxf(x, 1e-6f));
                                const float ts = T * s;
                                Cr = fmaf(ts, cr[i], Cr);
                                Cg = fmaf(ts, cg[i], Cg);
                                Cb = fmaf(ts, cb[i], Cb);
                                T *= w;
                            }
                        }
                    }
                    tbuffer += slab_spacing;
                }
                out_r = Cr + T * bg; out_g = Cg + T * bg; out_b = Cb + T * bg;
            }
        }
        P.ray_colors[3 * ray] = out_r;
        P.ray_colors[3 * ray + 1] = out_g;
        P.ray_colors[3 * ray + 2] = out_b;
    }
    flush_stats(P.stats, cn);
}

// ---------------------------------------------------------------------------
// Backward: __raygen__rg of cuda_train/backward/gaussians_aabb.cu:209-497.
//
// Per blended slab: (1) per-sample density s_k and e_k = g.c_k/s_k over the hit
// list (accumulateChunk_backw, 113-184); (2) the prefix loop (330-352) giving,
// per sample, T_k (transmittance before the sample) and D_k = g.(C_final - C
// accumulated before k); (3) per hit, the sum over its in-range samples
// (353-442).  Writing w = exp(-power/2), a_k = T_k (1 - exp(-s_k dt)) / s_k,
// X_k = (T_k e_k - D_k) dt + a_k (g.c_i - e_k), every accumulator of the
// reference's per-hit loop is a moment of y_k = X_k w_k over the slab:
//   ddensity      = sum y_k
//   drgb          = g * rho * sum w_k a_k
//   dscale, dpos, dR: sums of y_k times polynomials of degree <= 2 in k, because
//   the sample point x_k = x_c + u_k dt dir (u_k = k - 15.5) is affine in k.
// So the inner loop carries three moments (sum y, sum y u, sum y u^2) instead of
// nineteen running sums; the `power < k^2` mask follows the reference's 32-step
// recurrence exactly.
__global__ __launch_bounds__(64) void k_march_bwd(const MarchParams P)
{
    __shared__ int32_t hits[RGX_LDS_HITS][64];
    int px, py;
    bool valid;
    tile_pixel(P, px, py, valid);
    Counters cn;
    if (valid) {
        const int64_t ray = (int64_t)py * P.cam.width + px;
        const f3 o = mk3(P.cam.eye[0], P.cam.eye[1], P.cam.eye[2]);
        const f3 dir = compute_ray(P.cam, (unsigned)px, (unsigned)py);
        const HitList hl = {&hits[0][threadIdx.x], P.spill ? P.spill + ray * P.spill_cap : nullptr};
        // backward/gaussians_aabb.cu:222-228 divides by the direction
        const float *bmn = P.hdr->bb_min, *bmx = P.hdr->bb_max;
        const float t0x = (bmn[0] - o.x) / dir.x, t1x = (bmx[0] - o.x) / dir.x;
        const float t0y = (bmn[1] - o.y) / dir.y, t1y = (bmx[1] - o.y) / dir.y;
        const float t0z = (bmn[2] - o.z) / dir.z, t1z = (bmx[2] - o.z) / dir.z;
        float tenter = fmaxf(0.0f, fmaxf(fminf(t0x, t1x), fmaxf(fminf(t0y, t1y), fminf(t0z, t1z))));
        const float texit = fminf(fmaxf(t0x, t1x), fminf(fmaxf(t0y, t1y), fmaxf(t0z, t1z)));
        const float dt_base = P.m.dt_step;
        float dt = dt_base, slab_spacing = dt * RGX_BUFFER_SIZE;
        const float fh = first_hit(P, o, dir, tenter, texit, cn);
        if (fh != -1.0f && fh < texit) {
            tenter = fh;
            float tbuffer = tenter, T = 1.0f;
            const f3 g = mk3(P.dloss[3 * ray], P.dloss[3 * ray + 1], P.dloss[3 * ray + 2]);
            float D = dot3(g, mk3(P.fwd_colors[3 * ray], P.fwd_colors[3 * ray + 1], P.fwd_colors[3 * ray + 2]));
            while (tbuffer < texit && T > P.m.t_eps) {
                if (!(tbuffer + slab_spacing > tbuffer)) break; // step below one ulp of t: no progress possible
                if (P.m.dynamic_sampling) {
                    const float dt_dist = fmaxf(tbuffer / 1024.0f, dt_base);
                    const float coeff = rcbrtf(T);
                    dt = fminf(dt_dist * coeff, 4.0f * dt_base);
                    slab_spacing = dt * RGX_BUFFER_SIZE;
                }
                const float t_min_slab = tbuffer; // unclipped: backward/gaussians_aabb.cu:279-280
                const float t_max_slab = tbuffer + slab_spacing;
                if (t_max_slab > tenter) {
                    bool ov;
                    const int p0 = collect(P, o, dir, t_min_slab, t_max_slab, P.m.max_prim_slice, hl, ov, cn);
                    if (ov) cn.overflow++;
                    if (p0 == 0) {
                        tbuffer += slab_spacing;
                        const float nt = first_hit(P, o, dir, tbuffer, texit, cn);
                        if (nt == -1.0f) break;
                        tbuffer = nt;
                        continue;
                    }
                    cn.slabs++;
                    cn.hit_pairs += p0;
                    // (1) s_k and g.c~_k  -> PA, PB
                    float PA[RGX_BUFFER_SIZE], PB[RGX_BUFFER_SIZE];
#pragma unroll
                    for (int i = 0; i < RGX_BUFFER_SIZE; ++i) PA[i] = PB[i] = 0.f;
                    const f3 rdt0 = dir * fmaf(dt, 0.5f, tbuffer);
                    const f3 rdt1 = dir * fmaf(dt, 16.5f, tbuffer);
                    for (int h = 0; h < p0; ++h) {
                        const Prim p = P.prims[hl.get(h)];
                        const float ddc = dot3(g, mk3(p.rgba4.x, p.rgba4.y, p.rgba4.z));
                        HitSetup hs = hit_setup(p, dir, rdt0, dt);
#pragma unroll
                        for (int i = 0; i < RGX_CHUNK_SIZE; ++i) {
                            const float gw = hs.power < hs.cut ? __expf(-0.5f * hs.power) : 0.0f;
                            PA[i] = fmaf(p.rgba4.w, gw, PA[i]);
                            PB[i] = fmaf(ddc, gw, PB[i]);
                            hs.power += hs.inc;
                            hs.inc += hs.inc_st;
                        }
                        hs = hit_setup(p, dir, rdt1, dt);
#pragma unroll
                        for (int i = RGX_CHUNK_SIZE; i < RGX_BUFFER_SIZE; ++i) {
                            const float gw = hs.power < hs.cut ? __expf(-0.5f * hs.power) : 0.0f;
                            PA[i] = fmaf(p.rgba4.w, gw, PA[i]);
                            PB[i] = fmaf(ddc, gw, PB[i]);
                            hs.power += hs.inc;
                            hs.inc += hs.inc_st;
                        }
                    }
                    // (2) prefix: PA <- a_k, PB <- (T_k e_k - D_k) dt - a_k e_k   (so X_k = PB + PA * g.c_i)
                    float T_after = T, D_after = D;
                    // the prefix always covers all 32 samples (330-352)
                    float T_mid = T; // transmittance at the chunk boundary: gates the second chunk (398)
#pragma unroll
                    for (int i = 0; i < RGX_BUFFER_SIZE; ++i) {
                        if (i == RGX_CHUNK_SIZE) T_mid = T_after;
                        const float sd = PA[i];
                        const float inv_d = sd > 0.0f ? 1.0f / sd : 0.0f;
                        const float e = PB[i] * inv_d;
                        const float w = __expf(-sd * dt);
                        const float a = T_after * (1.0f - w) * inv_d;
                        PA[i] = a;
                        PB[i] = (T_after * e - D_after) * dt - a * e;
                        D_after -= T_after * (1.0f - w) * e;
                        T_after *= w;
                    }
                    const bool use_second = T_mid > P.m.t_eps;
                    // (3) per hit
                    const f3 xdir_c = dir * fmaf(dt, 16.0f, tbuffer); // slab centre: t_c = tbuffer + 16 dt
                    for (int h = 0; h < p0; ++h) {
                        const int32_t pid = hl.get(h);
                        const Prim p = P.prims[pid];
                        const float k = p.inv_inter4.w;
                        const f3 inv_s = mk3(p.inv_inter4.x * k, p.inv_inter4.y * k, p.inv_inter4.z * k);
                        const float cut = k * k;
                        f3 U, V, W;
                        quat_to_cols(p.quat4, U, V, W);
                        const float rho = p.rgba4.w;
                        const float dcg = dot3(mk3(p.rgba4.x, p.rgba4.y, p.rgba4.z), g) / rho;
                        // mask recurrence exactly as backward/gaussians_aabb.cu:375-396, 437-438
                        const f3 Us = U * inv_s.x, Vs = V * inv_s.y, Ws = W * inv_s.z;
                        const f3 M1 = mk3(Us.x, Vs.x, Ws.x), M2 = mk3(Us.y, Vs.y, Ws.y), M3 = mk3(Us.z, Vs.z, Ws.z);
                        const f3 prel = mk3(p.pos4.x, p.pos4.y, p.pos4.z);
                        const f3 x0 = prel + dir * (tbuffer + 0.5f * dt);
                        const f3 Mx0 = (M1 * x0.x + M2 * x0.y) + M3 * x0.z;
                        const f3 Md = (M1 * dir.x + M2 * dir.y) + M3 * dir.z;
                        const float Md2 = dot3(Md, Md);
                        const float Md_dt_2 = (dt * dt) * Md2;
                        float power = dot3(Mx0, Mx0);
                        float inc = Md_dt_2 + 2.0f * dot3(Mx0, Md) * dt;
                        const float inc_st = 2.0f * Md_dt_2;
                        float s0 = 0.f, s1 = 0.f, s2 = 0.f, gc = 0.f;
#pragma unroll
                        for (int i = 0; i < RGX_BUFFER_SIZE; ++i) {
                            const bool on = power < cut && (i < RGX_CHUNK_SIZE || use_second);
                            const float wd = on ? __expf(-0.5f * power) : 0.0f;
                            const float y = fmaf(PA[i], dcg, PB[i]) * wd;
                            const float u = (float)i - 15.5f;
                            s0 += y;
                            s1 = fmaf(y, u, s1);
                            s2 = fmaf(y, u * u, s2);
                            gc = fmaf(wd, PA[i], gc);
                            power += inc;
                            inc += inc_st;
                        }
                        // moments -> gradients.  x_k = xc + u_k dt dir, (Mx)_k = Mxc + u_k dt Md
                        const f3 xc = prel + xdir_c;
                        const f3 Mxc = (M1 * xc.x + M2 * xc.y) + M3 * xc.z;
                        const float m1 = s1 * dt, m2 = s2 * (dt * dt);
                        // sum y (Mx)
                        const f3 Vy = Mxc * s0 + Md * m1;
                        // sum y (Mx)_a^2
                        const f3 Sy = mk3(fmaf(Mxc.x * Mxc.x, s0, fmaf(2.0f * Mxc.x * Md.x, m1, Md.x * Md.x * m2)),
                                          fmaf(Mxc.y * Mxc.y, s0, fmaf(2.0f * Mxc.y * Md.y, m1, Md.y * Md.y * m2)),
                                          fmaf(Mxc.z * Mxc.z, s0, fmaf(2.0f * Mxc.z * Md.z, m1, Md.z * Md.z * m2)));
                        // Q_a = sum y x (Mx)_a  (a vector per row a)
                        const f3 Qx = (xc * (Mxc.x * s0) + (xc * Md.x + dir * Mxc.x) * m1) + dir * (Md.x * m2);
                        const f3 Qy = (xc * (Mxc.y * s0) + (xc * Md.y + dir * Mxc.y) * m1) + dir * (Md.y * m2);
                        const f3 Qz = (xc * (Mxc.z * s0) + (xc * Md.z + dir * Mxc.z) * m1) + dir * (Md.z * m2);
                        float out[14];
                        out[0] = s0;                                  // d density
                        const float gcol = gc * rho;
                        out[1] = g.x * gcol; out[2] = g.y * gcol; out[3] = g.z * gcol; // d rgb
                        out[4] = rho * dot3(M1, Vy); out[5] = rho * dot3(M2, Vy); out[6] = rho * dot3(M3, Vy); // d position
                        out[7] = rho * Sy.x * inv_s.x; out[8] = rho * Sy.y * inv_s.y; out[9] = rho * Sy.z * inv_s.z; // d scale
                        const f3 d1 = Qx * (-rho * inv_s.x), d2 = Qy * (-rho * inv_s.y), d3 = Qz * (-rho * inv_s.z); // d R columns
                        const float qx = p.quat4.x, qy = p.quat4.y, qz = p.quat4.z, qw = p.quat4.w;
                        // backward/gaussians_aabb.cu:469-481
                        out[10] = 2 * qw * d1.y - 2 * qz * d1.z - 2 * qw * d2.x + 2 * qy * d2.z + 2 * qz * d3.x - 2 * qy * d3.y;
                        out[11] = 2 * qz * d1.y + 2 * qw * d1.z + 2 * qz * d2.x - 4 * qy * d2.y + 2 * qx * d2.z + 2 * qw * d3.x -
                                  2 * qx * d3.y - 4 * qy * d3.z;
                        out[12] = -4 * qz * d1.x + 2 * qy * d1.y - 2 * qx * d1.z + 2 * qy * d2.x + 2 * qw * d2.z + 2 * qx * d3.x +
                                  2 * qw * d3.y - 4 * qz * d3.z;
                        out[13] = -4 * qw * d1.x + 2 * qx * d1.y + 2 * qy * d1.z - 2 * qx * d2.x - 4 * qw * d2.y + 2 * qz * d2.z +
                                  2 * qy * d3.x + 2 * qz * d3.y;
                        float *dst = P.gbuf + (int64_t)pid * 16;
#pragma unroll
                        for (int c = 0; c < 14; ++c) unsafeAtomicAdd(dst + c, out[c]);
                    }
                    D = D_after;
                    T = T_after;
                }
                tbuffer += slab_spacing;
            }
        }
    }
    flush_stats(P.stats, cn);
}

// gbuf (Morton order, 16 floats per Gaussian) -> the five gradient tensors in input order
__global__ __launch_bounds__(256) void k_unpermute_grads(const float4 *__restrict__ gbuf, const uint32_t *__restrict__ order,
                                                         int64_t n, float *__restrict__ ddens, float *__restrict__ drgb,
                                                         float *__restrict__ dpos, float *__restrict__ dscale,
                                                         float *__restrict__ dquat)
{
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const int64_t i = order[j];
    const float4 a = gbuf[4 * j], b = gbuf[4 * j + 1], c = gbuf[4 * j + 2], d = gbuf[4 * j + 3];
    ddens[i] = a.x;
    drgb[3 * i] = a.y; drgb[3 * i + 1] = a.z; drgb[3 * i + 2] = a.w;
    dpos[3 * i] = b.x; dpos[3 * i + 1] = b.y; dpos[3 * i + 2] = b.z;
    dscale[3 * i] = b.w; dscale[3 * i + 1] = c.x; dscale[3 * i + 2] = c.y;
    dquat[4 * i] = c.z; dquat[4 * i + 1] = c.w; dquat[4 * i + 2] = d.x; dquat[4 * i + 3] = d.y;
}

__global__ __launch_bounds__(256) void k_zero4(float4 *p, int64_t n4)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n4) p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// ---------------------------------------------------------------------------
// Test hooks: the two queries on caller-supplied segments.
__global__ __launch_bounds__(64) void k_first_hit(const MarchParams P, f3 o, int64_t n, const float *__restrict__ dirs,
                                                  const float *__restrict__ tlo, const float *__restrict__ thi,
                                                  float *__restrict__ out)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= n) return;
    Counters cn;
    out[r] = first_hit(P, o, mk3(dirs[3 * r], dirs[3 * r + 1], dirs[3 * r + 2]), tlo[r], thi[r], cn);
}

__global__ __launch_bounds__(64) void k_trace_segments(const MarchParams P, f3 o, int64_t n, const float *__restrict__ dirs,
                                                       const float *__restrict__ tlo, const float *__restrict__ thi, int cap,
                                                       int32_t *__restrict__ counts, int32_t *__restrict__ ids)
{
    __shared__ int32_t hits[RGX_LDS_HITS][64];
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= n) return;
    Counters cn;
    // the id row doubles as the spill area; LDS entries are copied out afterwards
    const HitList hl = {&hits[0][threadIdx.x], ids + r * cap + RGX_LDS_HITS};
    bool ov;
    const int p0 = collect(P, o, mk3(dirs[3 * r], dirs[3 * r + 1], dirs[3 * r + 2]), tlo[r], thi[r], cap, hl, ov, cn);
    for (int j = 0; j < p0; ++j) ids[r * cap + j] = (int32_t)P.order[hl.get(j)];
    counts[r] = ov ? -p0 : p0;
}

// ---------------------------------------------------------------------------
static inline dim3 grid_for(int64_t n, int block) { return dim3((unsigned)((n + block - 1) / block)); }

struct MarchWs {
    size_t gbuf, spill, total;
    int32_t spill_cap;
};
static inline MarchWs march_ws_layout(int64_t n, int64_t n_rays, int32_t max_prim_slice)
{
    MarchWs L;
    L.spill_cap = max_prim_slice > RGX_LDS_HITS ? max_prim_slice - RGX_LDS_HITS : 0;
    size_t off = 0;
    L.gbuf = off;  off = rgx_align_up(off + (size_t)(n > 0 ? n : 1) * 16 * sizeof(float), 256);
    L.spill = off; off = rgx_align_up(off + (size_t)(n_rays > 0 ? n_rays : 1) * (size_t)L.spill_cap * sizeof(int32_t), 256);
    L.total = off;
    return L;
}

extern "C" int rgx_march_workspace_bytes(int64_t n, int64_t n_rays, int32_t max_prim_slice, size_t *bytes)
{
    if (n < 0 || n_rays < 0 || max_prim_slice < 0 || !bytes) return RGX_EINVAL;
    *bytes = march_ws_layout(n, n_rays, max_prim_slice).total;
    return RGX_OK;
}

static int fill_params(MarchParams &P, const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims,
                       int64_t n, void *march_ws, size_t march_ws_bytes, RgxStats *stats)
{
    if (!ws || !cam || !march || n < 0 || (n > 0 && !prims) || cam->width <= 0 || cam->height <= 0 ||
        march->max_prim_slice < 0 || !(march->dt_step > 0.0f) || ((uintptr_t)prims & 15u))
        return RGX_EINVAL;
    const int64_t n_rays = (int64_t)cam->width * cam->height;
    const MarchWs M = march_ws_layout(n, n_rays, march->max_prim_slice);
    if (!march_ws || march_ws_bytes < M.total || ((uintptr_t)march_ws & 255u)) return RGX_EWORKSPACE;
    const WsLayout L = rgx_ws_layout(n);
    const char *w = (const char *)ws;
    P.cam = *cam;
    P.m = *march;
    P.nodes = (const Node *)(w + L.nodes);
    P.order = (const uint32_t *)(w + L.vals0);
    P.hdr = (const WsHeader *)(w + L.header);
    P.prims = (const Prim *)prims;
    P.n = n;
    P.ray_colors = nullptr;
    P.fwd_colors = nullptr;
    P.dloss = nullptr;
    P.gbuf = (float *)((char *)march_ws + M.gbuf);
    P.spill = M.spill_cap ? (int32_t *)((char *)march_ws + M.spill) : nullptr;
    P.spill_cap = M.spill_cap;
    P.stats = stats;
    P.tiles_x = (cam->width + 7) / 8;
    P.tiles_y = (cam->height + 7) / 8;
    return RGX_OK;
}

static inline dim3 march_grid(const MarchParams &P)
{
    const int ntiles = P.tiles_x * P.tiles_y;
    return dim3((unsigned)((ntiles + 7) / 8 * 8));
}

extern "C" int rgx_march_forward(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims, int64_t n,
                                 float *ray_colors, void *march_ws, size_t march_ws_bytes, RgxStats *stats, void *stream)
{
    MarchParams P;
    const int rc = fill_params(P, ws, cam, march, prims, n, march_ws, march_ws_bytes, stats);
    if (rc) return rc;
    if (!ray_colors) return RGX_EINVAL;
    P.ray_colors = ray_colors;
    void *span = rgx_span_begin(RGX_T_MARCH_FWD, (hipStream_t)stream);
    hipLaunchKernelGGL(k_march_fwd, march_grid(P), dim3(64), 0, (hipStream_t)stream, P);
    rgx_span_end(span, (hipStream_t)stream);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

extern "C" int rgx_march_backward(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims, int64_t n,
                                  const float *ray_colors, const float *dloss, float *ddens, float *drgb, float *dpos,
                                  float *dscale, float *dquat, void *march_ws, size_t march_ws_bytes, RgxStats *stats,
                                  void *stream)
{
    MarchParams P;
    const int rc = fill_params(P, ws, cam, march, prims, n, march_ws, march_ws_bytes, stats);
    if (rc) return rc;
    if (!ray_colors || !dloss || (n > 0 && (!ddens || !drgb || !dpos || !dscale || !dquat))) return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    P.fwd_colors = ray_colors;
    P.dloss = dloss;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(k_zero4, grid_for(4 * n, 256), dim3(256), 0, s, (float4 *)P.gbuf, 4 * n);
    void *span = rgx_span_begin(RGX_T_MARCH_BWD, s);
    hipLaunchKernelGGL(k_march_bwd, march_grid(P), dim3(64), 0, s, P);
    rgx_span_end(span, s);
    span = rgx_span_begin(RGX_T_UNPERMUTE, s);
    hipLaunchKernelGGL(k_unpermute_grads, grid_for(n, 256), dim3(256), 0, s, (const float4 *)P.gbuf, P.order, n, ddens, drgb,
                       dpos, dscale, dquat);
    rgx_span_end(span, s);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

static int hook_params(MarchParams &P, const void *ws, const float *prims, int64_t n_prims)
{
    if (!ws || n_prims < 0 || (n_prims > 0 && !prims)) return RGX_EINVAL;
    const WsLayout L = rgx_ws_layout(n_prims);
    const char *w = (const char *)ws;
    P = MarchParams{};
    P.nodes = (const Node *)(w + L.nodes);
    P.order = (const uint32_t *)(w + L.vals0);
    P.hdr = (const WsHeader *)(w + L.header);
    P.prims = (const Prim *)prims;
    P.n = n_prims;
    return RGX_OK;
}

extern "C" int rgx_first_hit(const void *ws, const float *prims, int64_t n_prims, const float *eye, int64_t n,
                             const float *dirs, const float *tlo, const float *thi, float *out_t, void *stream)
{
    MarchParams P;
    const int rc = hook_params(P, ws, prims, n_prims);
    if (rc) return rc;
    if (!eye || n < 0 || (n > 0 && (!dirs || !tlo || !thi || !out_t))) return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    hipLaunchKernelGGL(k_first_hit, grid_for(n, 64), dim3(64), 0, (hipStream_t)stream, P, f3{eye[0], eye[1], eye[2]}, n, dirs,
                       tlo, thi, out_t);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

extern "C" int rgx_trace_segments(const void *ws, const float *prims, int64_t n_prims, const float *eye, int64_t n,
                                  const float *dirs, const float *tlo, const float *thi, int32_t cap, int32_t *counts,
                                  int32_t *ids, void *stream)
{
    MarchParams P;
    const int rc = hook_params(P, ws, prims, n_prims);
    if (rc) return rc;
    if (!eye || n < 0 || cap <= 0 || (n > 0 && (!dirs || !tlo || !thi || !counts || !ids))) return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    hipLaunchKernelGGL(k_trace_segments, grid_for(n, 64), dim3(64), 0, (hipStream_t)stream, P, f3{eye[0], eye[1], eye[2]}, n,
                       dirs, tlo, thi, (int)cap, counts, ids);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}
