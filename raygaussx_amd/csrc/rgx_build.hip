// LBVH construction on the GPU: k-sigma AABBs + scene bbox, 63-bit Morton
// codes, LDS-staged LSD radix sort, Karras radix tree, bottom-up refit, skip
// links.  Replaces the OptiX GAS build (optix_raycasting/optix_utils.py:139-142)
// and the AABB pass feeding it (optix_utils.py:36-109).  Also hosts the 30-bit
// Morton ordering of the point cloud (utils/reordering_utils.py:55-104).
#include "rgx_device.h"
#include <float.h>

#include <algorithm>

// ---------------------------------------------------------------------------
// order-preserving float <-> int encoding for atomicMin/atomicMax
__device__ __forceinline__ int32_t enc_f(float f)
{
    int32_t i = __float_as_int(f);
    return i >= 0 ? i : i ^ 0x7fffffff;
}
__device__ __forceinline__ float dec_f(int32_t i) { return __int_as_float(i >= 0 ? i : i ^ 0x7fffffff); }

__global__ void k_init_header(WsHeader *h, int64_t n)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        for (int a = 0; a < 3; ++a) {
            h->bb_min_enc[a] = enc_f(INFINITY);
            h->bb_max_enc[a] = enc_f(-INFINITY);
            h->bb_min[a] = INFINITY;
            h->bb_max[a] = -INFINITY;
        }
        h->n = n;
        h->root = 0;
        h->built = 0;
        h->refit_ok = 0;
    }
}

// First kernel of a refit.  A refit walks the parent / child / order arrays the last build left in the
// workspace, so it may only run over a finished tree of exactly n boxes: anything else (a workspace never
// built, built for another n, or left unfinished) would send the refit kernels to indices that mean nothing.
// The check runs on the device, in stream order after whatever build precedes it; when it fails the header is
// left not built, `refit_ok` stays 0 and every later kernel of the refit returns at once (`gate`).
__global__ void k_refit_begin(WsHeader *h, int64_t n)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        const bool ok = h->built == 1 && h->n == n && h->root == 0;
        for (int a = 0; a < 3; ++a) {
            h->bb_min_enc[a] = enc_f(INFINITY);
            h->bb_max_enc[a] = enc_f(-INFINITY);
            if (ok) {
                h->bb_min[a] = INFINITY;
                h->bb_max[a] = -INFINITY;
            }
        }
        h->built = 0;
        h->refit_ok = ok ? 1 : 0;
    }
}
__device__ __forceinline__ bool gate_closed(const int32_t *gate) { return gate != nullptr && *gate == 0; }

__device__ __forceinline__ float wave_min(float v)
{
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// k-sigma AABB of a rotated ellipsoid (optix_utils.py:49-77), canonical arithmetic.
__global__ __launch_bounds__(256) void k_aabb(const float *__restrict__ pos, const float *__restrict__ scale,
                                              const float *__restrict__ quat, const float *__restrict__ dens,
                                              int64_t n, float thr, float *__restrict__ boxes, int32_t *mn_enc, int32_t *mx_enc)
{
    // (a block takes several rounds of 256 Gaussians: every block ends with six atomics on the same six words,
    // and one per 256 Gaussians made those the kernel's time)
    float b[6] = {INFINITY, INFINITY, INFINITY, -INFINITY, -INFINITY, -INFINITY};
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float t = dens[i] / thr;
        float d = canon_logf(t * t);
        if (!(d > 0.0f)) d = 0.0f;
        d = sqrtf(d);
        float W = quat[4 * i], X = quat[4 * i + 1], Y = quat[4 * i + 2], Z = quat[4 * i + 3];
        const float nn = ((W * W + X * X) + Y * Y) + Z * Z;
        const float invn = 1.0f / sqrtf(nn + 1e-20f);
        W *= invn; X *= invn; Y *= invn; Z *= invn;
        const float L1x = 1.f - 2.f * (Y * Y + Z * Z), L1y = 2.f * (X * Y - W * Z), L1z = 2.f * (X * Z + W * Y);
        const float L2x = 2.f * (X * Y + W * Z), L2y = 1.f - 2.f * (X * X + Z * Z), L2z = 2.f * (Y * Z - W * X);
        const float L3x = 2.f * (X * Z - W * Y), L3y = 2.f * (Y * Z + W * X), L3z = 1.f - 2.f * (X * X + Y * Y);
        const float s0 = scale[3 * i], s1 = scale[3 * i + 1], s2 = scale[3 * i + 2];
        const float hx = d * sqrtf(((s0 * L1x) * (s0 * L1x) + (s1 * L1y) * (s1 * L1y)) + (s2 * L1z) * (s2 * L1z));
        const float hy = d * sqrtf(((s0 * L2x) * (s0 * L2x) + (s1 * L2y) * (s1 * L2y)) + (s2 * L2z) * (s2 * L2z));
        const float hz = d * sqrtf(((s0 * L3x) * (s0 * L3x) + (s1 * L3y) * (s1 * L3y)) + (s2 * L3z) * (s2 * L3z));
        const float c0 = pos[3 * i], c1 = pos[3 * i + 1], c2 = pos[3 * i + 2];
        const float e[6] = {c0 - hx, c1 - hy, c2 - hz, c0 + hx, c1 + hy, c2 + hz};
        if (boxes)
            for (int a = 0; a < 6; ++a) boxes[6 * i + a] = e[a];
        for (int a = 0; a < 3; ++a) {
            b[a] = fminf(b[a], e[a]);
            b[a + 3] = fmaxf(b[a + 3], e[a + 3]);
        }
    }
    __shared__ float red[4][6];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int a = 0; a < 3; ++a) {
        const float mn = wave_min(b[a]), mx = wave_max(b[a + 3]);
        if (lane == 0) { red[wave][a] = mn; red[wave][a + 3] = mx; }
    }
    __syncthreads();
    if (threadIdx.x < 3 && mn_enc) {
        const int a = threadIdx.x;
        const float mn = fminf(fminf(red[0][a], red[1][a]), fminf(red[2][a], red[3][a]));
        const float mx = fmaxf(fmaxf(red[0][a + 3], red[1][a + 3]), fmaxf(red[2][a + 3], red[3][a + 3]));
        atomicMin(&mn_enc[a], enc_f(mn));
        atomicMax(&mx_enc[a], enc_f(mx));
    }
}

// stand-alone reductions keep their encoded running min/max in the output buffers themselves
__global__ void k_init_enc(int32_t *mn, int32_t *mx)
{
    if (threadIdx.x < 3) {
        mn[threadIdx.x] = enc_f(INFINITY);
        mx[threadIdx.x] = enc_f(-INFINITY);
    }
}
__global__ void k_decode_enc(int32_t *mn, int32_t *mx)
{
    if (threadIdx.x < 3) {
        ((float *)mn)[threadIdx.x] = dec_f(mn[threadIdx.x]);
        ((float *)mx)[threadIdx.x] = dec_f(mx[threadIdx.x]);
    }
}

__global__ void k_finish_bbox(WsHeader *h, float *bb_min, float *bb_max, const int32_t *gate = nullptr)
{
    const int a = threadIdx.x;
    if (gate_closed(gate)) return;
    if (a < 3) {
        const float mn = dec_f(h->bb_min_enc[a]), mx = dec_f(h->bb_max_enc[a]);
        h->bb_min[a] = mn;
        h->bb_max[a] = mx;
        if (bb_min) bb_min[a] = mn;
        if (bb_max) bb_max[a] = mx;
    }
}

// ---------------------------------------------------------------------------
__device__ __forceinline__ uint64_t expand21(uint64_t x)
{
    x &= 0x1fffffull;
    x = (x | x << 32) & 0x1f00000000ffffull;
    x = (x | x << 16) & 0x1f0000ff0000ffull;
    x = (x | x << 8) & 0x100f00f00f00f00full;
    x = (x | x << 4) & 0x10c30c30c30c30c3ull;
    x = (x | x << 2) & 0x1249249249249249ull;
    return x;
}

// 21 bits per axis of the box centre, relative to the scene bbox
__global__ __launch_bounds__(256) void k_morton63(const float *__restrict__ boxes, int64_t n, const WsHeader *hdr,
                                                  uint64_t *__restrict__ keys, uint32_t *__restrict__ vals)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t q[3];
    for (int a = 0; a < 3; ++a) {
        const float lo = hdr->bb_min[a], ext = hdr->bb_max[a] - lo;
        const float c = 0.5f * boxes[6 * i + a] + 0.5f * boxes[6 * i + 3 + a];
        float u = ext > 0.f ? (c - lo) / ext : 0.f;
        u = fminf(fmaxf(u, 0.f), 1.f);
        const float s = u * 2097152.0f;
        q[a] = s >= 2097151.0f ? 2097151ull : (uint64_t)s;
    }
    keys[i] = (expand21(q[0]) << 2) | (expand21(q[1]) << 1) | expand21(q[2]);
    vals[i] = (uint32_t)i;
}

// ---------------------------------------------------------------------------
// LSD radix sort, 8 bits per pass, keys u64 + values u32, stable.  Per pass:
// per-tile digit histogram -> exclusive scan over (digit, tile) -> scatter.
// The scatter keeps its per-wave digit cursors in LDS and ranks the 64 keys a
// wave handles at a time with ballot matching, so equal digits leave in input
// order.
template <typename K>
__global__ __launch_bounds__(RGX_RS_THREADS) void k_rs_hist(const K *__restrict__ keys, int64_t n, int shift,
                                                            uint32_t *__restrict__ hist, int nblocks)
{
    __shared__ uint32_t h[256];
    h[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * RGX_RS_TILE;
    for (int r = 0; r < RGX_RS_ITEMS; ++r) {
        const int64_t i = base + r * RGX_RS_THREADS + threadIdx.x;
        if (i < n) atomicAdd(&h[(uint32_t)(keys[i] >> shift) & 255u], 1u);
    }
    __syncthreads();
    hist[(size_t)threadIdx.x * nblocks + blockIdx.x] = h[threadIdx.x];
}

// Exclusive scan of the (digit, tile) counts in two levels: block d scans its digit's row of tile
// counts in place and leaves the row total; every block of the scatter scans the 256 totals into
// digit bases for itself (a launch of one block for that cost more than 500 blocks doing it again).
__global__ __launch_bounds__(256) void k_rs_scan_rows(uint32_t *__restrict__ hist, int nblocks, uint32_t *__restrict__ totals)
{
    __shared__ uint32_t part[256];
    uint32_t *row = hist + (size_t)blockIdx.x * nblocks;
    uint32_t carry = 0;
    for (int base = 0; base < nblocks; base += 256) {
        const int i = base + threadIdx.x;
        const uint32_t v = i < nblocks ? row[i] : 0u;
        part[threadIdx.x] = v;
        __syncthreads();
        for (int o = 1; o < 256; o <<= 1) { // Hillis-Steele inclusive scan
            const uint32_t t = threadIdx.x >= o ? part[threadIdx.x - o] : 0u;
            __syncthreads();
            part[threadIdx.x] += t;
            __syncthreads();
        }
        if (i < nblocks) row[i] = carry + part[threadIdx.x] - v;
        carry += part[255];
        __syncthreads();
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

template <typename K>
__global__ __launch_bounds__(RGX_RS_THREADS) void k_rs_scatter(const K *__restrict__ kin, const uint32_t *__restrict__ vin,
                                                               K *__restrict__ kout, uint32_t *__restrict__ vout, int64_t n,
                                                               int shift, const uint32_t *__restrict__ hist, int nblocks,
                                                               const uint32_t *__restrict__ totals)
{
    static_assert(RGX_RS_THREADS == 256, "one thread per digit");
    __shared__ uint32_t cnt[4][256];
    __shared__ uint32_t wave_total[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int w = 0; w < 4; ++w) cnt[w][threadIdx.x] = 0;
    // digit_base: exclusive scan of the digits' totals, thread d for digit d
    const uint32_t total = totals[threadIdx.x];
    uint32_t incl = total;
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t t = __shfl_up(incl, o);
        if (lane >= o) incl += t;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    uint32_t digit_base = incl - total;
    for (int w = 0; w < wave; ++w) digit_base += wave_total[w];
    // wave w owns the contiguous 512 keys [base + 512 w, +512), 64 per round
    const int64_t base = (int64_t)blockIdx.x * RGX_RS_TILE + (int64_t)wave * (64 * RGX_RS_ITEMS);
    K key[RGX_RS_ITEMS];
    uint32_t val[RGX_RS_ITEMS];
    for (int r = 0; r < RGX_RS_ITEMS; ++r) {
        const int64_t i = base + r * 64 + lane;
        key[r] = 0;
        val[r] = 0;
        if (i < n) {
            key[r] = kin[i];
            val[r] = vin[i];
            atomicAdd(&cnt[wave][(uint32_t)(key[r] >> shift) & 255u], 1u);
        }
    }
    __syncthreads();
    // The tile's keys are put in digit order in LDS first and leave from there: keys of one digit are neighbours
    // in the tile's order as they are in the output, so thread after thread writes consecutive words instead of
    // 64 lanes writing to as many streams.  local: where a (wave, digit) run starts in the tile's order;
    // delta[d]: output position minus position in the tile's order, for digit d.
    __shared__ uint32_t delta[256];
    __shared__ K lkey[RGX_RS_TILE];
    __shared__ uint32_t lval[RGX_RS_TILE];
    {
        const int d = threadIdx.x;
        uint32_t c[4], tile_count = 0;
        for (int w = 0; w < 4; ++w) tile_count += c[w] = cnt[w][d];
        uint32_t upto = tile_count; // inclusive scan of the tile's digit counts
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t t = __shfl_up(upto, o);
            if (lane >= o) upto += t;
        }
        __syncthreads(); // (wave_total's first use is over)
        if (lane == 63) wave_total[wave] = upto;
        __syncthreads();
        uint32_t local = upto - tile_count;
        for (int w = 0; w < wave; ++w) local += wave_total[w];
        delta[d] = digit_base + hist[(size_t)d * nblocks + blockIdx.x] - local;
        for (int w = 0; w < 4; ++w) {
            cnt[w][d] = local;
            local += c[w];
        }
    }
    __syncthreads();
    volatile uint32_t *cur = cnt[wave];
    for (int r = 0; r < RGX_RS_ITEMS; ++r) {
        const int64_t i = base + r * 64 + lane;
        const bool valid = i < n;
        const uint32_t d = (uint32_t)(key[r] >> shift) & 255u;
        uint64_t same = __ballot(valid);
        for (int b = 0; b < 8; ++b) {
            const bool bit = (d >> b) & 1u;
            const uint64_t bal = __ballot(bit);
            same &= bit ? bal : ~bal;
        }
        if (valid) {
            const uint32_t rank = __popcll(same & ((1ull << lane) - 1ull));
            const uint32_t off = cur[d];
            lkey[off + rank] = key[r];
            lval[off + rank] = val[r];
        }
        __builtin_amdgcn_wave_barrier();
        if (valid && (same & ((1ull << lane) - 1ull)) == 0) cur[d] += __popcll(same);
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    const int64_t tile_base = (int64_t)blockIdx.x * RGX_RS_TILE;
    const int tile_n = (int)(n - tile_base < RGX_RS_TILE ? n - tile_base : RGX_RS_TILE);
    for (int p = threadIdx.x; p < tile_n; p += RGX_RS_THREADS) {
        const K k = lkey[p];
        const uint32_t out = (uint32_t)p + delta[(uint32_t)(k >> shift) & 255u];
        kout[out] = k;
        vout[out] = lval[p];
    }
}

template <typename K>
static int radix_sort(K *k0, uint32_t *v0, K *k1, uint32_t *v1, int64_t n, int bits, uint32_t *hist, hipStream_t s)
{
    const int nblocks = (int)((n + RGX_RS_TILE - 1) / RGX_RS_TILE);
    K *ki = k0, *ko = k1;
    uint32_t *vi = v0, *vo = v1;
    for (int shift = 0; shift < bits; shift += 8) {
        hipLaunchKernelGGL(k_rs_hist<K>, dim3(nblocks), dim3(RGX_RS_THREADS), 0, s, ki, n, shift, hist, nblocks);
        uint32_t *totals = hist + (size_t)256 * nblocks;
        hipLaunchKernelGGL(k_rs_scan_rows, dim3(256), dim3(256), 0, s, hist, nblocks, totals);
        hipLaunchKernelGGL(k_rs_scatter<K>, dim3(nblocks), dim3(RGX_RS_THREADS), 0, s, ki, vi, ko, vo, n, shift, hist, nblocks,
                           totals);
        K *tk = ki; ki = ko; ko = tk;
        uint32_t *tv = vi; vi = vo; vo = tv;
    }
    RGX_LAUNCH_CHECK();
    return ((bits + 7) / 8) & 1; // 1 when the result ended in (k1, v1)
}

// ---------------------------------------------------------------------------
// Leaves, radix tree (Karras 2012), refit, skip links.
__global__ __launch_bounds__(256) void k_leaves(const float *__restrict__ boxes, const uint32_t *__restrict__ order, int64_t n,
                                                Node *__restrict__ nodes, int32_t *__restrict__ parent, int32_t *__restrict__ flags,
                                                uint32_t *__restrict__ place, const int32_t *gate = nullptr)
{
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n || gate_closed(gate)) return;
    const int64_t in = order[j];
    place[in] = (uint32_t)j; // the inverse permutation, for the kernels that go through the Gaussians in input order
    const float *b = boxes + 6 * in;
    Node nd;
    nd.lo[0] = b[0]; nd.lo[1] = b[1]; nd.lo[2] = b[2];
    nd.hi[0] = b[3]; nd.hi[1] = b[4]; nd.hi[2] = b[5];
    nd.left = ~(int32_t)j;
    nd.skip = -1;
    nodes[n - 1 + j] = nd;
    flags[j] = 0;
    if (j == 0) parent[0] = -1;
}

__device__ __forceinline__ int delta(const uint64_t *keys, int64_t n, int64_t i, int64_t j)
{
    if (j < 0 || j >= n) return -1;
    const uint64_t a = keys[i], b = keys[j];
    if (a != b) return __clzll((long long)(a ^ b));
    return 64 + __clz((int)((uint32_t)i ^ (uint32_t)j));
}

// other_end[i]: internal node i covers the sorted leaves between i and other_end[i]
__global__ __launch_bounds__(256) void k_karras(const uint64_t *__restrict__ keys, int64_t n, Node *__restrict__ nodes,
                                                int32_t *__restrict__ parent, int32_t *__restrict__ right,
                                                int32_t *__restrict__ other_end)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n - 1) return;
    const int d = delta(keys, n, i, i + 1) - delta(keys, n, i, i - 1) >= 0 ? 1 : -1;
    const int dmin = delta(keys, n, i, i - d);
    int64_t lmax = 2;
    while (delta(keys, n, i, i + lmax * d) > dmin) lmax <<= 1;
    int64_t l = 0;
    for (int64_t t = lmax >> 1; t >= 1; t >>= 1)
        if (delta(keys, n, i, i + (l + t) * d) > dmin) l += t;
    const int64_t j = i + l * d;
    const int dnode = delta(keys, n, i, j);
    int64_t s = 0, t = l;
    do {
        t = (t + 1) >> 1;
        if (delta(keys, n, i, i + (s + t) * d) > dnode) s += t;
    } while (t > 1);
    const int64_t gamma = i + s * d + (d < 0 ? -1 : 0);
    const int64_t lo = i < j ? i : j, hi = i < j ? j : i;
    const int32_t lc = (int32_t)(lo == gamma ? n - 1 + gamma : gamma);
    const int32_t rc = (int32_t)(hi == gamma + 1 ? n - 1 + gamma + 1 : gamma + 1);
    nodes[i].left = lc;
    right[i] = rc;
    parent[lc] = (int32_t)i;
    parent[rc] = (int32_t)i;
    other_end[i] = (int32_t)j;
}

// Bottom-up refit: every leaf walks towards the root; the second thread to reach a node
// (counted with an atomic) merges the two child boxes and goes on.  A workgroup owns 256
// consecutive leaves of the sorted order; the nodes whose leaves all lie among them (internal node
// i covers the leaves between i and other_end[i], so its index is one of them) are met in LDS:
// counters, and the box of whichever child arrived first.  Only the few subtree roots a workgroup
// ends up with go on through memory, where box words travel between threads through agent-scope
// atomic stores and loads (write-through to, and read from, the memory all XCDs share).  The thread
// that arrives second at a node may run in another workgroup on another XCD, so the first arriver's
// box stores -- also those it made in the LDS phase -- must have completed before its count becomes
// visible: it waits for them (s_waitcnt vmcnt(0)) before the counter's atomic.  That is the part of
// an agent-scope release these stores need; the full fence also writes the whole L2 back, which
// nothing here depends on (no plain store of this kernel is read by another workgroup) and which made
// the build 2.6 times slower (0.64 -> 1.69 ms at 1 M Gaussians).  The second arriver's loads are
// issued after its atomic has returned (its branch depends on the result).
__device__ __forceinline__ void st_agent(float *p, float v)
{
    __hip_atomic_store((int *)p, __float_as_int(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_agent(const float *p)
{
    return __int_as_float(__hip_atomic_load((const int *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

__global__ __launch_bounds__(256) void k_refit(int64_t n, Node *nodes, const int32_t *__restrict__ parent,
                                               const int32_t *__restrict__ right, const int32_t *__restrict__ other_end,
                                               int32_t *flags, const int32_t *gate = nullptr)
{
    __shared__ float s_box[2][6][256]; // [which child][lo xyz, hi xyz][node - first leaf of the workgroup]
    __shared__ int s_arrived[256];
    if (gate_closed(gate)) return; // the whole grid
    const int64_t b0 = (int64_t)blockIdx.x * 256, j = b0 + threadIdx.x;
    s_arrived[threadIdx.x] = 0;
    __syncthreads();
    if (j >= n) return;
    const int64_t b1 = b0 + 255 < n - 1 ? b0 + 255 : n - 1;
    int32_t child = (int32_t)(n - 1 + j);
    float lo[3], hi[3];
    for (int c = 0; c < 3; ++c) {
        lo[c] = nodes[child].lo[c];
        hi[c] = nodes[child].hi[c];
    }
    int32_t node = parent[child];
    // nodes inside the workgroup's leaves: through LDS
    while (node >= 0) {
        const int32_t o = other_end[node];
        if ((node < o ? node : o) < b0 || (node < o ? o : node) > b1) break;
        const int slot = (int)(node - b0), side = nodes[node].left == child ? 0 : 1;
        for (int c = 0; c < 3; ++c) {
            s_box[side][c][slot] = lo[c];
            s_box[side][3 + c][slot] = hi[c];
        }
        __threadfence_block();
        if (atomicAdd(&s_arrived[slot], 1) == 0) return; // the sibling subtree is not done yet
        __threadfence_block();
        for (int c = 0; c < 3; ++c) {
            lo[c] = fminf(lo[c], s_box[1 - side][c][slot]);
            hi[c] = fmaxf(hi[c], s_box[1 - side][3 + c][slot]);
        }
        child = node;
        node = parent[node];
        // This box is read again inside this kernel only if the parent is met through memory (then by whichever
        // thread arrives there second, maybe on another XCD): only then does it have to go out as agent-scope
        // stores.  Everything below such a subtree root is next read by other kernels: plain stores.
        bool inside = false;
        if (node >= 0) {
            const int32_t o = other_end[node];
            inside = (node < o ? node : o) >= b0 && (node < o ? o : node) <= b1;
        }
        if (inside) {
            for (int c = 0; c < 3; ++c) {
                nodes[child].lo[c] = lo[c];
                nodes[child].hi[c] = hi[c];
            }
        } else {
            for (int c = 0; c < 3; ++c) {
                st_agent(&nodes[child].lo[c], lo[c]);
                st_agent(&nodes[child].hi[c], hi[c]);
            }
            break;
        }
    }
    // the rest of the way: through memory.  The thread carries its child's box in registers and reads only the
    // sibling's; the indices it will need after the counter (children, next parent) are asked for before the wait,
    // so that each level is three trips to memory one after the other (stores acknowledged, counter, sibling's box)
    // and not five.
    while (node >= 0) {
        const int32_t left = nodes[node].left, rgt = right[node], up = parent[node];
#if defined(__gfx942__) || defined(__gfx950__)
        // (the immediate below is the gfx9 encoding of vmcnt(0) with the other counters left alone, and the
        // argument that the wait suffices rests on how these chips complete agent-scope atomic stores)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup"); // compiler ordering
        __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0): this thread's box stores have completed
        if (atomicAdd(&flags[node], 1) == 0) return; // the sibling subtree is not done yet
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#else
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        if (atomicAdd(&flags[node], 1) == 0) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#endif
        const Node *sibling = &nodes[left == child ? rgt : left];
        for (int c = 0; c < 3; ++c) {
            lo[c] = fminf(lo[c], ld_agent(&sibling->lo[c]));
            hi[c] = fmaxf(hi[c], ld_agent(&sibling->hi[c]));
            st_agent(&nodes[node].lo[c], lo[c]);
            st_agent(&nodes[node].hi[c], hi[c]);
        }
        child = node;
        node = up;
    }
}

__global__ __launch_bounds__(256) void k_skip_links(int64_t n, Node *__restrict__ nodes, const int32_t *__restrict__ parent,
                                                    const int32_t *__restrict__ right, const int32_t *gate = nullptr)
{
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= 2 * n - 1 || gate_closed(gate)) return;
    int32_t cur = (int32_t)id, skip = -1;
    for (;;) {
        const int32_t p = parent[cur];
        if (p < 0) break;
        if (nodes[p].left == cur) { skip = right[p]; break; }
        cur = p;
    }
    nodes[id].skip = skip;
}

__global__ void k_mark_built(WsHeader *h, const int32_t *gate = nullptr)
{
    if (!gate_closed(gate)) h->built = 1;
}

// ---------------------------------------------------------------------------
static inline dim3 grid_for(int64_t n, int block) { return dim3((unsigned)((n + block - 1) / block)); }
// For the kernels that loop over their input and end with atomics on a few shared words: two blocks per CU.
static inline dim3 grid_reduce(int64_t n, int block) { return dim3((unsigned)std::min<int64_t>((n + block - 1) / block, 512)); }

extern "C" int rgx_aabb(const float *pos, const float *scale, const float *quat, const float *dens, int64_t n,
                        float sigma_threshold, float *bboxes, float *bb_min, float *bb_max, void *stream)
{
    const DeviceScope on_device(pos);
    if (n < 0 || (n > 0 && (!pos || !scale || !quat || !dens)) || ((bb_min == nullptr) != (bb_max == nullptr)))
        return RGX_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    int32_t *mn = (int32_t *)bb_min, *mx = (int32_t *)bb_max;
    if (mn) hipLaunchKernelGGL(k_init_enc, dim3(1), dim3(64), 0, s, mn, mx);
    if (n > 0)
        hipLaunchKernelGGL(k_aabb, grid_reduce(n, 256), dim3(256), 0, s, pos, scale, quat, dens, n, sigma_threshold, bboxes, mn, mx);
    if (mn) hipLaunchKernelGGL(k_decode_enc, dim3(1), dim3(64), 0, s, mn, mx);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

extern "C" int rgx_build_workspace_bytes(int64_t n, size_t *bytes)
{
    if (n < 0 || !bytes || n > 0x3fffffff) return RGX_EINVAL;
    *bytes = rgx_ws_layout(n).total;
    return RGX_OK;
}

// Copies caller-supplied boxes into the workspace and reduces the scene bbox.
__global__ __launch_bounds__(256) void k_take_boxes(const float *__restrict__ in, int64_t n, float *__restrict__ boxes,
                                                    int32_t *mn_enc, int32_t *mx_enc, const int32_t *gate = nullptr)
{
    if (gate_closed(gate)) return; // the whole grid
    float b[6] = {INFINITY, INFINITY, INFINITY, -INFINITY, -INFINITY, -INFINITY};
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        for (int a = 0; a < 6; ++a) {
            const float v = boxes[6 * i + a] = in[6 * i + a];
            b[a] = a < 3 ? fminf(b[a], v) : fmaxf(b[a], v);
        }
    __shared__ float red[4][6];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int a = 0; a < 3; ++a) {
        const float mn = wave_min(b[a]), mx = wave_max(b[a + 3]);
        if (lane == 0) { red[wave][a] = mn; red[wave][a + 3] = mx; }
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        const int a = threadIdx.x;
        atomicMin(&mn_enc[a], enc_f(fminf(fminf(red[0][a], red[1][a]), fminf(red[2][a], red[3][a]))));
        atomicMax(&mx_enc[a], enc_f(fmaxf(fmaxf(red[0][a + 3], red[1][a + 3]), fmaxf(red[2][a + 3], red[3][a + 3]))));
    }
}

static int build_impl(const float *pos, const float *scale, const float *quat, const float *dens, const float *in_boxes,
                      int64_t n, float sigma_threshold, void *ws, size_t ws_bytes, void *stream);

extern "C" int rgx_build(const float *pos, const float *scale, const float *quat, const float *dens, int64_t n,
                         float sigma_threshold, void *ws, size_t ws_bytes, void *stream)
{
    if (n > 0 && (!pos || !scale || !quat || !dens)) return RGX_EINVAL;
    return build_impl(pos, scale, quat, dens, nullptr, n, sigma_threshold, ws, ws_bytes, stream);
}

extern "C" int rgx_build_aabbs(const float *bboxes, int64_t n, void *ws, size_t ws_bytes, void *stream)
{
    if (n > 0 && !bboxes) return RGX_EINVAL;
    return build_impl(nullptr, nullptr, nullptr, nullptr, bboxes, n, 0.f, ws, ws_bytes, stream);
}

static int build_impl(const float *pos, const float *scale, const float *quat, const float *dens, const float *in_boxes,
                      int64_t n, float sigma_threshold, void *ws, size_t ws_bytes, void *stream)
{
    const DeviceScope on_device(ws);
    if (n < 0 || n > 0x3fffffff || !ws) return RGX_EINVAL;
    const WsLayout L = rgx_ws_layout(n);
    if (ws_bytes < L.total || ((uintptr_t)ws & 255u)) return RGX_EWORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char *w = (char *)ws;
    WsHeader *hdr = (WsHeader *)(w + L.header);
    float *boxes = (float *)(w + L.aabb);
    uint64_t *k0 = (uint64_t *)(w + L.keys0), *k1 = (uint64_t *)(w + L.keys1);
    uint32_t *v0 = (uint32_t *)(w + L.vals0), *v1 = (uint32_t *)(w + L.vals1);
    Node *nodes = (Node *)(w + L.nodes);
    int32_t *parent = (int32_t *)(w + L.parent), *right = (int32_t *)(w + L.right), *flags = (int32_t *)(w + L.flags);
    uint32_t *hist = (uint32_t *)(w + L.hist);

    void *span = rgx_span_begin(RGX_T_BUILD, s);
    hipLaunchKernelGGL(k_init_header, dim3(1), dim3(64), 0, s, hdr, n);
    if (n > 0) {
        if (in_boxes)
            hipLaunchKernelGGL(k_take_boxes, grid_reduce(n, 256), dim3(256), 0, s, in_boxes, n, boxes, hdr->bb_min_enc,
                               hdr->bb_max_enc);
        else
            hipLaunchKernelGGL(k_aabb, grid_reduce(n, 256), dim3(256), 0, s, pos, scale, quat, dens, n, sigma_threshold, boxes,
                               hdr->bb_min_enc, hdr->bb_max_enc);
        hipLaunchKernelGGL(k_finish_bbox, dim3(1), dim3(64), 0, s, hdr, (float *)nullptr, (float *)nullptr);
        hipLaunchKernelGGL(k_morton63, grid_for(n, 256), dim3(256), 0, s, boxes, n, hdr, k0, v0);
        RGX_LAUNCH_CHECK();
        const int r = radix_sort<uint64_t>(k0, v0, k1, v1, n, 64, hist, s);
        if (r < 0) return r;
        // 8 passes: the sorted keys / permutation are back in (k0, v0)
        hipLaunchKernelGGL(k_leaves, grid_for(n, 256), dim3(256), 0, s, boxes, v0, n, nodes, parent, flags, v1); // (the sort's second value buffer is free again)
        if (n > 1) {
            int32_t *other_end = (int32_t *)k1; // the sort's second key buffer is free again
            hipLaunchKernelGGL(k_karras, grid_for(n - 1, 256), dim3(256), 0, s, k0, n, nodes, parent, right, other_end);
            hipLaunchKernelGGL(k_refit, grid_for(n, 256), dim3(256), 0, s, n, nodes, parent, right, other_end, flags);
        }
        hipLaunchKernelGGL(k_skip_links, grid_for(2 * n - 1, 256), dim3(256), 0, s, n, nodes, parent, right);
    }
    hipLaunchKernelGGL(k_mark_built, dim3(1), dim3(1), 0, s, hdr);
    rgx_span_end(span, s);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

// Refit: the tree's shape (children, parents, sorted order) stays as the last build into `ws` left it;
// leaf boxes are taken from `bboxes`, internal boxes and the scene box recomputed bottom-up.
// Precondition, checked on the device by the refit's first kernel: `ws` holds a finished tree over exactly
// `n` boxes.  If it does not, no kernel of the refit touches the tree, the workspace is left marked not
// built (rgx_scene_bbox then reports RGX_EWORKSPACE) and the call still returns RGX_OK: the check runs in
// stream order and the host does not wait for it.
extern "C" int rgx_refit_aabbs(const float *bboxes, int64_t n, void *ws, size_t ws_bytes, void *stream)
{
    if (n < 0 || n > 0x3fffffff || !ws || (n > 0 && !bboxes)) return RGX_EINVAL;
    const DeviceScope on_device(ws);
    const WsLayout L = rgx_ws_layout(n);
    if (ws_bytes < L.total || ((uintptr_t)ws & 255u)) return RGX_EWORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    char *w = (char *)ws;
    WsHeader *hdr = (WsHeader *)(w + L.header);
    float *boxes = (float *)(w + L.aabb);
    const uint32_t *order = (const uint32_t *)(w + L.vals0);
    Node *nodes = (Node *)(w + L.nodes);
    int32_t *parent = (int32_t *)(w + L.parent), *right = (int32_t *)(w + L.right), *flags = (int32_t *)(w + L.flags);
    const int32_t *other_end = (const int32_t *)(w + L.keys1); // left there by the build
    void *span = rgx_span_begin(RGX_T_BUILD, s);
    const int32_t *gate = &hdr->refit_ok;
    hipLaunchKernelGGL(k_refit_begin, dim3(1), dim3(64), 0, s, hdr, n);
    if (n > 0) {
        hipLaunchKernelGGL(k_take_boxes, grid_reduce(n, 256), dim3(256), 0, s, bboxes, n, boxes, hdr->bb_min_enc, hdr->bb_max_enc, gate);
        hipLaunchKernelGGL(k_finish_bbox, dim3(1), dim3(64), 0, s, hdr, (float *)nullptr, (float *)nullptr, gate);
        hipLaunchKernelGGL(k_leaves, grid_for(n, 256), dim3(256), 0, s, boxes, order, n, nodes, parent, flags, (uint32_t *)(w + L.vals1), gate);
        if (n > 1) hipLaunchKernelGGL(k_refit, grid_for(n, 256), dim3(256), 0, s, n, nodes, parent, right, other_end, flags, gate);
        hipLaunchKernelGGL(k_skip_links, grid_for(2 * n - 1, 256), dim3(256), 0, s, n, nodes, parent, right, gate);
    }
    hipLaunchKernelGGL(k_mark_built, dim3(1), dim3(1), 0, s, hdr, gate);
    rgx_span_end(span, s);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

extern "C" int rgx_build_layout(int64_t n, size_t *host_out6)
{
    if (n < 0 || n > 0x3fffffff || !host_out6) return RGX_EINVAL;
    const WsLayout L = rgx_ws_layout(n);
    host_out6[0] = L.aabb;
    host_out6[1] = L.vals0;
    host_out6[2] = L.nodes;
    host_out6[3] = L.parent;
    host_out6[4] = L.right;
    host_out6[5] = L.header;
    return RGX_OK;
}

// ---------------------------------------------------------------------------
// Synchronous / small read-backs of a built workspace.
extern "C" int rgx_scene_bbox(const void *ws, float *host_out6, void *stream)
{
    const DeviceScope on_device(ws);
    if (!ws || !host_out6) return RGX_EINVAL;
    WsHeader h;
    RGX_HIP(hipMemcpyAsync(&h, ws, sizeof h, hipMemcpyDeviceToHost, (hipStream_t)stream));
    RGX_HIP(hipStreamSynchronize((hipStream_t)stream));
    if (h.built != 1) return RGX_EWORKSPACE; // never built, or a refit that found no tree of its size to refit
    for (int a = 0; a < 3; ++a) {
        host_out6[a] = h.bb_min[a];
        host_out6[3 + a] = h.bb_max[a];
    }
    return RGX_OK;
}

__global__ __launch_bounds__(256) void k_copy_order(const uint32_t *__restrict__ v, int64_t n, int32_t *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (int32_t)v[i];
}

extern "C" int rgx_build_order(const void *ws, int64_t n, int32_t *order_out, void *stream)
{
    const DeviceScope on_device(ws);
    if (!ws || n < 0 || (n > 0 && !order_out)) return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    const WsLayout L = rgx_ws_layout(n);
    hipLaunchKernelGGL(k_copy_order, grid_for(n, 256), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t *)((const char *)ws + L.vals0), n, order_out);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

// ---------------------------------------------------------------------------
// 30-bit Morton ordering of the point cloud (utils/reordering_utils.py:55-104,
// classes/point_cloud.py:1017-1024).
__global__ __launch_bounds__(256) void k_pos_minmax(const float *__restrict__ pos, int64_t n, int32_t *mn_enc, int32_t *mx_enc)
{
    float b[6] = {INFINITY, INFINITY, INFINITY, -INFINITY, -INFINITY, -INFINITY};
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        for (int a = 0; a < 3; ++a) {
            const float v = pos[3 * i + a];
            b[a] = fminf(b[a], v);
            b[a + 3] = fmaxf(b[a + 3], v);
        }
    __shared__ float red[4][6];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int a = 0; a < 3; ++a) {
        const float mn = wave_min(b[a]), mx = wave_max(b[a + 3]);
        if (lane == 0) { red[wave][a] = mn; red[wave][a + 3] = mx; }
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        const int a = threadIdx.x;
        atomicMin(&mn_enc[a], enc_f(fminf(fminf(red[0][a], red[1][a]), fminf(red[2][a], red[3][a]))));
        atomicMax(&mx_enc[a], enc_f(fmaxf(fmaxf(red[0][a + 3], red[1][a + 3]), fmaxf(red[2][a + 3], red[3][a + 3]))));
    }
}

__global__ __launch_bounds__(256) void k_morton30(const float *__restrict__ pos, int64_t n, const float *__restrict__ mn,
                                                  const float *__restrict__ mx, uint32_t *__restrict__ keys,
                                                  uint32_t *__restrict__ vals, int64_t *__restrict__ codes)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint32_t code = 0;
    for (int a = 0; a < 3; ++a) {
        const float scale = 1023.0f / ((mx[a] - mn[a]) + 1e-9f); // reordering_utils.py:73
        const int32_t q = (int32_t)((pos[3 * i + a] - mn[a]) * scale); // .to(torch.int32): truncation
        for (int b = 0; b < 10; ++b) code |= (uint32_t)((q >> b) & 1) << (3 * b + a); // reordering_utils.py:98-102
    }
    keys[i] = code;
    vals[i] = (uint32_t)i;
    if (codes) codes[i] = (int64_t)code;
}

__global__ __launch_bounds__(256) void k_order64(const uint32_t *__restrict__ v, int64_t n, int64_t *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (int64_t)v[i];
}

struct MortonLayout {
    size_t enc, keys0, keys1, vals0, vals1, hist, total;
};
static inline MortonLayout morton_layout(int64_t n)
{
    MortonLayout L;
    const size_t nn = (size_t)(n > 0 ? n : 1), nblocks = (nn + RGX_RS_TILE - 1) / RGX_RS_TILE;
    size_t off = 0;
    L.enc = off;   off = rgx_align_up(off + 8 * sizeof(int32_t), 256);
    L.keys0 = off; off = rgx_align_up(off + nn * 4, 256);
    L.keys1 = off; off = rgx_align_up(off + nn * 4, 256);
    L.vals0 = off; off = rgx_align_up(off + nn * 4, 256);
    L.vals1 = off; off = rgx_align_up(off + nn * 4, 256);
    L.hist = off;  off = rgx_align_up(off + 256 * (nblocks + 1) * 4, 256);
    L.total = off;
    return L;
}

extern "C" int rgx_morton_workspace_bytes(int64_t n, size_t *bytes)
{
    if (n < 0 || !bytes || n > 0x3fffffff) return RGX_EINVAL;
    *bytes = morton_layout(n).total;
    return RGX_OK;
}

extern "C" int rgx_morton_order(const float *pos, int64_t n, int64_t *codes, int64_t *order, void *ws, size_t ws_bytes,
                                void *stream)
{
    const DeviceScope on_device(pos);
    if (n < 0 || n > 0x3fffffff || !ws || (n > 0 && !pos)) return RGX_EINVAL;
    const MortonLayout L = morton_layout(n);
    if (ws_bytes < L.total || ((uintptr_t)ws & 255u)) return RGX_EWORKSPACE;
    if (n == 0) return RGX_OK;
    hipStream_t s = (hipStream_t)stream;
    char *w = (char *)ws;
    int32_t *mn = (int32_t *)(w + L.enc), *mx = mn + 4;
    uint32_t *k0 = (uint32_t *)(w + L.keys0), *k1 = (uint32_t *)(w + L.keys1);
    uint32_t *v0 = (uint32_t *)(w + L.vals0), *v1 = (uint32_t *)(w + L.vals1);
    hipLaunchKernelGGL(k_init_enc, dim3(1), dim3(64), 0, s, mn, mx);
    hipLaunchKernelGGL(k_pos_minmax, grid_reduce(n, 256), dim3(256), 0, s, pos, n, mn, mx);
    hipLaunchKernelGGL(k_decode_enc, dim3(1), dim3(64), 0, s, mn, mx);
    hipLaunchKernelGGL(k_morton30, grid_for(n, 256), dim3(256), 0, s, pos, n, (const float *)mn, (const float *)mx, k0, v0, codes);
    RGX_LAUNCH_CHECK();
    if (order) {
        const int r = radix_sort<uint32_t>(k0, v0, k1, v1, n, 32, (uint32_t *)(w + L.hist), s);
        if (r < 0) return r;
        hipLaunchKernelGGL(k_order64, grid_for(n, 256), dim3(256), 0, s, v0, n, order);
        RGX_LAUNCH_CHECK();
    }
    return RGX_OK;
}

// ---------------------------------------------------------------------------
// Fused multi-tensor gather for the periodic reordering of the point cloud: every
// per-Gaussian tensor (parameters, Adam moments, statistics) is permuted with the same index
// (classes/point_cloud.py:1031-1044, classes/optimizer.py:54-66: one `tensor[index]` launch per
// tensor there).  blockIdx.y picks the tensor; a thread moves one 32-bit word, so writes are
// coalesced and the reads of a row are contiguous.
#define RGX_GATHER_MAX 24
struct GatherArgs {
    const uint32_t *src[RGX_GATHER_MAX];
    uint32_t *dst[RGX_GATHER_MAX];
    int32_t row_words[RGX_GATHER_MAX];
};

__global__ __launch_bounds__(256) void k_gather_rows(const GatherArgs A, const int64_t *__restrict__ order, int64_t n)
{
    const int t = blockIdx.y;
    const int64_t rw = A.row_words[t];
    const int64_t total = n * rw;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = e / rw, w = e - row * rw;
        A.dst[t][e] = A.src[t][order[row] * rw + w];
    }
}

extern "C" int rgx_gather_rows(int32_t count, const void *const *src, void *const *dst, const int64_t *row_bytes,
                               const int64_t *order, int64_t n, void *stream)
{
    const DeviceScope on_device(order);
    if (count < 0 || n < 0 || (count > 0 && (!src || !dst || !row_bytes)) || (n > 0 && count > 0 && !order)) return RGX_EINVAL;
    for (int i = 0; i < count; ++i)
        if (row_bytes[i] <= 0 || (row_bytes[i] & 3) || row_bytes[i] > 0x7fffffff || ((!src[i] || !dst[i]) && n > 0) || src[i] == dst[i])
            return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    for (int base = 0; base < count; base += RGX_GATHER_MAX) {
        GatherArgs A;
        const int m = count - base < RGX_GATHER_MAX ? count - base : RGX_GATHER_MAX;
        int64_t most = 0;
        for (int i = 0; i < m; ++i) {
            A.src[i] = (const uint32_t *)src[base + i];
            A.dst[i] = (uint32_t *)dst[base + i];
            A.row_words[i] = (int32_t)(row_bytes[base + i] / 4);
            most = most > n * A.row_words[i] ? most : n * A.row_words[i];
        }
        int64_t blocks = (most + 255) / 256;
        if (blocks > 65536) blocks = 65536; // grid-stride beyond that
        hipLaunchKernelGGL(k_gather_rows, dim3((unsigned)blocks, (unsigned)m), dim3(256), 0, (hipStream_t)stream, A, order, n);
        RGX_LAUNCH_CHECK();
    }
    return RGX_OK;
}

// ---------------------------------------------------------------------------
// Mean squared distance of every point to its three nearest neighbours: distCUDA2 of the
// simple-knn extension (submodules/simple-knn/simple_knn.cu:186-222; used to initialise the scales,
// classes/point_cloud.py:252).  As there: points sorted along a Morton curve, boxes of consecutive
// sorted points, every point scans the boxes that can still hold one of its three nearest (the
// pruning is exact, so the result is the exact 3-NN mean whatever the order and the box size).
// Here the boxes have two levels (256 points, 64 boxes) so that a point looks at a few hundred box
// bounds instead of all n / 256, and the sorted points are gathered once so that the scans read
// consecutive memory.  Distances are (dx*dx + dy*dy) + dz*dz without contraction.
#define RGX_KNN_BOX 256
#define RGX_KNN_SUPER 64

__global__ __launch_bounds__(256) void k_knn_gather(const float *__restrict__ pos, const uint32_t *__restrict__ order, int64_t n,
                                                    float4 *__restrict__ pts)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t j = order[i];
    pts[i] = make_float4(pos[3 * j], pos[3 * j + 1], pos[3 * j + 2], 0.f);
}

// bounds of `per` consecutive items: points (float4) at level 0, boxes (lo, hi pairs) above
__global__ __launch_bounds__(256) void k_knn_bounds(const float4 *__restrict__ lo_in, const float4 *__restrict__ hi_in,
                                                    int stride, int64_t n_in, int per, float4 *__restrict__ out)
{
    const int64_t b = blockIdx.x;
    float mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
    for (int64_t i = b * per + threadIdx.x; i < n_in && i < (b + 1) * per; i += blockDim.x) {
        const float4 l = lo_in[i * stride], h = hi_in[i * stride];
        mn[0] = fminf(mn[0], l.x); mn[1] = fminf(mn[1], l.y); mn[2] = fminf(mn[2], l.z);
        mx[0] = fmaxf(mx[0], h.x); mx[1] = fmaxf(mx[1], h.y); mx[2] = fmaxf(mx[2], h.z);
    }
    __shared__ float red[4][6];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int a = 0; a < 3; ++a) {
        const float l = wave_min(mn[a]), h = wave_max(mx[a]);
        if (lane == 0) { red[wave][a] = l; red[wave][a + 3] = h; }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int a = 0; a < 6; ++a)
            for (int w = 1; w < 4; ++w) red[0][a] = a < 3 ? fminf(red[0][a], red[w][a]) : fmaxf(red[0][a], red[w][a]);
        out[2 * b] = make_float4(red[0][0], red[0][1], red[0][2], 0.f);
        out[2 * b + 1] = make_float4(red[0][3], red[0][4], red[0][5], 0.f);
    }
}

// simple_knn.cu:124-135 distBoxPoint
__device__ __forceinline__ float knn_box_dist(float4 lo, float4 hi, float4 p)
{
    float dx = 0.f, dy = 0.f, dz = 0.f;
    if (p.x < lo.x || p.x > hi.x) dx = fminf(fabsf(p.x - lo.x), fabsf(p.x - hi.x));
    if (p.y < lo.y || p.y > hi.y) dy = fminf(fabsf(p.y - lo.y), fabsf(p.y - hi.y));
    if (p.z < lo.z || p.z > hi.z) dz = fminf(fabsf(p.z - lo.z), fabsf(p.z - hi.z));
    return (dx * dx + dy * dy) + dz * dz;
}

// simple_knn.cu:137-151 updateKBest<3>
__device__ __forceinline__ void knn_update(float4 ref, float4 q, float *best)
{
    const float dx = q.x - ref.x, dy = q.y - ref.y, dz = q.z - ref.z;
    float dist = (dx * dx + dy * dy) + dz * dz;
#pragma unroll
    for (int j = 0; j < 3; ++j)
        if (best[j] > dist) {
            const float t = best[j];
            best[j] = dist;
            dist = t;
        }
}

// simple_knn.cu:153-184 boxMeanDist
__global__ __launch_bounds__(256) void k_knn3(const float4 *__restrict__ pts, const uint32_t *__restrict__ order, int64_t n,
                                              const float4 *__restrict__ boxes, int64_t nb, const float4 *__restrict__ supers,
                                              int64_t ns, float *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float4 p = pts[i];
    float best[3] = {FLT_MAX, FLT_MAX, FLT_MAX};
    for (int64_t j = i - 3 < 0 ? 0 : i - 3; j <= (i + 3 > n - 1 ? n - 1 : i + 3); ++j)
        if (j != i) knn_update(p, pts[j], best);
    const float reject = best[2];
    best[0] = best[1] = best[2] = FLT_MAX;
    for (int64_t s = 0; s < ns; ++s) {
        const float ds = knn_box_dist(supers[2 * s], supers[2 * s + 1], p);
        if (ds > reject || ds > best[2]) continue;
        const int64_t b1 = (s + 1) * RGX_KNN_SUPER < nb ? (s + 1) * RGX_KNN_SUPER : nb;
        for (int64_t b = s * RGX_KNN_SUPER; b < b1; ++b) {
            const float d = knn_box_dist(boxes[2 * b], boxes[2 * b + 1], p);
            if (d > reject || d > best[2]) continue;
            const int64_t j1 = (b + 1) * RGX_KNN_BOX < n ? (b + 1) * RGX_KNN_BOX : n;
            for (int64_t j = b * RGX_KNN_BOX; j < j1; ++j)
                if (j != i) knn_update(p, pts[j], best);
        }
    }
    out[order[i]] = ((best[0] + best[1]) + best[2]) / 3.0f;
}

struct KnnLayout {
    MortonLayout m;
    size_t pts, boxes, supers, total;
    int64_t nb, ns;
};
static inline KnnLayout knn_layout(int64_t n)
{
    KnnLayout K;
    K.m = morton_layout(n);
    const size_t nn = (size_t)(n > 0 ? n : 1);
    K.nb = (int64_t)((nn + RGX_KNN_BOX - 1) / RGX_KNN_BOX);
    K.ns = (K.nb + RGX_KNN_SUPER - 1) / RGX_KNN_SUPER;
    size_t off = K.m.total;
    K.pts = off;    off = rgx_align_up(off + nn * 16, 256);
    K.boxes = off;  off = rgx_align_up(off + (size_t)K.nb * 32, 256);
    K.supers = off; off = rgx_align_up(off + (size_t)K.ns * 32, 256);
    K.total = off;
    return K;
}

extern "C" int rgx_knn_workspace_bytes(int64_t n, size_t *bytes)
{
    if (n < 0 || !bytes || n > 0x3fffffff) return RGX_EINVAL;
    *bytes = knn_layout(n).total;
    return RGX_OK;
}

extern "C" int rgx_dist2_knn3(const float *pos, int64_t n, float *mean_dist2, void *ws, size_t ws_bytes, void *stream)
{
    const DeviceScope on_device(pos);
    if (n < 0 || n > 0x3fffffff || !ws || (n > 0 && (!pos || !mean_dist2))) return RGX_EINVAL;
    const KnnLayout K = knn_layout(n);
    if (ws_bytes < K.total || ((uintptr_t)ws & 255u)) return RGX_EWORKSPACE;
    if (n == 0) return RGX_OK;
    hipStream_t s = (hipStream_t)stream;
    char *w = (char *)ws;
    int32_t *mn = (int32_t *)(w + K.m.enc), *mx = mn + 4;
    uint32_t *k0 = (uint32_t *)(w + K.m.keys0), *k1 = (uint32_t *)(w + K.m.keys1);
    uint32_t *v0 = (uint32_t *)(w + K.m.vals0), *v1 = (uint32_t *)(w + K.m.vals1);
    float4 *pts = (float4 *)(w + K.pts), *boxes = (float4 *)(w + K.boxes), *supers = (float4 *)(w + K.supers);
    hipLaunchKernelGGL(k_init_enc, dim3(1), dim3(64), 0, s, mn, mx);
    hipLaunchKernelGGL(k_pos_minmax, grid_reduce(n, 256), dim3(256), 0, s, pos, n, mn, mx);
    hipLaunchKernelGGL(k_decode_enc, dim3(1), dim3(64), 0, s, mn, mx);
    hipLaunchKernelGGL(k_morton30, grid_for(n, 256), dim3(256), 0, s, pos, n, (const float *)mn, (const float *)mx, k0, v0,
                       (int64_t *)nullptr);
    RGX_LAUNCH_CHECK();
    const int r = radix_sort<uint32_t>(k0, v0, k1, v1, n, 32, (uint32_t *)(w + K.m.hist), s);
    if (r < 0) return r;
    hipLaunchKernelGGL(k_knn_gather, grid_for(n, 256), dim3(256), 0, s, pos, v0, n, pts);
    hipLaunchKernelGGL(k_knn_bounds, dim3((unsigned)K.nb), dim3(256), 0, s, pts, pts, 1, n, RGX_KNN_BOX, boxes);
    hipLaunchKernelGGL(k_knn_bounds, dim3((unsigned)K.ns), dim3(256), 0, s, boxes, boxes + 1, 2, K.nb, RGX_KNN_SUPER, supers);
    hipLaunchKernelGGL(k_knn3, grid_for(n, 256), dim3(256), 0, s, pts, v0, n, boxes, K.nb, supers, K.ns, mean_dist2);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}
