// Per-Gaussian streaming kernels: view-dependent colour from spherical
// harmonics + spherical Gaussians (utils/sh_utils.cu:122-216), its gradient
// (utils/sh_utils.cu:218-412) and packing of the 64-byte primitive record
// (optix_raycasting/optix_utils.py:268-304).  One thread per Gaussian.
#include "rgx_device.h"

__constant__ float SH_C0 = 0.28209479177387814f;
__constant__ float SH_C1 = 0.4886025119029199f;
__constant__ float SH_C2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                               -1.0925484305920792f, 0.5462742152960396f};
__constant__ float SH_C3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                               0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                               -0.5900435899266435f};

// basis_j(dir), j < (degree+1)^2, in the order forward_sh multiplies sh[j] (sh_utils.cu:157-209)
template <int DEG>
__device__ __forceinline__ void sh_basis(float x, float y, float z, float *b)
{
    b[0] = SH_C0;
    if constexpr (DEG > 0) {
        b[1] = -SH_C1 * y; b[2] = SH_C1 * z; b[3] = -SH_C1 * x;
    }
    if constexpr (DEG > 1) {
        const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
        b[4] = SH_C2[0] * xy; b[5] = SH_C2[1] * yz; b[6] = SH_C2[2] * (2.0f * zz - xx - yy);
        b[7] = SH_C2[3] * xz; b[8] = SH_C2[4] * (xx - yy);
        if constexpr (DEG > 2) {
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

// The colour of one Gaussian (sh_utils.cu:122-216).  coeff: its coefficients, Ks per channel.
template <int DEG>
__device__ __forceinline__ void sh_fwd_one(f3 eye, const float *__restrict__ pos, const float *__restrict__ coeff,
                                           const float *__restrict__ sg, const float *__restrict__ sharp,
                                           const float *__restrict__ axis, int G, int Gs, int Ks, int64_t i,
                                           float *__restrict__ rgb)
{
    // Gs, Ks: lobes / coefficients STORED per Gaussian and channel (>= G, >= K): the viewer keeps
    // room for the largest model and evaluates the first G lobes and K coefficients (gui_sh,
    // sh_utils.cu:25-119); everywhere else they equal G and K.
    constexpr int K = (DEG + 1) * (DEG + 1);
    const f3 v = mk3(pos[3 * i] - eye.x, pos[3 * i + 1] - eye.y, pos[3 * i + 2] - eye.z);
    const float len = sqrtf(dot3(v, v));
    const f3 d = mk3(v.x / len, v.y / len, v.z / len);
    float res[3] = {0.f, 0.f, 0.f};
    for (int l = 0; l < G; ++l) {
        const f3 ax = mk3(axis[(i * Gs + l) * 3], axis[(i * Gs + l) * 3 + 1], axis[(i * Gs + l) * 3 + 2]);
        const float g = expf(sharp[i * Gs + l] * (dot3(d, ax) - 1.0f));
        for (int c = 0; c < 3; ++c) res[c] += sg[i * Gs * 3 + c * Gs + l] * g;
    }
    float b[K];
    sh_basis<DEG>(d.x, d.y, d.z, b);
    for (int c = 0; c < 3; ++c) {
        const float *s = coeff + c * Ks;
        float r = res[c];
#pragma unroll
        for (int j = 0; j < K; ++j) r += b[j] * s[j];
        rgb[3 * i + c] = r + 0.5f;
    }
}

template <int DEG>
__global__ __launch_bounds__(256) void k_sh_fwd(f3 eye, const float *__restrict__ pos, const float *__restrict__ sh,
                                                const float *__restrict__ sg, const float *__restrict__ sharp,
                                                const float *__restrict__ axis, int G, int Gs, int Ks, int64_t n,
                                                float *__restrict__ rgb)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    sh_fwd_one<DEG>(eye, pos, sh + i * 3 * Ks, sg, sharp, axis, G, Gs, Ks, i, rgb);
}

// Degree 3 with 16 coefficients stored per channel: the 192-byte rows of a workgroup's 256 Gaussians staged in LDS
// (see k_sh_bwd3_rows).
__global__ __launch_bounds__(256) void k_sh_fwd3_rows(f3 eye, const float *__restrict__ pos, const float *__restrict__ sh,
                                                      const float *__restrict__ sg, const float *__restrict__ sharp,
                                                      const float *__restrict__ axis, int G, int Gs, int64_t n,
                                                      float *__restrict__ rgb)
{
    constexpr int ROW4 = 12, STRIDE4 = 13;
    __shared__ float4 s_rows[256 * STRIDE4];
    const int64_t i0 = (int64_t)blockIdx.x * 256;
    const int rows = (int)(n - i0 < 256 ? n - i0 : 256);
    const float4 *src = (const float4 *)sh + i0 * ROW4;
    for (int g = threadIdx.x; g < rows * ROW4; g += 256) {
        const int r = g / ROW4;
        s_rows[r * STRIDE4 + (g - r * ROW4)] = src[g];
    }
    __syncthreads();
    if ((int)threadIdx.x < rows)
        sh_fwd_one<3>(eye, pos, (const float *)&s_rows[threadIdx.x * STRIDE4], sg, sharp, axis, G, Gs, 16, i0 + threadIdx.x, rgb);
}

// The gradient of one Gaussian (sh_utils.cu:218-412).  coeff: its 3 K coefficients; o_sh: where their gradient goes
// (may be the same memory: every coefficient is read before the first gradient is written).
template <int DEG>
__device__ __forceinline__ void sh_bwd_one(f3 eye, const float *__restrict__ pos, const float *coeff,
                                           const float *__restrict__ sg, const float *__restrict__ sharp,
                                           const float *__restrict__ axis, int G, int64_t i,
                                           const float *__restrict__ drgb, float *o_sh,
                                           float *__restrict__ dpos, float *__restrict__ dsg,
                                           float *__restrict__ dsharp, float *__restrict__ daxis)
{
    constexpr int K = (DEG + 1) * (DEG + 1);
    const float gr[3] = {drgb[3 * i], drgb[3 * i + 1], drgb[3 * i + 2]};
    if (gr[0] == 0.f && gr[1] == 0.f && gr[2] == 0.f) { // sh_utils.cu:226 (outputs stay zero)
        for (int j = 0; j < 3 * K; ++j) o_sh[j] = 0.f;
        dpos[3 * i] = dpos[3 * i + 1] = dpos[3 * i + 2] = 0.f;
        for (int l = 0; l < G; ++l) {
            for (int c = 0; c < 3; ++c) { dsg[i * G * 3 + c * G + l] = 0.f; daxis[(i * G + l) * 3 + c] = 0.f; }
            dsharp[i * G + l] = 0.f;
        }
        return;
    }
    const f3 v = mk3(pos[3 * i] - eye.x, pos[3 * i + 1] - eye.y, pos[3 * i + 2] - eye.z);
    const float len = sqrtf(dot3(v, v));
    const float x = v.x / len, y = v.y / len, z = v.z / len;
    float b[K];
    sh_basis<DEG>(x, y, z, b);
    float dx[3] = {0, 0, 0}, dy[3] = {0, 0, 0}, dz[3] = {0, 0, 0};
    if constexpr (DEG > 0) {
        const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
        for (int c = 0; c < 3; ++c) {
            const float *s = coeff + c * K;
            dx[c] = -SH_C1 * s[3]; dy[c] = -SH_C1 * s[1]; dz[c] = SH_C1 * s[2];
            if constexpr (DEG > 1) {
                dx[c] += SH_C2[0] * y * s[4] + SH_C2[2] * 2.0f * -x * s[6] + SH_C2[3] * z * s[7] + SH_C2[4] * 2.0f * x * s[8];
                dy[c] += SH_C2[0] * x * s[4] + SH_C2[1] * z * s[5] + SH_C2[2] * 2.0f * -y * s[6] + SH_C2[4] * 2.0f * -y * s[8];
                dz[c] += SH_C2[1] * y * s[5] + SH_C2[2] * 2.0f * 2.0f * z * s[6] + SH_C2[3] * x * s[7];
            }
            if constexpr (DEG > 2) {
                // sh_utils.cu:357-376.  The (3xx - yy) factor of the basis-9 term in dy is the
                // reference's (calculus gives 3(xx - yy)); kept so gradients equal the reference's.
                dx[c] += SH_C3[0] * s[9] * 3.0f * 2.0f * xy + SH_C3[1] * s[10] * yz + SH_C3[2] * s[11] * -2.0f * xy +
                         SH_C3[3] * s[12] * -3.0f * 2.0f * xz + SH_C3[4] * s[13] * (-3.0f * xx + 4.0f * zz - yy) +
                         SH_C3[5] * s[14] * 2.0f * xz + SH_C3[6] * s[15] * 3.0f * (xx - yy);
                dy[c] += SH_C3[0] * s[9] * (3.0f * xx - yy) + SH_C3[1] * s[10] * xz + SH_C3[2] * s[11] * (-3.0f * yy + 4.0f * zz - xx) +
                         SH_C3[3] * s[12] * -3.0f * 2.0f * yz + SH_C3[4] * s[13] * -2.0f * xy + SH_C3[5] * s[14] * -2.0f * yz +
                         SH_C3[6] * s[15] * -3.0f * 2.0f * xy;
                dz[c] += SH_C3[1] * s[10] * xy + SH_C3[2] * s[11] * 4.0f * 2.0f * yz + SH_C3[3] * s[12] * 3.0f * (2.0f * zz - xx - yy) +
                         SH_C3[4] * s[13] * 4.0f * 2.0f * xz + SH_C3[5] * s[14] * (xx - yy);
            }
        }
    }
    // (the coefficients have all been read: `o_sh` may be the memory `coeff` points to)
    for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int j = 0; j < K; ++j) o_sh[c * K + j] = b[j] * gr[c];
    f3 ddir = mk3((gr[0] * dx[0] + gr[1] * dx[1]) + gr[2] * dx[2], (gr[0] * dy[0] + gr[1] * dy[1]) + gr[2] * dy[2],
                  (gr[0] * dz[0] + gr[1] * dz[1]) + gr[2] * dz[2]);
    for (int l = 0; l < G; ++l) { // sh_utils.cu:385-405
        const f3 feat = mk3(sg[i * G * 3 + l], sg[i * G * 3 + G + l], sg[i * G * 3 + 2 * G + l]);
        const f3 ax = mk3(axis[(i * G + l) * 3], axis[(i * G + l) * 3 + 1], axis[(i * G + l) * 3 + 2]);
        const float sp = sharp[i * G + l];
        const float dm1 = dot3(mk3(x, y, z), ax) - 1.0f;
        const float wgt = expf(dm1 * sp);
        for (int c = 0; c < 3; ++c) dsg[i * G * 3 + c * G + l] = gr[c] * wgt;
        const float dwgt = dot3(mk3(gr[0], gr[1], gr[2]), feat);
        daxis[(i * G + l) * 3 + 0] = dwgt * sp * x * wgt;
        daxis[(i * G + l) * 3 + 1] = dwgt * sp * y * wgt;
        daxis[(i * G + l) * 3 + 2] = dwgt * sp * z * wgt;
        dsharp[i * G + l] = dwgt * dm1 * wgt;
        ddir = ddir + ax * (dwgt * sp * wgt);
    }
    const float sum2 = dot3(v, v); // sh_utils.cu:406-410: Jacobian of the normalisation
    const float inv32 = 1.0f / sqrtf(sum2 * sum2 * sum2);
    dpos[3 * i + 0] = ((sum2 - v.x * v.x) * ddir.x - v.y * v.x * ddir.y - v.z * v.x * ddir.z) * inv32;
    dpos[3 * i + 1] = (-v.x * v.y * ddir.x + (sum2 - v.y * v.y) * ddir.y - v.z * v.y * ddir.z) * inv32;
    dpos[3 * i + 2] = (-v.x * v.z * ddir.x - v.y * v.z * ddir.y + (sum2 - v.z * v.z) * ddir.z) * inv32;
}

template <int DEG>
__global__ __launch_bounds__(256) void k_sh_bwd(f3 eye, const float *__restrict__ pos, const float *__restrict__ sh,
                                                const float *__restrict__ sg, const float *__restrict__ sharp,
                                                const float *__restrict__ axis, int G, int64_t n,
                                                const float *__restrict__ drgb, float *__restrict__ dsh,
                                                float *__restrict__ dpos, float *__restrict__ dsg,
                                                float *__restrict__ dsharp, float *__restrict__ daxis)
{
    constexpr int K = (DEG + 1) * (DEG + 1);
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    sh_bwd_one<DEG>(eye, pos, sh + i * 3 * K, sg, sharp, axis, G, i, drgb, dsh + i * 3 * K, dpos, dsg, dsharp, daxis);
}

// Degree 3 (48 coefficients, 192 bytes per Gaussian) with the rows of a workgroup's 256 Gaussians staged in LDS: the
// workgroup reads and writes its 48 KiB of coefficients and gradients as consecutive 16-byte pieces, lane after lane,
// instead of 64 lanes each working through a 192-byte row of its own (the same bytes, a quarter of the requests).
// Rows are 13 float4 apart in LDS, so that the 8 lanes an LDS access serves together fall into different banks.
__global__ __launch_bounds__(256) void k_sh_bwd3_rows(f3 eye, const float *__restrict__ pos, const float *__restrict__ sh,
                                                      const float *__restrict__ sg, const float *__restrict__ sharp,
                                                      const float *__restrict__ axis, int G, int64_t n,
                                                      const float *__restrict__ drgb, float *__restrict__ dsh,
                                                      float *__restrict__ dpos, float *__restrict__ dsg,
                                                      float *__restrict__ dsharp, float *__restrict__ daxis)
{
    constexpr int ROW4 = 12, STRIDE4 = 13;
    __shared__ float4 s_rows[256 * STRIDE4];
    const int64_t i0 = (int64_t)blockIdx.x * 256;
    const int rows = (int)(n - i0 < 256 ? n - i0 : 256);
    const float4 *src = (const float4 *)sh + i0 * ROW4;
    for (int g = threadIdx.x; g < rows * ROW4; g += 256) {
        const int r = g / ROW4;
        s_rows[r * STRIDE4 + (g - r * ROW4)] = src[g];
    }
    __syncthreads();
    float *row = (float *)&s_rows[threadIdx.x * STRIDE4];
    if ((int)threadIdx.x < rows) sh_bwd_one<3>(eye, pos, row, sg, sharp, axis, G, i0 + threadIdx.x, drgb, row, dpos, dsg, dsharp, daxis);
    __syncthreads();
    float4 *dst = (float4 *)dsh + i0 * ROW4;
    for (int g = threadIdx.x; g < rows * ROW4; g += 256) {
        const int r = g / ROW4;
        dst[g] = s_rows[r * STRIDE4 + (g - r * ROW4)];
    }
}

// One thread per output record j; reads Gaussian order[j] (or j when order == NULL).
__global__ __launch_bounds__(256) void k_pack(f3 eye, const float *__restrict__ pos, const float *__restrict__ scale,
                                              const float *__restrict__ quat, const float *__restrict__ dens,
                                              const float *__restrict__ rgb, const uint32_t *__restrict__ place, int64_t n,
                                              float thr, Prim *__restrict__ prims)
{
    // in input order: the five arrays are read in whole cache lines, and a record is one 64-byte write wherever it goes
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t j = place ? (int64_t)place[i] : i;
    const float rho = dens[i];
    const float k = sqrtf(2.0f * canon_logf(rho / thr)); // optix_utils.py:288; NaN below the threshold
    Prim p;
    p.pos4 = make_float4(eye.x - pos[3 * i], eye.y - pos[3 * i + 1], eye.z - pos[3 * i + 2], 0.0f);
    p.inv_inter4 = make_float4((1.0f / scale[3 * i]) / k, (1.0f / scale[3 * i + 1]) / k, (1.0f / scale[3 * i + 2]) / k, k);
    p.quat4 = make_float4(quat[4 * i], quat[4 * i + 1], quat[4 * i + 2], quat[4 * i + 3]);
    p.rgba4 = make_float4(rgb[3 * i] * rho, rgb[3 * i + 1] * rho, rgb[3 * i + 2] * rho, rho);
    prims[j] = p;
}

static inline dim3 grid_for(int64_t n, int block) { return dim3((unsigned)((n + block - 1) / block)); }

static int sh_forward_launch(const float *eye, const float *pos, const float *sh, const float *sg, const float *sharp,
                             const float *axis, int32_t g, int32_t degree, int32_t gs, int32_t ks, int64_t n, float *rgb,
                             void *stream)
{
    const DeviceScope on_device(pos);
    if (!eye || n < 0 || degree < 0 || degree > 3 || g < 0 || gs < g || ks < (degree + 1) * (degree + 1) ||
        (n > 0 && (!pos || !sh || !rgb)) || (g > 0 && n > 0 && (!sg || !sharp || !axis)))
        return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    hipStream_t s = (hipStream_t)stream;
    const f3 e = f3{eye[0], eye[1], eye[2]};
    const dim3 grid = grid_for(n, 256), block(256);
    void *span = rgx_span_begin(RGX_T_SH_FWD, s);
    switch (degree) {
    case 0: hipLaunchKernelGGL(k_sh_fwd<0>, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, gs, ks, n, rgb); break;
    case 1: hipLaunchKernelGGL(k_sh_fwd<1>, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, gs, ks, n, rgb); break;
    case 2: hipLaunchKernelGGL(k_sh_fwd<2>, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, gs, ks, n, rgb); break;
    default:
        if (ks == 16 && ((uintptr_t)sh & 15u) == 0)
            hipLaunchKernelGGL(k_sh_fwd3_rows, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, gs, n, rgb);
        else
            hipLaunchKernelGGL(k_sh_fwd<3>, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, gs, ks, n, rgb);
        break;
    }
    rgx_span_end(span, s);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

extern "C" int rgx_sh_forward(const float *eye, const float *pos, const float *sh, const float *sg, const float *sharp,
                              const float *axis, int32_t g, int32_t degree, int64_t n, float *rgb, void *stream)
{
    return sh_forward_launch(eye, pos, sh, sg, sharp, axis, g, degree, g, (degree + 1) * (degree + 1), n, rgb, stream);
}

extern "C" int rgx_sh_viewer(const float *eye, const float *pos, const float *sh, const float *sg, const float *sharp,
                             const float *axis, int32_t g, int32_t degree, int32_t max_num_sh, int32_t max_sg_display,
                             int64_t n, float *rgb, void *stream)
{
    return sh_forward_launch(eye, pos, sh, sg, sharp, axis, g, degree, max_sg_display, max_num_sh, n, rgb, stream);
}

extern "C" int rgx_sh_backward(const float *eye, const float *pos, const float *sh, const float *sg, const float *sharp,
                               const float *axis, int32_t g, int32_t degree, int64_t n, const float *drgb, float *dsh,
                               float *dpos, float *dsg, float *dsharp, float *daxis, void *stream)
{
    const DeviceScope on_device(pos);
    if (!eye || n < 0 || degree < 0 || degree > 3 || g < 0 || (n > 0 && (!pos || !sh || !drgb || !dsh || !dpos)) ||
        (g > 0 && n > 0 && (!sg || !sharp || !axis || !dsg || !dsharp || !daxis)))
        return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    hipStream_t s = (hipStream_t)stream;
    const f3 e = f3{eye[0], eye[1], eye[2]};
    const dim3 grid = grid_for(n, 256), block(256);
#define RGX_SHB(D)                                                                                                      \
    hipLaunchKernelGGL(k_sh_bwd<D>, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, n, drgb, dsh, dpos, dsg, dsharp, \
                       daxis)
    void *span = rgx_span_begin(RGX_T_SH_BWD, s);
    switch (degree) {
    case 0: RGX_SHB(0); break;
    case 1: RGX_SHB(1); break;
    case 2: RGX_SHB(2); break;
    default:
        if ((((uintptr_t)sh | (uintptr_t)dsh) & 15u) == 0)
            hipLaunchKernelGGL(k_sh_bwd3_rows, grid, block, 0, s, e, pos, sh, sg, sharp, axis, g, n, drgb, dsh, dpos, dsg, dsharp, daxis);
        else
            RGX_SHB(3);
        break;
    }
#undef RGX_SHB
    rgx_span_end(span, s);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}

extern "C" int rgx_pack_prims(const void *ws, const float *eye, const float *pos, const float *scale, const float *quat,
                              const float *dens, const float *rgb, int64_t n, float sigma_threshold, float *prims,
                              void *stream)
{
    const DeviceScope on_device(prims);
    if (!eye || n < 0 || (n > 0 && (!pos || !scale || !quat || !dens || !rgb || !prims)) || ((uintptr_t)prims & 15u))
        return RGX_EINVAL;
    if (n == 0) return RGX_OK;
    const uint32_t *place = nullptr; // input index -> sorted position
    if (ws) place = (const uint32_t *)((const char *)ws + rgx_ws_layout(n).vals1);
    void *span = rgx_span_begin(RGX_T_PACK, (hipStream_t)stream);
    hipLaunchKernelGGL(k_pack, grid_for(n, 256), dim3(256), 0, (hipStream_t)stream, f3{eye[0], eye[1], eye[2]}, pos, scale,
                       quat, dens, rgb, place, n, sigma_threshold, (Prim *)prims);
    rgx_span_end(span, (hipStream_t)stream);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}
