// Image epilogue of the inference loop: average the supersampled rays of each pixel
// (utils/general_utils.py:489-502 reduce_supersampling), optionally clip to [0, 1]
// (scripts/test.py:200 `.clip(0,1)`) and quantise to 8 bits (`np.uint8(255*arr)`,
// utils/general_utils.py:167).  One thread per output pixel; the sums run in the reference's
// order -- along x first, then along y, one division at the end -- so the floats are its floats.
#include "rgx_device.h"

__global__ __launch_bounds__(256) void k_reduce_supersampling(const float *__restrict__ rays, int width, int height, int fx,
                                                              int fy, int clip, float *__restrict__ out,
                                                              uint8_t *__restrict__ out8)
{
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= (int64_t)width * height) return;
    const int x = (int)(p % width), y = (int)(p / width);
    const int64_t row_stride = (int64_t)width * fx; // rays per supersampled row
    float acc[3] = {0.f, 0.f, 0.f};
    for (int j = 0; j < fy; ++j) {
        const float *r = rays + 3 * (((int64_t)y * fy + j) * row_stride + (int64_t)x * fx);
        float sx[3] = {r[0], r[1], r[2]};
        for (int i = 1; i < fx; ++i)
            for (int c = 0; c < 3; ++c) sx[c] += r[3 * i + c];
        for (int c = 0; c < 3; ++c) acc[c] = j == 0 ? sx[c] : acc[c] + sx[c];
    }
    const float div = (float)(fx * fy);
    for (int c = 0; c < 3; ++c) {
        float v = acc[c] / div;
        if (clip) v = fminf(fmaxf(v, 0.0f), 1.0f);
        if (out) out[3 * p + c] = v;
        if (out8) out8[3 * p + c] = (uint8_t)(255.0f * fminf(fmaxf(v, 0.0f), 1.0f));
    }
}

extern "C" int rgx_reduce_supersampling(const float *ray_colors, int32_t width, int32_t height, int32_t factor_x,
                                        int32_t factor_y, int32_t clip, float *out, uint8_t *out8, void *stream)
{
    const DeviceScope on_device(ray_colors);
    if (width <= 0 || height <= 0 || factor_x <= 0 || factor_y <= 0 || !ray_colors || (!out && !out8)) return RGX_EINVAL;
    const int64_t n = (int64_t)width * height;
    hipLaunchKernelGGL(k_reduce_supersampling, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, ray_colors, width, height,
                       factor_x, factor_y, clip, out, out8);
    RGX_LAUNCH_CHECK();
    return RGX_OK;
}
