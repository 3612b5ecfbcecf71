"""Host mirror of the image helpers the inference loop calls after the renderer
(utils/general_utils.py:489-502, scripts/test.py:197-200)."""
import ctypes as C

import torch

from . import _lib as L


def reduce_supersampling(target_width, target_height, ray_colors, factor, clip=False, to_uint8=False):
    """utils/general_utils.py:489-502: the mean over each pixel's ``factor = (fx, fy)`` rays,
    ``(target_height, target_width, 3)``.  ``clip`` folds in the ``.clip(0, 1)`` of
    scripts/test.py:200; ``to_uint8`` returns ``uint8(255 * clipped)`` as well (second result)."""
    fx, fy = int(factor[0]), int(factor[1])
    ray_colors = L.f32(ray_colors)
    if ray_colors.numel() != target_width * fx * target_height * fy * 3:
        raise L.RgxError("reduce_supersampling: ray_colors does not hold (W*fx)*(H*fy) rays")
    dev = ray_colors.device
    out = torch.empty(target_height, target_width, 3, dtype=torch.float32, device=dev)
    out8 = torch.empty(target_height, target_width, 3, dtype=torch.uint8, device=dev) if to_uint8 else None
    L.check(L.lib().rgx_reduce_supersampling(L.ptr(ray_colors), C.c_int32(target_width), C.c_int32(target_height),
                                             C.c_int32(fx), C.c_int32(fy), C.c_int32(int(bool(clip))), L.ptr(out),
                                             L.ptr(out8), L.stream(dev)))
    return (out, out8) if to_uint8 else out
