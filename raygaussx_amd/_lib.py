"""ctypes binding of librgx.so (the C ABI declared in include/rgx.h).

The library is the product path: if it is missing or a call fails this module
raises -- there is no CPU or PyTorch fallback.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# RGX_LIB_PATH selects another build of the same library (e.g. one compiled with extra flags)
LIB_PATH = os.environ.get("RGX_LIB_PATH") or os.path.join(_HERE, "librgx.so")


class RgxError(RuntimeError):
    pass


class RgxCamera(C.Structure):
    _fields_ = [("eye", C.c_float * 3), ("u", C.c_float * 3), ("v", C.c_float * 3), ("w", C.c_float * 3),
                ("tan_half_fov_x", C.c_float), ("tan_half_fov_y", C.c_float), ("principal_x", C.c_float),
                ("principal_y", C.c_float), ("width", C.c_int32), ("height", C.c_int32)]


class RgxMarch(C.Structure):
    _fields_ = [("dt_step", C.c_float), ("dynamic_sampling", C.c_int32), ("max_prim_slice", C.c_int32),
                ("white_background", C.c_int32), ("t_eps", C.c_float), ("record_format", C.c_int32)]


STATS_FIELDS = ("hit_pairs", "slabs", "empty_slabs", "overflow_rays", "rays_hit", "nodes_visited", "candidates",
                "candidates_hit", "replay_lost", "grad_atomics")

ABI_VERSION = 6   # RGX_ABI_VERSION of include/rgx.h

# every symbol include/rgx.h declares
SYMBOLS = ("rgx_abi_version", "rgx_strerror", "rgx_last_hip_error", "rgx_aabb", "rgx_sh_forward",
           "rgx_sh_backward", "rgx_build_workspace_bytes", "rgx_build", "rgx_build_aabbs", "rgx_refit_aabbs", "rgx_scene_bbox",
           "rgx_build_order", "rgx_build_layout", "rgx_pack_prims", "rgx_march_workspace_bytes", "rgx_march_records_bytes", "rgx_march_forward", "rgx_march_forward_counts",
           "rgx_march_backward", "rgx_march_backward_noalloc", "rgx_march_faults", "rgx_first_hit", "rgx_trace_segments", "rgx_collect_tiles", "rgx_morton_workspace_bytes",
           "rgx_morton_order", "rgx_sh_viewer", "rgx_march_viewer", "rgx_gather_rows", "rgx_knn_workspace_bytes", "rgx_dist2_knn3", "rgx_reduce_supersampling", "rgx_check_plain_arith", "rgx_probe_valu_rate", "rgx_timing_enable", "rgx_timing_reset", "rgx_timing_name", "rgx_timing_read")

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RgxError(f"{LIB_PATH} is not built; run `python -m raygaussx_amd.build` "
                           "(there is no fallback path)")
        _lib = C.CDLL(LIB_PATH)
        _lib.rgx_strerror.restype = C.c_char_p
        _lib.rgx_timing_name.restype = C.c_char_p
        for name in SYMBOLS:
            getattr(_lib, name)  # fail at load time if the library is stale
        if _lib.rgx_abi_version() != ABI_VERSION:
            got, _lib = _lib.rgx_abi_version(), None
            raise RgxError(f"{LIB_PATH} has ABI version {got}, this binding needs {ABI_VERSION}; rebuild it")
    return _lib


def check(rc):
    if rc != 0:
        l = lib()
        msg = l.rgx_strerror(rc).decode()
        if rc == -3:
            msg += f" [hipError_t {l.rgx_last_hip_error()}]"
        raise RgxError(f"librgx: {msg} ({rc})")


def ptr(t):
    """Device pointer of a contiguous tensor; NULL for None / empty tensors."""
    if t is None or t.numel() == 0:
        return C.c_void_p(0)
    if not t.is_contiguous():
        raise RgxError("librgx needs contiguous tensors")
    return C.c_void_p(t.data_ptr())


def stream(device=None):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def f32(t):
    if t.dtype != torch.float32:
        raise RgxError(f"librgx needs float32 tensors, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def host3(t):
    """Three host floats from a tensor / sequence (one small D2H copy if it lives on the GPU)."""
    if isinstance(t, torch.Tensor):
        t = t.detach().reshape(-1).to("cpu", torch.float32).tolist()
    return (C.c_float * 3)(*[float(x) for x in t][:3])


def size_query(fn, *args):
    out = C.c_size_t(0)
    check(fn(*args, C.byref(out)))
    return int(out.value)


def timing_enable(on=True):
    check(lib().rgx_timing_reset())
    check(lib().rgx_timing_enable(int(bool(on))))


def timing_read():
    """{kernel name: (total milliseconds, launches)} since timing was enabled."""
    out = {}
    i = 0
    while True:
        name = lib().rgx_timing_name(i)
        if not name:
            break
        ms, cnt = C.c_double(0), C.c_int64(0)
        check(lib().rgx_timing_read(i, C.byref(ms), C.byref(cnt)))
        out[name.decode()] = (ms.value, cnt.value)
        i += 1
    return out
