"""Host mirror of the simple-knn extension's one function (submodules/simple-knn/ext.cpp:
``from simple_knn._C import distCUDA2``), used to initialise the Gaussians' scales
(classes/point_cloud.py:252)."""
import ctypes as C

import torch

from . import _lib as L
from .optix_utils import _workspace


def distCUDA2(points):
    """Mean squared distance of every point to its three nearest neighbours, ``(N,)`` float32."""
    pts = L.f32(points.detach())
    if pts.dim() != 2 or pts.shape[1] != 3:
        raise L.RgxError("distCUDA2 needs an (N, 3) tensor")
    n, dev = pts.shape[0], pts.device
    ws = _workspace("knn", L.size_query(L.lib().rgx_knn_workspace_bytes, C.c_int64(n)), dev)
    out = torch.empty(n, dtype=torch.float32, device=dev)
    L.check(L.lib().rgx_dist2_knn3(L.ptr(pts), C.c_int64(n), L.ptr(out), L.ptr(ws), C.c_size_t(ws.numel()), L.stream(dev)))
    return out
