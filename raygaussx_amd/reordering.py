"""Morton (z-order) reordering of the point cloud on the GPU.

Replaces ``quantify_pos_min_max`` + ``morton_code`` + ``torch.argsort``
(utils/reordering_utils.py:55-104) as used by ``PointCloud.reorder_zordercurve``
(classes/point_cloud.py:1017-1046) and ``OptimizerManager._reorder_tensors``
(classes/optimizer.py:54-66).
"""
import ctypes as C

import torch

from . import _lib as L
from .optix_utils import _workspace


def morton_order(positions, return_codes=False):
    """Permutation that sorts the points along the 30-bit z-order curve (stable: ties keep input order)."""
    pos = L.f32(positions.detach())
    n, dev = pos.shape[0], pos.device
    ws = _workspace("morton", L.size_query(L.lib().rgx_morton_workspace_bytes, C.c_int64(n)), dev)
    order = torch.empty(n, dtype=torch.int64, device=dev)
    codes = torch.empty(n, dtype=torch.int64, device=dev) if return_codes else None
    L.check(L.lib().rgx_morton_order(L.ptr(pos), C.c_int64(n), L.ptr(codes), L.ptr(order), L.ptr(ws),
                                     C.c_size_t(ws.numel()), L.stream(dev)))
    return (order, codes) if return_codes else order


@torch.no_grad()
def reorder_tensors(order, tensors):
    """Gather every per-Gaussian tensor (parameters, Adam moments, statistics) with one permutation."""
    return [None if t is None else t.index_select(0, order) for t in tensors]
