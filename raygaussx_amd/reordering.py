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
    """Gathers every per-Gaussian tensor (parameters, Adam moments, statistics) with one
    permutation in one launch: ``[t[order] for t in tensors]`` (``None`` entries pass through).
    Tensors must have 4- or 8-byte elements (rows that are multiples of 4 bytes)."""
    order = order.to(torch.int64).contiguous()
    n = order.shape[0]
    live = [t for t in tensors if t is not None]
    if not live:
        return list(tensors)
    srcs, dsts = [], []
    for t in live:
        if t.shape[0] != n:
            raise L.RgxError("reorder_tensors: a tensor's first dimension differs from the permutation's length")
        if not t.is_cuda or (t[0].numel() * t.element_size()) % 4 if n else False:
            raise L.RgxError("reorder_tensors needs device tensors whose rows are multiples of 4 bytes")
        srcs.append(t.detach().contiguous())
        dsts.append(torch.empty_like(srcs[-1]))
    m = len(srcs)
    if n:
        src_p = (C.c_void_p * m)(*[s.data_ptr() for s in srcs])
        dst_p = (C.c_void_p * m)(*[d.data_ptr() for d in dsts])
        rows = (C.c_int64 * m)(*[s[0].numel() * s.element_size() for s in srcs])
        L.check(L.lib().rgx_gather_rows(C.c_int32(m), src_p, dst_p, rows, L.ptr(order), C.c_int64(n), L.stream(order.device)))
    it = iter(dsts)
    return [None if t is None else next(it) for t in tensors]
