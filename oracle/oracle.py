"""ctypes front end of the CPU oracle (oracle/rgx_oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by ``__graft_entry__.smoke()``
and by ``bench.py``'s ``cpu_baseline`` leg -- never by the product package.
All arrays are host numpy arrays; nothing here touches a GPU.

``render_forward`` / ``render_backward`` restate the orchestration of
``RenderOptixFunction.forward/backward`` (optix_raycasting/render_optix.py:94-199):
AABB + scene bbox -> SH colour -> prim packing -> march; and for the backward
march -> SH backward -> ``positions_grad += dL_dpos_dir`` (line 185).
"""
import ctypes as C
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liborc.so")

SIGMA_THRESHOLD = 0.1       # cuda_train/forward/gaussians_aabb.h:5
TRANSMITTANCE_EPSILON = 1e-3  # cuda_train/forward/gaussians_aabb.h:4


def build(force=False):
    """Compile liborc.so with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "rgx_oracle.c"))):
        subprocess.check_call(["make", "-B", "-C", _HERE, "liborc.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class OrcCamera(C.Structure):
    _fields_ = [("eye", C.c_float * 3), ("u", C.c_float * 3), ("v", C.c_float * 3),
                ("w", C.c_float * 3), ("tan_x", C.c_float), ("tan_y", C.c_float),
                ("px", C.c_float), ("py", C.c_float), ("width", C.c_int), ("height", C.c_int)]


class OrcMarch(C.Structure):
    _fields_ = [("dt_step", C.c_float), ("dynamic_sampling", C.c_int), ("max_prim_slice", C.c_int),
                ("white_background", C.c_int), ("t_eps", C.c_float)]


class OrcStats(C.Structure):
    _fields_ = [("hit_pairs", C.c_int64), ("slabs", C.c_int64), ("empty_slabs", C.c_int64),
                ("overflow_rays", C.c_int64), ("rays_hit", C.c_int64)]

    def as_dict(self):
        return {k: int(getattr(self, k)) for k, _ in self._fields_}


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_march_trace.restype = C.c_int
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


def set_step_scale(scale):
    """Scale the adaptive step's coefficient 1 / cbrt(T) (1.0: the reference's arithmetic).  A probe
    for how far a last-bit difference in cbrt moves the results of ``dynamic_sampling``."""
    lib().orc_set_step_scale(C.c_float(scale))


def set_backward_mask_form(forward_form):
    """0: the backward's gradient loop decides ``power < k^2`` as the reference's backward does; 1: by the
    forward's arrangement of the same arithmetic (see orc_set_backward_mask_form in rgx_oracle.c)."""
    lib().orc_set_backward_mask_form(C.c_int(int(bool(forward_form))))


def march_backward_in_cut(cam_struct, march, bmin, bmax, prims, ray_colors, ray_ids=None):
    """Per ray (n, 2): samples the backward's gradient loop took as inside a Gaussian's cut-off, and samples on
    which the reference's forward and backward arrangements of ``power`` decide differently."""
    prims, bmin, bmax, ray_colors = _f(prims), _f(bmin), _f(bmax), _f(ray_colors)
    ids = None if ray_ids is None else np.ascontiguousarray(ray_ids, dtype=np.int64)
    n = cam_struct.width * cam_struct.height if ids is None else len(ids)
    out = np.zeros((n, 2), np.int64)
    lib().orc_march_backward_in_cut(C.byref(cam_struct), C.byref(march), _p(bmin), _p(bmax), C.c_int64(prims.shape[0]),
                                    _p(prims), C.c_int64(0 if ids is None else len(ids)), _p(ids), _p(ray_colors), _p(out))
    return out


def cull_build(prims):
    """Build the oracle's optional bounding-volume tree over this primitive block (the timed CPU baseline
    uses it; results are those of the brute force).  Keep ``prims`` alive and pass the same array to the
    march calls; ``cull_free()`` drops the tree."""
    assert prims.dtype == np.float32 and prims.flags["C_CONTIGUOUS"]
    lib().orc_cull_build(C.c_int64(prims.shape[0]), _p(prims))


def cull_free():
    lib().orc_cull_free()


def camera_struct(cam, supersampling=(1, 1)):
    """``cam`` exposes the reference Camera attributes read at optix_utils.py:258-266."""
    c = OrcCamera()
    eye = np.asarray(cam.camera_center, dtype=np.float32).reshape(3)
    wvt = np.asarray(cam.world_view_transform, dtype=np.float32)
    for a in range(3):
        c.eye[a] = eye[a]
        c.u[a] = wvt[a, 0]
        c.v[a] = wvt[a, 1]
        c.w[a] = wvt[a, 2]
    c.tan_x = np.float32(math.tan(cam.FoVx / 2))
    c.tan_y = np.float32(math.tan(cam.FoVy / 2))
    c.px = np.float32(cam.Px)
    c.py = np.float32(cam.Py)
    c.width = int(cam.image_width) * supersampling[0]
    c.height = int(cam.image_height) * supersampling[1]
    return c


def march_struct(dt_step, dynamic_sampling, max_prim_slice, white_background,
                 t_eps=TRANSMITTANCE_EPSILON):
    return OrcMarch(np.float32(dt_step), int(bool(dynamic_sampling)), int(max_prim_slice),
                    int(bool(white_background)), np.float32(t_eps))


def aabb(pos, scale, quat, dens, sigma_thr=SIGMA_THRESHOLD):
    pos, scale, quat, dens = _f(pos), _f(scale), _f(quat), _f(dens)
    N = pos.shape[0]
    boxes = np.empty((N, 6), np.float32)
    bmin = np.empty(3, np.float32)
    bmax = np.empty(3, np.float32)
    lib().orc_aabb(C.c_int64(N), _p(pos), _p(scale), _p(quat), _p(dens), C.c_float(sigma_thr),
                   _p(boxes), _p(bmin), _p(bmax))
    return boxes, bmin, bmax


def pack_prims(eye, pos, scale, quat, dens, rgb, sigma_thr=SIGMA_THRESHOLD):
    eye, pos, scale, quat, dens, rgb = _f(eye), _f(pos), _f(scale), _f(quat), _f(dens), _f(rgb)
    N = pos.shape[0]
    prims = np.empty((N, 16), np.float32)
    with np.errstate(all="ignore"):
        lib().orc_pack_prims(C.c_int64(N), _p(eye), _p(pos), _p(scale), _p(quat), _p(dens), _p(rgb),
                             C.c_float(sigma_thr), _p(prims))
    return prims


def _sg_args(N, sg, sharp, axis):
    G = 0 if sg is None else int(np.asarray(sg).shape[2])
    if G == 0:
        z = np.zeros(1, np.float32)
        return 0, z, z, z
    return G, _f(sg), _f(sharp), _f(axis)


def sh_forward(eye, pos, sh, sg=None, sharp=None, axis=None):
    eye, pos, sh = _f(eye), _f(pos), _f(sh)
    N, _, K = sh.shape
    degree = int(round(math.sqrt(K))) - 1
    G, sg, sharp, axis = _sg_args(N, sg, sharp, axis)
    rgb = np.empty((N, 3), np.float32)
    lib().orc_sh_forward(C.c_int64(N), _p(eye), _p(pos), _p(sh), _p(sg), _p(sharp), _p(axis),
                         C.c_int(G), C.c_int(degree), _p(rgb))
    return rgb


def sh_backward(eye, pos, sh, drgb, sg=None, sharp=None, axis=None, exact_dy9=False):
    eye, pos, sh, drgb = _f(eye), _f(pos), _f(sh), _f(drgb)
    N, _, K = sh.shape
    degree = int(round(math.sqrt(K))) - 1
    G, sg, sharp, axis = _sg_args(N, sg, sharp, axis)
    dsh = np.empty((N, 3, K), np.float32)
    dpos = np.empty((N, 3), np.float32)
    dsg = np.zeros((N, 3, max(G, 1)), np.float32)
    dsharp = np.zeros((N, max(G, 1)), np.float32)
    daxis = np.zeros((N, max(G, 1), 3), np.float32)
    lib().orc_sh_backward(C.c_int64(N), _p(eye), _p(pos), _p(sh), _p(sg), _p(sharp), _p(axis),
                          C.c_int(G), C.c_int(degree), _p(drgb), C.c_int(int(exact_dy9)),
                          _p(dsh), _p(dpos), _p(dsg), _p(dsharp), _p(daxis))
    if G == 0:
        return dsh, dpos, None, None, None
    return dsh, dpos, dsg, dsharp, daxis


def ray_dirs(cam_struct, ray_ids=None):
    n = cam_struct.width * cam_struct.height if ray_ids is None else len(ray_ids)
    ids = None if ray_ids is None else np.ascontiguousarray(ray_ids, dtype=np.int64)
    dirs = np.empty((n, 3), np.float32)
    lib().orc_ray_dirs(C.byref(cam_struct), C.c_int64(n), _p(ids), _p(dirs))
    return dirs


def first_hit(prims, dirs, tlo, thi):
    prims, dirs, tlo, thi = _f(prims), _f(dirs), _f(tlo), _f(thi)
    out = np.empty(dirs.shape[0], np.float32)
    lib().orc_first_hit(C.c_int64(prims.shape[0]), _p(prims), C.c_int64(dirs.shape[0]), _p(dirs),
                        _p(tlo), _p(thi), _p(out))
    return out


def trace_segments(prims, dirs, tlo, thi, cap):
    """Per segment: (count, ids[:count] ascending).  count < 0 means truncated at cap."""
    prims, dirs, tlo, thi = _f(prims), _f(dirs), _f(tlo), _f(thi)
    n = dirs.shape[0]
    counts = np.empty(n, np.int32)
    ids = np.full((n, cap), -1, np.int32)
    lib().orc_trace_segments(C.c_int64(prims.shape[0]), _p(prims), C.c_int64(n), _p(dirs), _p(tlo),
                             _p(thi), C.c_int(cap), _p(counts), _p(ids))
    return counts, ids


def march_forward(cam_struct, march, bmin, bmax, prims, ray_ids=None, out=None):
    prims, bmin, bmax = _f(prims), _f(bmin), _f(bmax)
    R = cam_struct.width * cam_struct.height
    if out is None:
        out = np.zeros((R, 3), np.float32)
    ids = None if ray_ids is None else np.ascontiguousarray(ray_ids, dtype=np.int64)
    st = OrcStats()
    lib().orc_march_forward(C.byref(cam_struct), C.byref(march), _p(bmin), _p(bmax),
                            C.c_int64(prims.shape[0]), _p(prims), C.c_int64(0 if ids is None else len(ids)),
                            _p(ids), _p(out), C.byref(st))
    return out, st.as_dict()


def march_forward_counts(cam_struct, march, bmin, bmax, prims, ray_ids=None):
    """The forward march with its counters kept per ray: (image, counts (n,2) = slabs blended and the
    sum of their hit-list lengths, for the rays of ``ray_ids``)."""
    prims, bmin, bmax = _f(prims), _f(bmin), _f(bmax)
    R = cam_struct.width * cam_struct.height
    out = np.zeros((R, 3), np.float32)
    ids = None if ray_ids is None else np.ascontiguousarray(ray_ids, dtype=np.int64)
    n = R if ids is None else len(ids)
    counts = np.zeros((n, 2), np.int64)
    lib().orc_march_forward_counts(C.byref(cam_struct), C.byref(march), _p(bmin), _p(bmax), C.c_int64(prims.shape[0]),
                                   _p(prims), C.c_int64(n), _p(ids), _p(out), _p(counts))
    return out, counts


def march_trace(cam_struct, march, bmin, bmax, prims, ray, max_slabs=4096, max_ids=1 << 20):
    """Slab-by-slab record of one ray: list of (tbuffer, dt, t_lo, t_hi, ids)."""
    prims, bmin, bmax = _f(prims), _f(bmin), _f(bmax)
    slab_t = np.zeros((max_slabs, 4), np.float32)
    off = np.zeros(max_slabs + 1, np.int32)
    ids = np.zeros(max_ids, np.int32)
    rgb = np.zeros(3, np.float32)
    n = lib().orc_march_trace(C.byref(cam_struct), C.byref(march), _p(bmin), _p(bmax),
                              C.c_int64(prims.shape[0]), _p(prims), C.c_int64(ray), C.c_int(max_slabs),
                              C.c_int(max_ids), _p(slab_t), _p(off), _p(ids), _p(rgb))
    slabs = []
    for s in range(n):
        slabs.append((float(slab_t[s, 0]), float(slab_t[s, 1]), float(slab_t[s, 2]), float(slab_t[s, 3]),
                      ids[off[s]:off[s + 1]].copy()))
    return slabs, rgb


def march_gui(cam_struct, march, bmin, bmax, prims):
    """The viewer's launch: (frame (R,4) uint8, expected depth (R,), unquantised colours (R,3))."""
    prims, bmin, bmax = _f(prims), _f(bmin), _f(bmax)
    R = cam_struct.width * cam_struct.height
    frame = np.zeros((R, 4), np.uint8)
    depth = np.zeros(R, np.float32)
    colors = np.zeros((R, 3), np.float32)
    lib().orc_march_gui(C.byref(cam_struct), C.byref(march), _p(bmin), _p(bmax), C.c_int64(prims.shape[0]),
                        _p(prims), _p(frame), _p(depth), _p(colors))
    return frame, depth, colors


def march_backward(cam_struct, march, bmin, bmax, prims, ray_colors, dloss, ray_ids=None):
    prims, bmin, bmax = _f(prims), _f(bmin), _f(bmax)
    ray_colors, dloss = _f(ray_colors), _f(dloss)
    N = prims.shape[0]
    ids = None if ray_ids is None else np.ascontiguousarray(ray_ids, dtype=np.int64)
    ddens = np.empty(N, np.float32)
    drgb = np.empty((N, 3), np.float32)
    dpos = np.empty((N, 3), np.float32)
    dscale = np.empty((N, 3), np.float32)
    dquat = np.empty((N, 4), np.float32)
    st = OrcStats()
    lib().orc_march_backward(C.byref(cam_struct), C.byref(march), _p(bmin), _p(bmax), C.c_int64(N),
                             _p(prims), C.c_int64(0 if ids is None else len(ids)), _p(ids),
                             _p(ray_colors), _p(dloss), _p(ddens), _p(drgb), _p(dpos), _p(dscale),
                             _p(dquat), C.byref(st))
    return dict(ddens=ddens, drgb=drgb, dpos=dpos, dscale=dscale, dquat=dquat), st.as_dict()


def morton_codes(pos):
    pos = _f(pos)
    codes = np.empty(pos.shape[0], np.int64)
    lib().orc_morton_codes(C.c_int64(pos.shape[0]), _p(pos), _p(codes))
    return codes


def morton_order(pos):
    """Stable argsort of the Morton codes (ties keep input order)."""
    return np.argsort(morton_codes(pos), kind="stable")


# --------------------------------------------------------------------------- #
# Whole-operator restatement (render_optix.py:94-199)
def render_forward(scene, cam, dt_step, dynamic_sampling, max_prim_slice, white_background=True,
                   supersampling=(1, 1), t_eps=TRANSMITTANCE_EPSILON, ray_ids=None, cull=False):
    """scene: dict of numpy arrays positions, scales, quaternions, densities,
    color_features (N,3,K) [+ sph_gauss_features, bandwidth_sharpness, lobe_axis].
    ``cull``: find candidates through the bounding-volume tree (same results, faster on large
    scenes); the tree belongs to this view's primitive block and stays until ``render_backward``
    with the returned context, or ``cull_free()``."""
    cs = camera_struct(cam, supersampling)
    ms = march_struct(dt_step, dynamic_sampling, max_prim_slice, white_background, t_eps)
    eye = np.asarray(cam.camera_center, np.float32)
    _, bmin, bmax = aabb(scene["positions"], scene["scales"], scene["quaternions"], scene["densities"])
    rgb = sh_forward(eye, scene["positions"], scene["color_features"], scene.get("sph_gauss_features"),
                     scene.get("bandwidth_sharpness"), scene.get("lobe_axis"))
    prims = pack_prims(eye, scene["positions"], scene["scales"], scene["quaternions"],
                       scene["densities"], rgb)
    if cull:
        cull_build(prims)
    img, stats = march_forward(cs, ms, bmin, bmax, prims, ray_ids)
    ctx = dict(cs=cs, ms=ms, bmin=bmin, bmax=bmax, rgb=rgb, prims=prims, eye=eye, ray_ids=ray_ids, cull=cull)
    return img, stats, ctx


def render_backward(scene, ctx, ray_colors, dloss):
    g, stats = march_backward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"],
                              ray_colors, dloss, ctx["ray_ids"])
    if ctx.get("cull"):
        cull_free()
    dsh, dpos_dir, dsg, dsharp, daxis = sh_backward(
        ctx["eye"], scene["positions"], scene["color_features"], g["drgb"],
        scene.get("sph_gauss_features"), scene.get("bandwidth_sharpness"), scene.get("lobe_axis"))
    out = dict(positions=g["dpos"] + dpos_dir, scales=g["dscale"], quaternions=g["dquat"],
               densities=g["ddens"], color_features=dsh, sph_gauss_features=dsg,
               bandwidth_sharpness=dsharp, lobe_axis=daxis, rgb=g["drgb"])
    return out, stats


def dist2_knn3(pos):
    """distCUDA2: mean squared distance to the three nearest other points (brute force)."""
    pos = _f(pos)
    out = np.empty(pos.shape[0], np.float32)
    lib().orc_dist2_knn3(C.c_int64(pos.shape[0]), _p(pos), _p(out))
    return out


def reduce_supersampling(target_width, target_height, ray_colors, factor):
    """utils/general_utils.py:489-502, restated with the same slicing and summation order."""
    fx, fy = factor
    ray_colors = np.asarray(ray_colors, np.float32)
    s = ray_colors[0::fx].copy()
    for i in range(1, fx):
        s += ray_colors[i::fx]
    s = s.reshape((target_height * fy, target_width, 3))
    m = s[0::fy].copy()
    for i in range(1, fy):
        m += s[i::fy]
    return m / np.float32(fx * fy)
