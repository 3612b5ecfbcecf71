"""Host launch glue with the names and argument meaning of the reference's
``optix_raycasting/optix_utils.py``, implemented on librgx (HIP, gfx950).

What was an OptiX object in the reference is an inert handle here (context,
module, program groups, pipeline, SBT): the kernels are compiled ahead of time
into librgx.so, so those constructors only exist to keep caller code unchanged.
The acceleration structure is real: an LBVH held in a torch byte tensor.
"""
import ctypes as C
import math

import torch

from . import _lib as L

SIGMA_THRESHOLD = 0.1            # cuda_train/forward/gaussians_aabb.h:5
TRANSMITTANCE_EPSILON = 1e-3     # cuda_train/forward/gaussians_aabb.h:4

_scratch = {}          # (key, device, stream handle) -> byte tensor, most recently used last
_SCRATCH_STREAMS = 8   # scratch sets kept per key and device: one per stream in use; older ones are dropped


def _workspace(key, nbytes, device):
    """Cached byte tensor (grown, never shrunk) -- keeps the hot path free of allocations.  One per
    stream: views rendered on different streams run concurrently and must not share scratch memory.
    A loop that keeps creating streams does not accumulate them: per key and device only the
    ``_SCRATCH_STREAMS`` most recently used streams keep their tensor (a dropped tensor's memory goes
    back to torch's allocator, which keeps it alive for work already queued on its stream)."""
    slot = (key, str(device), torch.cuda.current_stream(device).cuda_stream)
    t = _scratch.pop(slot, None)
    if t is None or t.numel() < nbytes:
        t = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=device)   # zeroed: the fault counters start at 0
    _scratch[slot] = t          # re-inserted: dicts keep insertion order, so this is now the newest
    mine = [k for k in _scratch if k[0] == key and k[1] == str(device)]
    for k in mine[:-_SCRATCH_STREAMS]:
        del _scratch[k]
    return t


class _Handle:
    """Stands in for an OptiX context / module / program group / pipeline / SBT."""

    def __init__(self, kind, **kw):
        self.kind = kind
        self.__dict__.update(kw)

    cache_enabled = False


class AccelerationStructure:
    """LBVH over the Gaussians' k-sigma boxes (replaces ``ox.AccelerationStructure``)."""

    def __init__(self, n, device):
        self.n = int(n)
        self.device = device
        self.built = False      # a build has been queued into ``ws``: only then is there a tree to refit
        nbytes = L.size_query(L.lib().rgx_build_workspace_bytes, C.c_int64(self.n))
        self.ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        self.ws[:256].zero_()   # the header: "not built" until a build has finished

    @property
    def handle(self):
        return self.ws.data_ptr()

    def build_from_gaussians(self, positions, scales, quaternions, densities):
        L.check(L.lib().rgx_build(L.ptr(positions), L.ptr(scales), L.ptr(quaternions), L.ptr(densities),
                                  C.c_int64(self.n), C.c_float(SIGMA_THRESHOLD), L.ptr(self.ws),
                                  C.c_size_t(self.ws.numel()), L.stream(self.device)))
        self.built = True
        return self

    def build_from_boxes(self, bboxes):
        bboxes = L.f32(bboxes)
        if tuple(bboxes.shape) != (self.n, 6):
            raise L.RgxError(f"librgx: {self.n} boxes expected as an ({self.n}, 6) tensor, got {tuple(bboxes.shape)}")
        L.check(L.lib().rgx_build_aabbs(L.ptr(bboxes), C.c_int64(self.n), L.ptr(self.ws),
                                        C.c_size_t(self.ws.numel()), L.stream(self.device)))
        self.built = True
        return self

    def update(self, bboxes):
        """New boxes for the same Gaussians: refit (the tree keeps its shape), as OptiX's accel update does.
        Only a structure that was built can be updated, and only with one box per Gaussian of that build: the
        refit walks the tree the build left in the workspace."""
        if not self.built:
            raise L.RgxError("librgx: update of an acceleration structure that was never built")
        bboxes = L.f32(bboxes)
        if tuple(bboxes.shape) != (self.n, 6) or bboxes.device != self.ws.device:
            raise L.RgxError(f"librgx: update needs an ({self.n}, 6) tensor of boxes on {self.ws.device}, got "
                             f"{tuple(bboxes.shape)} on {bboxes.device}")
        L.check(L.lib().rgx_refit_aabbs(L.ptr(bboxes), C.c_int64(self.n), L.ptr(self.ws), C.c_size_t(self.ws.numel()),
                                        L.stream(self.device)))
        return self

    def scene_bbox(self):
        out = (C.c_float * 6)()
        L.check(L.lib().rgx_scene_bbox(L.ptr(self.ws), out, L.stream(self.device)))
        return list(out[:3]), list(out[3:])

    def order(self):
        out = torch.empty(self.n, dtype=torch.int32, device=self.device)
        L.check(L.lib().rgx_build_order(L.ptr(self.ws), C.c_int64(self.n), L.ptr(out), L.stream(self.device)))
        return out


def ellipsoids_bbox_from_quat(quaternions, centers, scales, densities):
    """optix_utils.py:82-109 -> (bboxes (N,6), bb_min (3), bb_max (3)), device tensors."""
    q, c, s, d = (L.f32(t) for t in (quaternions, centers, scales, densities))
    n = c.shape[0]
    boxes = torch.empty(n, 6, dtype=torch.float32, device=c.device)
    bb = torch.empty(2, 3, dtype=torch.float32, device=c.device)
    L.check(L.lib().rgx_aabb(L.ptr(c), L.ptr(s), L.ptr(q), L.ptr(d), C.c_int64(n), C.c_float(SIGMA_THRESHOLD),
                             L.ptr(boxes), C.c_void_p(bb[0].data_ptr()), C.c_void_p(bb[1].data_ptr()),
                             L.stream(c.device)))
    return boxes, bb[0], bb[1]


def quaternion_to_rotation(quaternion):
    """optix_utils.py:111-123: rows of the rotation matrix of (w,x,y,z)."""
    w, x, y, z = quaternion.unbind(1)
    L1 = torch.stack([1 - 2 * (y ** 2 + z ** 2), 2 * (x * y - w * z), 2 * (x * z + w * y)], 1)
    L2 = torch.stack([2 * (x * y + w * z), 1 - 2 * (x ** 2 + z ** 2), 2 * (y * z - w * x)], 1)
    L3 = torch.stack([2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x ** 2 + y ** 2)], 1)
    return L1, L2, L3


def compute_ellipsoids_bbox(centers, scales, L1, L2, L3, densities):
    """optix_utils.py:125-137 (the legacy box routine scripts/test.py:65-66 calls)."""
    delta = torch.log((densities / SIGMA_THRESHOLD) ** 2).clamp_min(0).sqrt()
    ext = torch.stack([torch.linalg.norm(delta[:, None] * scales * Li, dim=1) for Li in (L1, L2, L3)], 1)
    return torch.cat([centers - ext, centers + ext], 1).float().contiguous()


def create_acceleration_structure(ctx, bboxes):
    """optix_utils.py:139-142: a fresh acceleration structure over (N,6) boxes."""
    bboxes = L.f32(bboxes)
    return AccelerationStructure(bboxes.shape[0], bboxes.device).build_from_boxes(bboxes)


def update_acceleration_structure(gas, bboxes):
    """optix_utils.py:144-146: refit of an existing acceleration structure to new boxes."""
    gas.update(bboxes)


def create_context(log=None):
    return _Handle("context", log=log)


def create_module(ctx, pipeline_opts, stage, debug_level=None, opt_level=None):
    """optix_utils.py:148-178.  "gui" stands for the viewer's kernels (``march_viewer``, ``sh_viewer``)."""
    if stage not in ("forward", "backward", "test", "gui"):
        raise ValueError("stage must be 'forward', 'backward', 'test' or 'gui'")
    L.lib()  # make a missing library surface here, like a failed module compile would
    return _Handle("module", stage=stage)


def create_program_groups(ctx, module):
    return [_Handle("program_group", stage=module.stage, index=i) for i in range(5)]


def create_pipeline(ctx, program_grps, pipeline_options, debug_level=None):
    return _Handle("pipeline", stage=program_grps[0].stage)


def create_sbt(program_grps):
    return _Handle("sbt")


# ---------------------------------------------------------------------------
def camera_struct(camera, supersampling=(1, 1)):
    """Launch constants read from a Camera (optix_utils.py:258-266).  The host copies of the
    camera tensors are cached on the camera object, so repeated views cost no device sync."""
    host = getattr(camera, "_rgx_host", None)
    if host is None:
        eye = camera.camera_center.detach().reshape(-1).to("cpu", torch.float32).tolist()
        wvt = camera.world_view_transform.detach().to("cpu", torch.float32)
        host = (eye, wvt[:3, 0].tolist(), wvt[:3, 1].tolist(), wvt[:3, 2].tolist())
        try:
            camera._rgx_host = host
        except AttributeError:
            pass
    c = L.RgxCamera()
    for a in range(3):
        c.eye[a], c.u[a], c.v[a], c.w[a] = host[0][a], host[1][a], host[2][a], host[3][a]
    c.tan_half_fov_x = math.tan(camera.FoVx / 2)
    c.tan_half_fov_y = math.tan(camera.FoVy / 2)
    c.principal_x = camera.Px
    c.principal_y = camera.Py
    c.width = int(camera.image_width) * int(supersampling[0])
    c.height = int(camera.image_height) * int(supersampling[1])
    return c


def pack_prims(gas, camera_or_eye, positions, scales, quaternions, densities, rgb, out=None):
    """The (N,16) PrimData block of optix_utils.py:268-304, in the acceleration structure's order."""
    n = positions.shape[0]
    eye = camera_or_eye.eye if isinstance(camera_or_eye, L.RgxCamera) else L.host3(camera_or_eye)
    if out is None:
        out = torch.empty(n, 16, dtype=torch.float32, device=positions.device)
    L.check(L.lib().rgx_pack_prims(L.ptr(gas.ws) if gas is not None else C.c_void_p(0), eye, L.ptr(positions),
                                   L.ptr(scales), L.ptr(quaternions), L.ptr(densities), L.ptr(rgb), C.c_int64(n),
                                   C.c_float(SIGMA_THRESHOLD), L.ptr(out), L.stream(positions.device)))
    return out


def _march_ws(n, n_rays, max_prim_slice, device):
    nbytes = L.size_query(L.lib().rgx_march_workspace_bytes, C.c_int64(n), C.c_int64(n_rays),
                          C.c_int32(max_prim_slice))
    return _workspace("march", nbytes, device)


# Record size per 8x8 pixel tile, 32-bit words: 16384 for the hit lists (64 KiB) and on average 64
# slots of 8192 words for the per-sample density and colour sums of a slab iteration (the slots are
# one pool shared by all tiles).  2.06 MiB per tile: 21 GB at 800x800.  16384 keeps the hit lists only.
# This is the most a record holds; what a launch is given is sized from use (new_records).
REC_TILE_WORDS = 16384 + 64 * 8192
# The first view of a scene size and image shape on a stream, of which nothing is known yet, gets a pool of
# this many slots per tile: its forward counts the slots it would have used, tiles that find the pool empty
# are replayed from their hit lists (slower, same gradients), and the second view's pool is sized from the count.
REC_FIRST_SLOTS = 12


REC_LIST_WORDS = 16384        # the hit lists' share of a tile's record
REC_SLOT_WORDS = 8192         # one slot of sample sums
REC_SLOT_WORDS_HALF = 2048 + 2 * 24 * 64 + 2 * 64   # ... with half-precision colour sums (record_format 1)
REC_MEMORY_SHARE = 0.4        # of the device's memory: the most a record may take by default


def records_bytes(cam, tile_words):
    return L.size_query(L.lib().rgx_march_records_bytes, C.c_int32(cam.width), C.c_int32(cam.height), C.c_int32(tile_words))


def fit_tile_words(cam, tile_words, budget_bytes):
    """The record size per tile that fits ``budget_bytes``: ``tile_words`` if it does; else the hit
    lists plus as many sample-sum slots per tile as fit (tiles that find the pool empty are replayed
    from their lists); else the hit lists alone; 0 when not even those fit (no record)."""
    if records_bytes(cam, tile_words) <= budget_bytes:
        return tile_words
    lists = min(tile_words, REC_LIST_WORDS)
    if records_bytes(cam, lists) > budget_bytes:
        return 0
    ntiles = ((cam.width + 7) // 8) * ((cam.height + 7) // 8)
    slots = (budget_bytes // (4 * ntiles) - lists) // REC_SLOT_WORDS
    return lists + slots * REC_SLOT_WORDS if (tile_words > lists and slots >= 1) else lists


# What the forward launches of one scene size and image shape on one stream asked of the sample-sum pool
# (the launch's whole demand: every blending slab iteration asks, served or not), so that the next record
# is allocated for the need:
# (device, stream, Gaussians, width, height) -> {"pinned": host int32[1], "event", "pending", "need": slots the
#                             last views asked for, "slots": the pool size in use, "allocated": bytes of the last record}
_rec_usage = {}
REC_POOL_MARGIN = 1.05        # pool = this times the largest need of the last views ...
REC_POOL_STEP = 1 << 12       # ... rounded up to a multiple of this many slots (128 MiB), so that the size stays put
REC_POOL_HISTORY = 8


def _usage_key(cam, device, n, record_format=0):
    return (str(device), torch.cuda.current_stream(device).cuda_stream, int(n), cam.width, cam.height, int(record_format))


def _slot_words(record_format):
    return REC_SLOT_WORDS_HALF if record_format == 1 else REC_SLOT_WORDS


def _pool_geometry(cam):
    ntiles = ((cam.width + 7) // 8) * ((cam.height + 7) // 8)
    return ntiles, ntiles * REC_LIST_WORDS * 4        # tiles, bytes of the hit-list regions (the pool header follows)


def new_records(cam, device, tile_words=REC_TILE_WORDS, budget_bytes=None, n=0, record_format=0):
    """Buffer for the record of one forward launch (see rgx_march_records_bytes), or None when no
    record fits the budget or the allocator.  The budget defaults to REC_MEMORY_SHARE of the device's
    memory and at most 80 % of what is free now.  With the default ``tile_words`` the pool of sample
    sums is sized from what the last forward launches of this scene size (``n`` Gaussians) and image
    shape on this stream asked for (``note_record_use``); the first such view, of which nothing is
    known, gets REC_FIRST_SLOTS slots per tile.  Tiles that find the pool empty are replayed from
    their hit lists alone, so a pool that is too small costs time, not correctness, and the forward's
    count of what it would have used sizes the next one."""
    if budget_bytes is None:
        free, total = torch.cuda.mem_get_info(device)
        budget_bytes = int(min(REC_MEMORY_SHARE * total, 0.8 * free))
    if tile_words == REC_TILE_WORDS:
        key = _usage_key(cam, device, n, record_format)
        use = _rec_usage.get(key)
        if use is None:
            if len(_rec_usage) >= 64:
                del _rec_usage[next(iter(_rec_usage))]
            use = _rec_usage[key] = dict(pinned=torch.zeros(1, dtype=torch.int32).pin_memory(), event=torch.cuda.Event(),
                                         pending=False, need=[], slots=0, allocated=0)
        if use["pending"] and not use["need"]:
            use["event"].synchronize()     # the second view of a key waits for the first view's count: once per key
        _read_record_use(use)
        ntiles, head = _pool_geometry(cam)
        have = use["slots"]
        if use["need"]:
            want = int(max(use["need"]) * REC_POOL_MARGIN) + 1
            if want > have or want * 1.5 < have:      # grow when short; shrink only when far too large
                have = (want + REC_POOL_STEP - 1) // REC_POOL_STEP * REC_POOL_STEP
        elif not have:
            have = REC_FIRST_SLOTS * ntiles
        have = max(min(have, 64 * ntiles), ntiles)     # (the library wants at least one slot per tile to keep sums at all)
        nbytes = max(head + 256 + have * _slot_words(record_format) * 4, ntiles * (REC_LIST_WORDS + REC_SLOT_WORDS) * 4)
        if nbytes <= budget_bytes:
            try:
                rec = torch.empty(nbytes, dtype=torch.uint8, device=device)
                use["slots"] = have
                return rec
            except torch.cuda.OutOfMemoryError:
                pass
    words = fit_tile_words(cam, tile_words, budget_bytes)
    while words:
        try:
            return torch.empty(records_bytes(cam, words), dtype=torch.uint8, device=device)
        except torch.cuda.OutOfMemoryError:
            words = REC_LIST_WORDS if words > REC_LIST_WORDS else 0   # try the hit lists alone, then give up
    return None


def _read_record_use(use):
    if use["pending"] and use["event"].query():
        use["pending"] = False
        use["need"] = (use["need"] + [int(use["pinned"][0])])[-REC_POOL_HISTORY:]


def note_record_use(records, cam, device, n=0, record_format=0):
    """After a forward launch that wrote ``records``: queue a 4-byte copy of the pool's bump counter
    (the slots the launch asked for, also beyond the pool's end) to pinned host memory.  Nothing waits
    for it; the next ``new_records`` of this scene size and image shape on this stream reads it."""
    ntiles, head = _pool_geometry(cam)
    use = _rec_usage.get(_usage_key(cam, device, n, record_format))
    # (the library keeps sample sums only in a record with room for the hit lists and at least one slot per tile)
    if use is None or records is None or records.numel() // 4 // ntiles < REC_LIST_WORDS + REC_SLOT_WORDS:
        return
    use["allocated"] = records.numel()
    _read_record_use(use)
    if use["pending"]:
        return                                  # the previous copy has not landed yet: leave its buffer alone
    use["pinned"].copy_(records[head:head + 4].view(torch.int32), non_blocking=True)
    use["event"].record(torch.cuda.current_stream(device))
    use["pending"] = True


def record_use(cam, device, n=0, record_format=0):
    """(bytes allocated for the last record of this scene size and image shape on this stream, bytes the last
    launch read back asked for: hit-list regions + sample-sum slots), or None before the first launch has reported."""
    use = _rec_usage.get(_usage_key(cam, device, n, record_format))
    if use is None:
        return None
    _read_record_use(use)
    if not use["need"]:
        return None
    ntiles, head = _pool_geometry(cam)
    return use["allocated"], head + 256 + use["need"][-1] * _slot_words(record_format) * 4


def march_forward(gas, cam, prims, dt_step, dynamic_sampling, max_prim_slice, white_background,
                  t_eps=TRANSMITTANCE_EPSILON, stats=None, records=None, ray_counts=False, record_format=0):
    """``ray_counts=True`` (test hook): also returns an (n_rays, 2) int32 tensor, per ray the slabs blended and
    the sum of their hit-list lengths."""
    n, dev = prims.shape[0], prims.device
    n_rays = cam.width * cam.height
    m = L.RgxMarch(dt_step, int(bool(dynamic_sampling)), int(max_prim_slice), int(bool(white_background)), t_eps, int(record_format))
    ws = _march_ws(n, n_rays, max_prim_slice, dev)
    ray_colors = torch.empty(n_rays, 3, dtype=torch.float32, device=dev)
    if ray_counts:
        counts = torch.zeros(n_rays, 2, dtype=torch.int32, device=dev)
        L.check(L.lib().rgx_march_forward_counts(L.ptr(gas.ws), C.byref(cam), C.byref(m), L.ptr(prims), C.c_int64(n),
                                                 L.ptr(ray_colors), L.ptr(ws), C.c_size_t(ws.numel()), L.ptr(records),
                                                 C.c_size_t(0 if records is None else records.numel()), L.ptr(stats),
                                                 L.ptr(counts), L.stream(dev)))
        return ray_colors, counts
    L.check(L.lib().rgx_march_forward(L.ptr(gas.ws), C.byref(cam), C.byref(m), L.ptr(prims), C.c_int64(n),
                                      L.ptr(ray_colors), L.ptr(ws), C.c_size_t(ws.numel()), L.ptr(records),
                                      C.c_size_t(0 if records is None else records.numel()), L.ptr(stats),
                                      L.stream(dev)))
    return ray_colors


def march_viewer(gas, cam, prims, dt_step, dynamic_sampling, max_prim_slice, t_eps=TRANSMITTANCE_EPSILON, stats=None):
    """The interactive viewer's launch (cuda_gui/gaussians_aabb.cu): ``(frame (H, W, 4) uint8, depth (H, W))``,
    black background, colours quantised as the viewer does, expected depth per ray."""
    n, dev = prims.shape[0], prims.device
    m = L.RgxMarch(dt_step, int(bool(dynamic_sampling)), int(max_prim_slice), 0, t_eps)
    ws = _march_ws(n, cam.width * cam.height, max_prim_slice, dev)
    frame = torch.empty(cam.height, cam.width, 4, dtype=torch.uint8, device=dev)
    depth = torch.empty(cam.height, cam.width, dtype=torch.float32, device=dev)
    L.check(L.lib().rgx_march_viewer(L.ptr(gas.ws), C.byref(cam), C.byref(m), L.ptr(prims), C.c_int64(n), L.ptr(frame),
                                     L.ptr(depth), L.ptr(ws), C.c_size_t(ws.numel()), L.ptr(stats), L.stream(dev)))
    return frame, depth


def sh_viewer(camera_center, positions, sh, sph_gauss_features, bandwidth_sharpness, lobe_axis, num_sph_gauss,
              sh_degree, max_num_sh, max_sg_display):
    """gui_sh (utils/sh_utils.cu:25-119): per-Gaussian colour from tensors that keep room for ``max_num_sh``
    coefficients per channel and ``max_sg_display`` lobes, evaluating the first ``(sh_degree+1)^2`` and
    ``num_sph_gauss`` of them."""
    n = positions.shape[0]
    rgb = torch.empty(n, 3, dtype=torch.float32, device=positions.device)
    L.check(L.lib().rgx_sh_viewer(L.host3(camera_center), L.ptr(L.f32(positions)), L.ptr(L.f32(sh)),
                                  L.ptr(sph_gauss_features), L.ptr(bandwidth_sharpness), L.ptr(lobe_axis),
                                  C.c_int32(num_sph_gauss), C.c_int32(sh_degree), C.c_int32(max_num_sh),
                                  C.c_int32(max_sg_display), C.c_int64(n), L.ptr(rgb), L.stream(positions.device)))
    return rgb


def march_backward(gas, cam, prims, ray_colors, dloss, dt_step, dynamic_sampling, max_prim_slice,
                   white_background=True, t_eps=TRANSMITTANCE_EPSILON, stats=None, records=None, out=None, record_format=0):
    """``out``: five preallocated gradient tensors (density, rgb, position, scale, quaternion) to write into."""
    n, dev = prims.shape[0], prims.device
    n_rays = cam.width * cam.height
    m = L.RgxMarch(dt_step, int(bool(dynamic_sampling)), int(max_prim_slice), int(bool(white_background)), t_eps, int(record_format))
    ws = _march_ws(n, n_rays, max_prim_slice, dev)
    ddens, drgb, dpos, dscale, dquat = out if out is not None else (
        torch.empty(n, dtype=torch.float32, device=dev), torch.empty(n, 3, dtype=torch.float32, device=dev),
        torch.empty(n, 3, dtype=torch.float32, device=dev), torch.empty(n, 3, dtype=torch.float32, device=dev),
        torch.empty(n, 4, dtype=torch.float32, device=dev))
    L.check(L.lib().rgx_march_backward(L.ptr(gas.ws), C.byref(cam), C.byref(m), L.ptr(prims), C.c_int64(n),
                                       L.ptr(ray_colors), L.ptr(dloss), L.ptr(ddens), L.ptr(drgb), L.ptr(dpos),
                                       L.ptr(dscale), L.ptr(dquat), L.ptr(ws), C.c_size_t(ws.numel()),
                                       L.ptr(records), C.c_size_t(0 if records is None else records.numel()),
                                       L.ptr(stats), L.stream(dev)))
    return ddens, drgb, dpos, dscale, dquat


def launch_pipeline_forward(pipeline, sbt, gas, bbox_min, bbox_max, dt_step, dynamic_sampling, camera,
                            densities, color_features, positions, scales, quaternions, max_prim_slice,
                            iteration=0, jitter=0, rnd_sample=0, supersampling=(1, 1), white_background=True,
                            hit_prim_idx=None, t_eps=TRANSMITTANCE_EPSILON, stats=None, return_prims=False):
    """optix_utils.py:222-322.  ``color_features`` is the per-Gaussian RGB (N,3).  ``bbox_min`` /
    ``bbox_max`` are accepted for signature compatibility: the acceleration structure already holds the
    scene box they were computed from.  ``iteration``, ``jitter``, ``rnd_sample`` are dead launch
    parameters in the reference too; ``hit_prim_idx`` (its per-ray hit scratch) is not needed."""
    cam = camera_struct(camera, supersampling)
    prims = pack_prims(gas, cam, L.f32(positions), L.f32(scales), L.f32(quaternions), L.f32(densities),
                       L.f32(color_features))
    out = march_forward(gas, cam, prims, dt_step, dynamic_sampling, max_prim_slice, white_background, t_eps, stats)
    return (out, prims) if return_prims else out


def launch_pipeline_test(pipeline, sbt, gas, bbox_min, bbox_max, dt_step, dynamic_sampling, camera, densities,
                         color_features, positions, scales, quaternions, max_prim_slice, rnd_sample=0,
                         supersampling=(1, 1), white_background=True, hit_prim_idx=None,
                         t_eps=TRANSMITTANCE_EPSILON, stats=None):
    """optix_utils.py:503-601: the inference launch; same kernel as the training forward."""
    return launch_pipeline_forward(pipeline, sbt, gas, bbox_min, bbox_max, dt_step, dynamic_sampling, camera,
                                   densities, color_features, positions, scales, quaternions, max_prim_slice,
                                   rnd_sample=rnd_sample, supersampling=supersampling,
                                   white_background=white_background, hit_prim_idx=hit_prim_idx, t_eps=t_eps,
                                   stats=stats)


def launch_pipeline_backward(pipeline, sbt, gas, bbox_min, bbox_max, dt_step, dynamic_sampling, camera,
                             densities, color_features, positions, scales, quaternions, ray_colors,
                             dloss_dray_colors, max_prim_slice, iteration=0, jitter=0, rnd_sample=0,
                             supersampling=(1, 1), hit_prim_idx=None, t_eps=TRANSMITTANCE_EPSILON, stats=None,
                             prims=None):
    """optix_utils.py:363-500 (+ reduce_temp_grads 325-361): returns densities_grad, color_features_grad
    (w.r.t. the per-Gaussian RGB), positions_grad, scales_grad, quaternions_grad."""
    cam = camera_struct(camera, supersampling)
    if prims is None:
        prims = pack_prims(gas, cam, L.f32(positions), L.f32(scales), L.f32(quaternions), L.f32(densities),
                           L.f32(color_features))
    return march_backward(gas, cam, prims, L.f32(ray_colors), L.f32(dloss_dray_colors), dt_step, dynamic_sampling,
                          max_prim_slice, True, t_eps, stats)


def new_stats(device):
    """Zeroed device counter block for the ``stats`` arguments."""
    return torch.zeros(len(L.STATS_FIELDS), dtype=torch.int64, device=device)


def read_stats(stats):
    return dict(zip(L.STATS_FIELDS, stats.tolist()))


def first_hit(gas, prims, eye, dirs, tlo, thi):
    out = torch.empty(dirs.shape[0], dtype=torch.float32, device=dirs.device)
    L.check(L.lib().rgx_first_hit(L.ptr(gas.ws), L.ptr(prims), C.c_int64(prims.shape[0]), L.host3(eye),
                                  C.c_int64(dirs.shape[0]), L.ptr(dirs), L.ptr(tlo), L.ptr(thi), L.ptr(out),
                                  L.stream(dirs.device)))
    return out


def trace_segments(gas, prims, eye, dirs, tlo, thi, cap):
    n = dirs.shape[0]
    counts = torch.empty(n, dtype=torch.int32, device=dirs.device)
    ids = torch.full((n, cap), -1, dtype=torch.int32, device=dirs.device)
    L.check(L.lib().rgx_trace_segments(L.ptr(gas.ws), L.ptr(prims), C.c_int64(prims.shape[0]), L.host3(eye),
                                       C.c_int64(n), L.ptr(dirs), L.ptr(tlo), L.ptr(thi), C.c_int32(cap),
                                       L.ptr(counts), L.ptr(ids), L.stream(dirs.device)))
    return counts, ids


def collect_tiles(gas, cam, prims, tlo, thi, cap, uncounted=False):
    """Hit lists of per-pixel segments through the tile-cooperative collect (test hook).  ``uncounted``:
    the filter as the kernels launched without a statistics block compile it (with its early exit)."""
    n_rays = cam.width * cam.height
    counts = torch.zeros(n_rays, dtype=torch.int32, device=prims.device)
    ids = torch.full((n_rays, cap), -1, dtype=torch.int32, device=prims.device)
    L.check(L.lib().rgx_collect_tiles(L.ptr(gas.ws), C.byref(cam), L.ptr(prims), C.c_int64(prims.shape[0]), L.ptr(tlo),
                                      L.ptr(thi), C.c_int32(cap), L.ptr(counts), L.ptr(ids), C.c_int32(int(bool(uncounted))),
                                      L.stream(prims.device)))
    return counts, ids


_fault_watch = {}    # (device, stream handle) -> [pinned int32 tensor, event, pending]
FAULTS_SEEN = {"replay_lost": 0, "sweep_dropped": 0}   # totals of what the lazy checks below have read so far


def _watch_faults(ws, n, device):
    """After a backward: queue a 16-byte copy of the workspace's fault counters to pinned host memory.
    Nothing waits for it; ``_check_faults`` looks at it when the same stream next starts a forward."""
    off = (max(int(n), 1) * 64 + 255) // 256 * 256
    if ws.numel() < off + 256:
        return
    key = (str(device), torch.cuda.current_stream(device).cuda_stream)
    w = _fault_watch.get(key)
    if w is None:
        w = _fault_watch[key] = [torch.zeros(4, dtype=torch.int32).pin_memory(), torch.cuda.Event(), False]
        if len(_fault_watch) > 4 * _SCRATCH_STREAMS:
            del _fault_watch[next(iter(_fault_watch))]
    if w[2] and not w[1].query():
        return                              # the previous copy is still in flight: keep its buffer untouched
    w[0].copy_(ws[off:off + 16].view(torch.int32), non_blocking=True)
    w[1].record(torch.cuda.current_stream(device))
    w[2] = True


def _check_faults(device):
    """Reads the counters a finished ``_watch_faults`` copy brought back.  A sweep that dropped tree nodes
    lost hits (wrong image and gradients): RgxError.  A replay that lost its record gave that tile the
    gradient of the iterations replayed so far (a difference at the transmittance floor): a warning."""
    w = _fault_watch.get((str(device), torch.cuda.current_stream(device).cuda_stream))
    if w is None or not w[2] or not w[1].query():
        return
    w[2] = False
    lost, dropped = int(w[0][0]), int(w[0][1])
    FAULTS_SEEN["replay_lost"] += lost
    FAULTS_SEEN["sweep_dropped"] += dropped
    if dropped:
        raise L.RgxError(f"librgx: {dropped} sweeps of an earlier launch dropped tree nodes (node stack full): "
                         "hits were lost, its image and gradients are wrong")
    if lost:
        import warnings
        warnings.warn(f"librgx: {lost} tiles of an earlier backward did not consume their hit-list record exactly; "
                      "their gradients stop at the last iteration replayed", RuntimeWarning, stacklevel=3)


def march_faults(n, device, ws=None):
    """(replays that lost their record, sweeps that dropped nodes) counted by the launches since the last
    forward on this stream's march workspace; waits for the stream."""
    if ws is None:
        ws = _scratch.get(("march", str(device), torch.cuda.current_stream(device).cuda_stream))
        if ws is None:
            return 0, 0
    out = (C.c_uint64 * 2)()
    L.check(L.lib().rgx_march_faults(L.ptr(ws), C.c_size_t(ws.numel()), C.c_int64(n), out, L.stream(device)))
    return int(out[0]), int(out[1])
