"""``RenderOptixFunction`` / ``RenderOptixSettings`` with the reference's signature and
semantics (optix_raycasting/render_optix.py:67-199), running on librgx.

Same tensors in -- positions (N,3), scales (N,3, already exponentiated), unit quaternions
(N,4 wxyz), densities (N,), color_features (N,3,K), sph_gauss_features (N,3,G),
bandwidth_sharpness (N,G), lobe_axis (N,G,3), settings -- same ``ray_colors`` (W*H,3) out,
and the same eight gradients (+ None) back.
"""
import ctypes as C
import math

import torch

from . import _lib as L
from . import optix_utils as u_ox


def compute_rgb(camera_center, positions, color_features, sph_gauss_features, bandwidth_sharpness, lobe_axis,
                num_sph_gauss, degree_sh):
    """render_optix.py:19-32 compute_cupy_rgb -> rgb (N,3)."""
    n = positions.shape[0]
    rgb = torch.empty(n, 3, dtype=torch.float32, device=positions.device)
    L.check(L.lib().rgx_sh_forward(L.host3(camera_center), L.ptr(positions), L.ptr(color_features),
                                   L.ptr(sph_gauss_features), L.ptr(bandwidth_sharpness), L.ptr(lobe_axis),
                                   C.c_int32(num_sph_gauss), C.c_int32(degree_sh), C.c_int64(n), L.ptr(rgb),
                                   L.stream(positions.device)))
    return rgb


def compute_sh_grad(camera_center, positions, color_features, sph_gauss_features, bandwidth_sharpness, lobe_axis,
                    num_sph_gauss, degree_sh, color_features_grad):
    """render_optix.py:34-52 compute_cupy_sh_grad -> dL_dsh (flat), dL_dpos, dL_dsph_gauss, dL_dsharpness,
    dL_dlobe_axis (flat, as the reference returns them)."""
    n, dev = positions.shape[0], positions.device
    k = (degree_sh + 1) ** 2
    g = num_sph_gauss
    dsh = torch.empty(n * 3 * k, dtype=torch.float32, device=dev)
    dpos = torch.empty(n, 3, dtype=torch.float32, device=dev)
    dsg = torch.empty(n * g * 3, dtype=torch.float32, device=dev)
    dsharp = torch.empty(n * g, dtype=torch.float32, device=dev)
    daxis = torch.empty(n * g * 3, dtype=torch.float32, device=dev)
    L.check(L.lib().rgx_sh_backward(L.host3(camera_center), L.ptr(positions), L.ptr(color_features),
                                    L.ptr(sph_gauss_features), L.ptr(bandwidth_sharpness), L.ptr(lobe_axis),
                                    C.c_int32(g), C.c_int32(degree_sh), C.c_int64(n), L.ptr(color_features_grad),
                                    L.ptr(dsh), L.ptr(dpos), L.ptr(dsg), L.ptr(dsharp), L.ptr(daxis), L.stream(dev)))
    return dsh, dpos, dsg, dsharp, daxis


def unnormalized_quaternion_grad(normalized_quaternions_grad, quaternions):
    """render_optix.py:54-63: gradient through q / |q|."""
    sum2 = torch.sum(quaternions ** 2, dim=1, keepdim=True)
    invsum32 = 1.0 / (torch.sqrt(sum2) * sum2)
    dots = (quaternions * normalized_quaternions_grad).sum(1, keepdim=True)
    return (sum2 * normalized_quaternions_grad - quaternions * dots) * invsum32


class RenderOptixSettings:
    """Attribute bag of render_optix.py:67-89.  ``context``, ``program_grps_*`` and ``pipeline_*`` are
    inert handles here; ``gas`` is an ``optix_utils.AccelerationStructure`` (or None);
    ``iteration`` / ``jitter`` / ``rnd_sample`` are unused by the reference's kernels as well.
    ``t_eps`` (not in the reference) exposes TRANSMITTANCE_EPSILON."""

    def __init__(self, context, update, gas, program_grps_fwd, pipeline_fwd, program_grps_bwd, pipeline_bwd,
                 dt_step, dynamic_sampling, viewpoint_cam, max_prim_slice, num_sph_gauss, iteration, jitter,
                 rnd_sample, supersampling, white_background, hit_prim_idx, t_eps=u_ox.TRANSMITTANCE_EPSILON):
        self.context = context
        self.update = update
        self.gas = gas
        self.program_grps_fwd = program_grps_fwd
        self.pipeline_fwd = pipeline_fwd
        self.program_grps_bwd = program_grps_bwd
        self.pipeline_bwd = pipeline_bwd
        self.dt_step = dt_step
        self.dynamic_sampling = dynamic_sampling
        self.viewpoint_cam = viewpoint_cam
        self.max_prim_slice = max_prim_slice
        self.num_sph_gauss = num_sph_gauss
        self.iteration = iteration
        self.jitter = jitter
        self.rnd_sample = rnd_sample
        self.supersampling = supersampling
        self.white_background = white_background
        self.hit_prim_idx = hit_prim_idx
        self.t_eps = t_eps
        self.stats = None   # optional optix_utils.new_stats() block
        self.record_hits = True   # forward records its hit lists for the backward to replay
        self.rec_tile_words = u_ox.REC_TILE_WORDS   # record size per 8x8 pixel tile, 32-bit words
        # True: the record keeps the per-sample colour sums in half precision with a power-of-two scale per ray and
        # 16 samples (two thirds of the record's bytes; gradients within about 1e-4 of those of the float record)
        self.rec_half_sums = False
        # True: ``gas`` was built from these very positions, scales, quaternions and densities (an earlier
        # view of the same accumulation window) -- the forward then skips the rebuild
        self.gas_is_current = False


def default_settings(viewpoint_cam, dt_step, dynamic_sampling, max_prim_slice, num_sph_gauss=0,
                     white_background=True, supersampling=(1, 1), update=False, gas=None,
                     t_eps=u_ox.TRANSMITTANCE_EPSILON):
    """A ``RenderOptixSettings`` with the inert handles filled in."""
    return RenderOptixSettings(None, update, gas, None, None, None, None, dt_step, dynamic_sampling, viewpoint_cam,
                               max_prim_slice, num_sph_gauss, 0, 0, 0, supersampling, white_background, None, t_eps)


class RenderOptixFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, positions, scales, normalized_quaternions, densities, color_features, sph_gauss_features,
                bandwidth_sharpness, lobe_axis, settings):
        positions, scales, normalized_quaternions, densities, color_features = (
            L.f32(t.detach()) for t in (positions, scales, normalized_quaternions, densities, color_features))
        sph_gauss_features, bandwidth_sharpness, lobe_axis = (
            L.f32(t.detach()) for t in (sph_gauss_features, bandwidth_sharpness, lobe_axis))
        n, dev = positions.shape[0], positions.device
        u_ox._check_faults(dev)     # what the previous backward on this stream reported, if it has finished
        # render_optix.py:109-117: boxes + acceleration structure (rebuilt unless settings.update)
        gas = settings.gas
        stale = gas is None or not isinstance(gas, u_ox.AccelerationStructure) or gas.n != n or gas.device != dev
        if stale:
            gas = u_ox.AccelerationStructure(n, dev)
        unbuilt = stale or not gas.built      # nothing in the workspace to refit or to reuse
        if settings.update and not unbuilt:
            # render_optix.py:114-115: the existing structure takes the new boxes and keeps its shape
            if not settings.gas_is_current:
                boxes, _, _ = u_ox.ellipsoids_bbox_from_quat(normalized_quaternions, positions, scales, densities)
                u_ox.update_acceleration_structure(gas, boxes)
        elif unbuilt or not settings.gas_is_current:
            gas.build_from_gaussians(positions, scales, normalized_quaternions, densities)
        settings.gas = gas
        order_sh = int(round(math.sqrt(color_features.shape[2]))) - 1   # render_optix.py:119
        cam = u_ox.camera_struct(settings.viewpoint_cam, settings.supersampling)
        rgb = compute_rgb(cam.eye, positions, color_features, sph_gauss_features, bandwidth_sharpness, lobe_axis,
                          settings.num_sph_gauss, order_sh)
        prims = u_ox.pack_prims(gas, cam, positions, scales, normalized_quaternions, densities, rgb)
        # when a backward will follow, the forward leaves a record of its hit lists for it to replay
        fmt = 1 if settings.rec_half_sums else 0
        records = (u_ox.new_records(cam, dev, settings.rec_tile_words, n=n, record_format=fmt)
                   if (any(ctx.needs_input_grad[:8]) and settings.record_hits) else None)
        ray_colors = u_ox.march_forward(gas, cam, prims, settings.dt_step, settings.dynamic_sampling,
                                        settings.max_prim_slice, settings.white_background, settings.t_eps,
                                        settings.stats, records, record_format=fmt)
        u_ox.note_record_use(records, cam, dev, n, fmt)
        ctx.record_format = fmt
        ctx.records = records
        ctx.settings = settings
        ctx.cam = cam
        ctx.gas = gas
        ctx.prims = prims
        ctx.order_sh = order_sh
        ctx.save_for_backward(positions, color_features, sph_gauss_features, bandwidth_sharpness, lobe_axis,
                              ray_colors.clone())
        return ray_colors

    @staticmethod
    def backward(ctx, dloss_dray_colors):
        dloss_dray_colors = L.f32(dloss_dray_colors)          # render_optix.py:146-147
        settings = ctx.settings
        positions, color_features, sph_gauss_features, bandwidth_sharpness, lobe_axis, ray_colors = ctx.saved_tensors
        with torch.cuda.device(positions.device):             # called from the autograd engine's thread
            densities_grad, rgb_grad, positions_grad, scales_grad, quaternions_grad = u_ox.march_backward(
                ctx.gas, ctx.cam, ctx.prims, ray_colors, dloss_dray_colors, settings.dt_step,
                settings.dynamic_sampling, settings.max_prim_slice, settings.white_background, settings.t_eps,
                settings.stats, ctx.records, record_format=ctx.record_format)
            ctx.records = None
            ws = u_ox._scratch.get(("march", str(positions.device), torch.cuda.current_stream(positions.device).cuda_stream))
            if ws is not None:
                u_ox._watch_faults(ws, positions.shape[0], positions.device)
            sh_grad, dpos_dir, dsg, dsharp, daxis = compute_sh_grad(
                ctx.cam.eye, positions, color_features, sph_gauss_features, bandwidth_sharpness, lobe_axis,
                settings.num_sph_gauss, ctx.order_sh, rgb_grad)
            positions_grad += dpos_dir                        # render_optix.py:185
        n = positions.shape[0]
        sh_grad = sh_grad.reshape(n, 3, (ctx.order_sh + 1) ** 2)
        if settings.num_sph_gauss != 0:                       # render_optix.py:190-197
            dsharp = dsharp.reshape(-1, settings.num_sph_gauss)
            daxis = daxis.reshape(-1, settings.num_sph_gauss, 3)
            dsg = dsg.reshape(-1, 3, settings.num_sph_gauss)
        else:
            dsharp = daxis = dsg = None
        return (positions_grad, scales_grad, quaternions_grad, densities_grad, sh_grad, dsg, dsharp, daxis, None)
