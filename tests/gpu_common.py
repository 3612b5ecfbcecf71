"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

from raygaussx_amd import optix_utils as u_ox
from raygaussx_amd import scenes
from raygaussx_amd.render_optix import RenderOptixFunction, compute_rgb, default_settings

DEV = "cuda:0"


def to_dev(scene_np):
    return {k: torch.from_numpy(np.ascontiguousarray(v)).to(DEV) for k, v in scene_np.items()}


def cos_rel(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return a @ b / (np.linalg.norm(a) * np.linalg.norm(b) + 1e-300), np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-300)


def gpu_render(scene_np, cam, cfg, white=True, supersampling=(1, 1), want_grad=None, stats=True, record_hits=True,
               rec_tile_words=None, half_sums=False):
    """Runs RenderOptixFunction (and its backward when ``want_grad`` = dL/dimage is given).
    ``record_hits``: the backward replays the forward's hit-list record (the default) or searches
    the tree again; ``rec_tile_words`` sizes the record per tile."""
    sc = to_dev(scene_np)
    names = ("positions", "scales", "quaternions", "densities", "color_features", "sph_gauss_features",
             "bandwidth_sharpness", "lobe_axis")
    n = sc["positions"].shape[0]
    if "sph_gauss_features" not in sc:
        sc["sph_gauss_features"] = torch.zeros(n, 3, 0, device=DEV)
        sc["bandwidth_sharpness"] = torch.zeros(n, 0, device=DEV)
        sc["lobe_axis"] = torch.zeros(n, 0, 3, device=DEV)
    g = sc["sph_gauss_features"].shape[2]
    args = [sc[k].clone().requires_grad_(want_grad is not None) for k in names]
    settings = default_settings(cam.to(DEV), cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"],
                                num_sph_gauss=g, white_background=white, supersampling=supersampling,
                                t_eps=cfg.get("t_eps", 1e-3))
    settings.record_hits = record_hits
    settings.rec_half_sums = half_sums
    if rec_tile_words is not None:
        settings.rec_tile_words = rec_tile_words
    if stats:
        settings.stats = u_ox.new_stats(DEV)
    img = RenderOptixFunction.apply(*args, settings)
    out = dict(image=img.detach().cpu().numpy(), settings=settings)
    if stats:
        out["stats_fwd"] = u_ox.read_stats(settings.stats)
    if want_grad is not None:
        if stats:
            settings.stats.zero_()
        img.backward(torch.from_numpy(want_grad).to(DEV))
        out["grads"] = {k: (None if a.grad is None else a.grad.cpu().numpy()) for k, a in zip(names, args)}
        if stats:
            out["stats_bwd"] = u_ox.read_stats(settings.stats)
            assert out["stats_bwd"]["replay_lost"] == 0
    torch.cuda.synchronize()
    return out


def gpu_forward_counts(scene_np, cam, cfg, white=True, supersampling=(1, 1)):
    """The forward through the counting kernels with the counters also kept per ray:
    (image (R,3), counts (R,2) = slabs blended, sum of their hit-list lengths).  Runs the recording
    forward, whose hit lists are whole as in the reference."""
    sc = to_dev(scene_np)
    n = sc["positions"].shape[0]
    gas = u_ox.AccelerationStructure(n, DEV).build_from_gaussians(sc["positions"], sc["scales"], sc["quaternions"], sc["densities"])
    cs = u_ox.camera_struct(cam.to(DEV), supersampling)
    k = sc["color_features"].shape[2]
    g = sc["sph_gauss_features"].shape[2] if "sph_gauss_features" in sc else 0
    rgb = compute_rgb(cam.camera_center, sc["positions"], sc["color_features"], sc.get("sph_gauss_features"),
                      sc.get("bandwidth_sharpness"), sc.get("lobe_axis"), g, int(round(k ** 0.5)) - 1)
    prims = u_ox.pack_prims(gas, cs, sc["positions"], sc["scales"], sc["quaternions"], sc["densities"], rgb)
    rec = u_ox.new_records(cs, DEV, tile_words=u_ox.REC_LIST_WORDS)     # hit lists only: no sample sums needed here
    img, counts = u_ox.march_forward(gas, cs, prims, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"], white,
                                     cfg.get("t_eps", 1e-3), records=rec, ray_counts=True)
    torch.cuda.synchronize()
    return img.cpu().numpy(), counts.cpu().numpy().astype(np.int64)


def comparable_rays(orc, ctx, img, gpu_counts, ids=None, rel=2.0 ** -20, tol=5e-5):
    """The rays on which the adaptive-step march can be compared at the gates of the fixed step:
    (mask over ``ids``, number re-phased, number on a cut-off edge).

    With dynamic_sampling the step is dt_dist / cbrt(T): the last bits of exp and cbrt (libm in the
    oracle, the hardware's on the GPU, CUDA's in the reference) move every later sample of a ray by a
    few parts in 10^7 of the distance marched.  Two things can then differ however exact the kernels
    are: (a) a slab boundary crosses a Gaussian's entry or exit, and the ray blends other slabs from
    there on (re-phased: its per-ray counters differ between the two sides); (b) the slabs stay, but one
    sample crosses a Gaussian's cut-off |M(x - mu)| = k, where the density jumps by the threshold 0.1:
    up to 0.1 dt |colour| in the image.  (b) is a property of the truncated-density model, not of an
    implementation: the oracle moves by as much against itself when its own step is scaled by
    1 +- ``rel`` (eight ulp, the size of the exp / cbrt differences accumulated along a ray).  Rays on
    which it does by more than ``tol`` (half the image gate) are set aside with the re-phased ones;
    every other ray has to meet the gates."""
    same, _ = same_march(orc, ctx, gpu_counts, ids)
    sel = slice(None) if ids is None else ids
    stable = np.ones(same.shape, bool)
    if ctx["ms"].dynamic_sampling:
        for scale in (1.0 - rel, 1.0 + rel):
            orc.set_step_scale(scale)
            try:
                moved, _ = orc.march_forward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], ids)
            finally:
                orc.set_step_scale(1.0)
            stable &= np.abs(moved[sel] - img[sel]).max(1) <= tol
    return same & stable, int((~same).sum()), int((same & ~stable).sum())


def same_march(orc, ctx, gpu_counts, ids=None):
    """Which rays marched the same slab sequence on both sides: (mask over ``ids``, the oracle's counts).
    With the adaptive step the slab length depends on cbrt(T), so the last bit of exp or cbrt can move a
    slab boundary across a Gaussian's edge and re-phase the rest of that ray; such a ray blends a
    different number of slabs or of hits."""
    _, oc = orc.march_forward_counts(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], ids)
    gc = gpu_counts if ids is None else gpu_counts[ids]
    return (oc == gc).all(1), oc


def cutoff_stable_rays(orc, ctx, img, ids=None):
    """Rays on none of whose samples the cut-off decision of the backward depends on the arrangement of the
    arithmetic: mask over ``ids``.

    The backward's gradient loop decides ``power < k^2`` per sample.  The reference forms that power in its
    backward by another arrangement than in its forward (backward/gaussians_aabb.cu:375-396: t0 = tbuffer +
    0.5 dt, a 3x3 matrix product; forward 112-180: fmaf, dot products); the kernels here use the forward's.
    One ulp of t moves the power of a thin Gaussian by 1e-4 of its value, so the two disagree on a sample that
    sits that close to k^2 -- and one sample flipped is, for a few hundred rays, 1e-3 of the whole gradient's
    norm.  The oracle counts such samples per ray, from its own two arrangements; a ray with one is set aside.
    Call before ``render_backward`` (which drops the oracle's candidate tree)."""
    counts = orc.march_backward_in_cut(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], img, ids)
    return counts[:, 1] == 0
