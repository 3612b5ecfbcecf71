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
               rec_tile_words=None):
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
