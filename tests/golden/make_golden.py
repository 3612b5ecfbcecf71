"""Writes tests/golden/config0.npz: the CPU oracle's results on benchmark configuration 0.

The reference ships no tests, golden vectors or fixtures of its own, and its renderer cannot
be imported without OptiX, so these vectors come from the oracle (oracle/rgx_oracle.c), whose
parts are pinned by tests/test_oracle_*.py against closed forms, float64 evaluations and brute
force.  The file pins the oracle against later change and gives the GPU tests fixed expected
values.  The scene's tensors are stored with the results (in_*): torch's CPU random and
transcendental kernels are vectorised per CPU model, so a scene regenerated from its seed on
another machine differs in the last bit here and there, which is enough to move a first-hit
distance by an ulp.  The camera comes from raygaussx_amd.scenes (float64 arithmetic rounded once).

    python tests/golden/make_golden.py

Contents (configuration 0: 4096 Gaussians, 128x128, dt 0.0025, MSE loss against a seeded target):
  in_<param>              positions, scales, quaternions, densities, color_features of the scene
  image (16384,3)         forward colours
  stats_* scalars         hit pairs, slabs, empty slabs, rays hit of the forward march
  d_<param>               gradients of the loss for positions, scales, quaternions, densities, color_features
  seg_ray, seg_lo, seg_hi, seg_off, seg_ids   per marched slab of every 61st ray: ray index, slab
                          bounds, and the sorted indices of the Gaussians hit (CSR layout)
  fh_ray, fh_lo, fh_hi, fh_t                  first-hit query on 2000 seeded segments (-1 = none)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

from oracle import oracle as orc  # noqa: E402
from raygaussx_amd import scenes  # noqa: E402

SEG_RAY_STRIDE = 61
TARGET_SEED = 7
FH_SEED = 3


def mse_dloss(img):
    target = np.random.default_rng(TARGET_SEED).random(img.shape, dtype=np.float32)
    return (2.0 * (img - target) / img.size).astype(np.float32)


def first_hit_segments(n_rays):
    rng = np.random.default_rng(FH_SEED)
    rays = rng.choice(n_rays, 2000, replace=False)
    tlo = rng.uniform(2.0, 5.0, 2000).astype(np.float32)
    thi = (tlo + rng.uniform(0.01, 1.5, 2000)).astype(np.float32)
    return rays, tlo, thi


PARAMS = ("positions", "scales", "quaternions", "densities", "color_features")


def scene_of(golden):
    """The stored scene as the dict of arrays the oracle and gpu_common.gpu_render take."""
    return {k: golden["in_" + k] for k in PARAMS}


def compute(sc=None):
    """All vectors for scene ``sc`` (default: configuration 0 generated on this machine)."""
    orc.build()
    if sc is None:
        sc = {k: v for k, v in scenes.scene_to_numpy(scenes.make_scene(0)).items() if k in PARAMS}
    cam, cfg = scenes.make_camera(0), scenes.CONFIGS[0]
    img, st, ctx = orc.render_forward(sc, cam, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"])
    grads, _ = orc.render_backward(sc, ctx, img, mse_dloss(img))
    out = {"in_" + k: sc[k] for k in PARAMS}
    out["image"] = img
    for k in ("hit_pairs", "slabs", "empty_slabs", "rays_hit"):
        out["stats_" + k] = np.int64(st[k])
    for k in PARAMS:
        out["d_" + k] = grads[k]
    seg_ray, seg_lo, seg_hi, seg_off, seg_ids = [], [], [], [0], []
    for r in range(0, cam.image_width * cam.image_height, SEG_RAY_STRIDE):
        slabs, _ = orc.march_trace(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], r)
        for tb, dt, lo, hi, ids in slabs:
            seg_ray.append(r); seg_lo.append(lo); seg_hi.append(hi)
            seg_ids.extend(sorted(ids.tolist()))
            seg_off.append(len(seg_ids))
    out.update(seg_ray=np.asarray(seg_ray, np.int32), seg_lo=np.asarray(seg_lo, np.float32),
               seg_hi=np.asarray(seg_hi, np.float32), seg_off=np.asarray(seg_off, np.int32),
               seg_ids=np.asarray(seg_ids, np.int32))
    rays, tlo, thi = first_hit_segments(cam.image_width * cam.image_height)
    dirs = orc.ray_dirs(ctx["cs"], rays)
    out.update(fh_ray=rays.astype(np.int32), fh_lo=tlo, fh_hi=thi, fh_t=orc.first_hit(ctx["prims"], dirs, tlo, thi))
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "config0.npz")
    np.savez_compressed(path, **compute())
    print(path, os.path.getsize(path), "bytes")
