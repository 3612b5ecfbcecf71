"""Independent float64 restatements used to pin the C oracle (tests only).

Nothing here shares code with oracle/rgx_oracle.c: geometry is written with
matrices and closed forms, the march evaluates each sample's Mahalanobis
distance directly (no forward-difference recurrence), and gradients come from
torch.autograd.
"""
import math

import numpy as np
import torch


def rot_from_quat(q):
    """Rotation matrix of a unit quaternion (w,x,y,z); textbook formula."""
    w, x, y, z = q[..., 0], q[..., 1], q[..., 2], q[..., 3]
    R = torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y),
        2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x),
        2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], dim=-1)
    return R.reshape(q.shape[:-1] + (3, 3))


def cutoff_k(dens, thr=0.1):
    return torch.sqrt(2.0 * torch.log(dens / thr))


def ray_dirs_pinhole(cam, ids=None):
    """K^-1 [u, v, 1] rotated by the camera-to-world rotation, float64."""
    W, H = cam.image_width, cam.image_height
    if ids is None:
        ids = np.arange(W * H)
    ids = np.asarray(ids)
    x = (ids % W).astype(np.float64)
    y = (ids // W).astype(np.float64)
    u = (x + 0.5) / W
    v = (y + 0.5) / H
    cx = 2.0 * (u - cam.Px) * math.tan(cam.FoVx / 2)
    cy = 2.0 * (v - cam.Py) * math.tan(cam.FoVy / 2)
    rot = cam.world_view_transform[:3, :3].double().numpy()
    d = cx[:, None] * rot[:, 0][None] + cy[:, None] * rot[:, 1][None] + rot[:, 2][None]
    return d / np.linalg.norm(d, axis=1, keepdims=True)


def ellipsoid_roots(eye, d, pos, scale, quat, dens):
    """Roots t of |S^-1 R^T (eye + t d - pos)|^2 = k^2 for every (ray, prim) pair, float64.
    Returns (valid, t_in, t_out, margin) with margin = normalised closest distance^2."""
    eye, d, pos, scale, quat, dens = [torch.as_tensor(a, dtype=torch.float64) for a in (eye, d, pos, scale, quat, dens)]
    R = rot_from_quat(quat)                      # (N,3,3)
    k = cutoff_k(dens)                           # (N,)
    A = R.transpose(1, 2) / (scale * k[:, None])[:, :, None]   # rows scaled: S^-1 R^T / k
    O = torch.einsum("nij,nj->ni", A, eye[None] - pos)          # (N,3)
    D = torch.einsum("nij,rj->rni", A, d)                        # (R,N,3)
    a = (D * D).sum(-1)
    b = (D * O[None]).sum(-1)
    c = (O * O).sum(-1)[None] - 1.0
    disc = b * b - a * c
    valid = disc > 0
    sq = torch.sqrt(torch.clamp(disc, min=0))
    t_in = (-b - sq) / a
    t_out = (-b + sq) / a
    closest2 = (O * O).sum(-1)[None] - b * b / a   # |P|^2 at closest approach
    return valid, t_in, t_out, closest2


def march_torch(params, eye, dirs, slabs_per_ray, dt_eps, white_bg=True):
    """Differentiable float64 forward over recorded slabs.

    params: dict of float64 tensors positions, scales, quaternions, densities, rgb.
    slabs_per_ray[r]: list of (tbuffer, dt, ids) actually blended for ray r.
    Hit sets and the ``power < k^2`` masks are constants of the graph, as in the reference.
    """
    pos, scale, quat, dens, rgb = (params[k] for k in ("positions", "scales", "quaternions", "densities", "rgb"))
    R_all = rot_from_quat(quat)
    out = []
    eye = torch.as_tensor(eye, dtype=torch.float64)
    for r, slabs in enumerate(slabs_per_ray):
        d = torch.as_tensor(dirs[r], dtype=torch.float64)
        T = torch.ones((), dtype=torch.float64)
        C = torch.zeros(3, dtype=torch.float64)
        for tb, dt, ids in slabs:
            ids = torch.as_tensor(np.asarray(ids), dtype=torch.long)
            t = tb + dt * (torch.arange(32, dtype=torch.float64) + 0.5)
            x = eye[None] + t[:, None] * d[None]                       # (32,3)
            rel = x[None] - pos[ids][:, None]                          # (h,32,3)
            loc = torch.einsum("hji,hsj->hsi", R_all[ids], rel) / scale[ids][:, None]
            power = (loc * loc).sum(-1)                                # (h,32)
            cut = (2.0 * torch.log(dens[ids] / 0.1)).detach()
            mask = (power.detach() < cut[:, None]).double()
            w = torch.exp(-0.5 * power) * mask
            sig = (dens[ids][:, None] * w).sum(0)                      # (32,)
            col = ((dens[ids][:, None] * w)[:, :, None] * rgb[ids][:, None]).sum(0)   # (32,3)
            for base in (0, 16):
                if not (T.item() > dt_eps):
                    break
                xx = sig[base:base + 16] * dt
                ww = torch.exp(-xx)
                s = dt * (1 - ww) / torch.clamp(xx, min=1e-6)
                t_before = T * torch.cat([torch.ones(1, dtype=torch.float64), torch.cumprod(ww, 0)[:-1]])
                C = C + ((t_before * s)[:, None] * col[base:base + 16]).sum(0)
                T = T * torch.prod(ww)
        out.append(C + T * (1.0 if white_bg else 0.0))
    return torch.stack(out)
