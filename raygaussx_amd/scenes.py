"""Seeded synthetic scenes and cameras for the benchmark configurations.

The reference ships no datasets (``dataset/.gitkeep`` only), so every workload
is generated.  Parameter conventions are those of the renderer's inputs
(optix_raycasting/render_optix.py:94-95): ``scales`` already exponentiated,
unit quaternions (w,x,y,z), raw densities, ``color_features`` (N,3,K)
channel-major, empty spherical-Gaussian tensors when G == 0.

Cameras expose exactly the attributes the renderer reads
(optix_raycasting/optix_utils.py:258-266): ``camera_center``,
``world_view_transform`` (columns 0..2 of its top-left 3x3 block are the
camera's right / down / forward axes in world space), ``FoVx``, ``FoVy``,
``Px``, ``Py``, ``image_width``, ``image_height``.
"""
import math
from dataclasses import dataclass

import torch


@dataclass
class Camera:
    camera_center: torch.Tensor         # (3,)
    world_view_transform: torch.Tensor  # (4,4), transposed world-to-view as in classes/cameras.py:49
    FoVx: float
    FoVy: float
    Px: float
    Py: float
    image_width: int
    image_height: int

    def to(self, device):
        return Camera(self.camera_center.to(device), self.world_view_transform.to(device), self.FoVx,
                      self.FoVy, self.Px, self.Py, self.image_width, self.image_height)


def look_at_camera(eye, target=(0.0, 0.0, 0.0), up=(0.0, 0.0, 1.0), fov_x_deg=40.0, width=128,
                   height=128, px=0.5, py=0.5):
    """forward = normalize(target-eye), right = normalize(forward x up), down = forward x right."""
    eye_t = torch.tensor(eye, dtype=torch.float64)
    fwd = torch.tensor(target, dtype=torch.float64) - eye_t
    fwd = fwd / fwd.norm()
    right = torch.linalg.cross(fwd, torch.tensor(up, dtype=torch.float64))
    right = right / right.norm()
    down = torch.linalg.cross(fwd, right)
    rot = torch.stack([right, down, fwd], dim=1)  # camera-to-world rotation, columns = axes
    wvt = torch.eye(4, dtype=torch.float64)
    wvt[:3, :3] = rot
    wvt[3, :3] = -(rot.T @ eye_t)
    fovx = math.radians(fov_x_deg)
    fovy = 2.0 * math.atan(math.tan(fovx / 2.0) * height / width)  # scene/dataset_readers.py:327
    return Camera(eye_t.float(), wvt.float(), fovx, fovy, px, py, width, height)


# name -> rendering parameters.  dt_step / dynamic_sampling / max_prim_slice follow
# configs/nerf_synthetic.yml:12 (object scenes) and configs/base.yml:12-13 (unbounded).
CONFIGS = {
    0: dict(n=4096, width=128, height=128, fov=40.0, dt_step=0.0025, dynamic_sampling=False,
            max_prim_slice=2048, t_eps=1e-3, n_cameras=1),
    1: dict(n=300_000, width=800, height=800, fov=39.6, dt_step=0.0025, dynamic_sampling=False,
            max_prim_slice=2048, t_eps=1e-3, n_cameras=100),
    2: dict(n=3_000_000, width=1237, height=822, fov=50.0, dt_step=0.005, dynamic_sampling=True,
            max_prim_slice=512, t_eps=1e-3, n_cameras=300),
    3: dict(n=3_000_000, width=1920, height=1080, fov=50.0, dt_step=0.005, dynamic_sampling=True,
            max_prim_slice=512, t_eps=1e-4, n_cameras=300),
    4: dict(n=1_000_000, width=1024, height=1024, fov=39.6, dt_step=0.0025, dynamic_sampling=False,
            max_prim_slice=2048, t_eps=1e-3, n_cameras=100),
    # Not a benchmark configuration: the march kernels' best case, for pricing the implementation apart from a
    # workload's sparsity.  A few hundred large, faint, isotropic Gaussians in the ball of configuration 4: each covers
    # hundreds of pixels and a dozen slabs, so all rays of a tile hit the same Gaussians, a ray's chord through a
    # Gaussian fills whole slabs, no ray saturates, and the tree is a few levels deep.
    "coherent": dict(n=512, width=800, height=800, fov=39.6, dt_step=0.0025, dynamic_sampling=False,
                     max_prim_slice=2048, t_eps=1e-3, n_cameras=100),
}


def _unit_vectors(n, gen):
    v = torch.randn(n, 3, generator=gen)
    return v / v.norm(dim=1, keepdim=True)


def _ball(n, radius, gen):
    return _unit_vectors(n, gen) * (torch.rand(n, 1, generator=gen) ** (1.0 / 3.0)) * radius


def make_scene(config, n=None, sh_degree=3, device="cpu", seed=None):
    """Gaussian parameters of benchmark configuration ``config`` (0..4).

    Draw order (fixed, so a seed names one scene): centres, log-scales,
    quaternions, densities, SH DC, SH rest.  Config 2/3's "N(0, 1.5 I)" is read
    as covariance 1.5 I (std sqrt(1.5) per axis).
    """
    cfg = CONFIGS[config]
    n = cfg["n"] if n is None else n
    gen = torch.Generator().manual_seed(1234 + {3: 2, "coherent": 9}.get(config, config) if seed is None else seed)
    if config == 0:
        pos = torch.rand(n, 3, generator=gen) * 2.0 - 1.0
        log_s = torch.randn(n, 3, generator=gen) * 0.4 - 3.5
    elif config == 1:
        pos = _ball(n, 1.0, gen)
        log_s = torch.randn(n, 3, generator=gen) * 0.5 - 4.5
    elif config in (2, 3):
        n_core = int(round(0.7 * n))
        core = torch.randn(n_core, 3, generator=gen) * math.sqrt(1.5)
        shell = _unit_vectors(n - n_core, gen) * (10.0 + 40.0 * torch.rand(n - n_core, 1, generator=gen))
        pos = torch.cat([core, shell])
        log_s = torch.cat([torch.randn(n_core, 3, generator=gen) * 0.6 - 4.0,
                           torch.randn(n - n_core, 3, generator=gen) * 0.5 - 1.5])
    elif config == 4:
        pos = _ball(n, 2.0, gen)
        log_s = torch.randn(n, 3, generator=gen) * 0.5 - 4.5
    elif config == "coherent":
        pos = _ball(n, 2.0, gen)
        log_s = torch.full((n, 3), math.log(0.5))
    else:
        raise ValueError(f"unknown config {config}")
    quat = torch.randn(n, 4, generator=gen)
    quat = quat / quat.norm(dim=1, keepdim=True)
    dens = torch.nn.functional.softplus(torch.randn(n, generator=gen))
    if config == "coherent":
        dens = torch.full((n,), 0.15)      # k = sqrt(2 ln 1.5) = 0.9: visible to 0.45 from the centre
    k = (sh_degree + 1) ** 2
    sh = torch.empty(n, 3, k)
    sh[:, :, 0] = torch.randn(n, 3, generator=gen) * 0.2 + 0.5
    if k > 1:
        sh[:, :, 1:] = torch.randn(n, 3, k - 1, generator=gen) * 0.05
    scene = dict(positions=pos, scales=log_s.exp(), quaternions=quat, densities=dens,
                 color_features=sh, sph_gauss_features=torch.zeros(n, 3, 0),
                 bandwidth_sharpness=torch.zeros(n, 0), lobe_axis=torch.zeros(n, 0, 3))
    return {k_: v.float().contiguous().to(device) for k_, v in scene.items()}


def make_camera(config, index=0, width=None, height=None):
    """Camera ``index`` of configuration ``config``."""
    cfg = CONFIGS[config]
    w = cfg["width"] if width is None else width
    h = cfg["height"] if height is None else height
    if config == 0:
        r = 4.0 / math.sqrt(3.0)
        eye = (r, r, r)
    elif config in (1, 4, "coherent"):
        # golden-angle spiral over the upper hemisphere, radius 4
        m = cfg["n_cameras"]
        z = (index % m + 0.5) / m
        phi = (index % m) * math.pi * (3.0 - math.sqrt(5.0))
        rho = math.sqrt(max(0.0, 1.0 - z * z))
        eye = (4.0 * rho * math.cos(phi), 4.0 * rho * math.sin(phi), 4.0 * z)
    else:
        th = 2.0 * math.pi * (index % cfg["n_cameras"]) / cfg["n_cameras"]
        eye = (3.0 * math.cos(th), 2.0 * math.sin(th), 0.5)
    return look_at_camera(eye, fov_x_deg=cfg["fov"], width=w, height=h)


def scene_to_numpy(scene):
    return {k: v.detach().cpu().numpy() for k, v in scene.items()}
