"""rgx_march_backward_noalloc: the backward for callers that cannot allocate device memory or bring a
workspace (its scratch memory is a file-scope device array of the library).  Called through the C ABI
and checked against rgx_march_backward on the same inputs, twice in a row, the second call on a
smaller scene and image (the array still holds the first call's gradient block and tile order)."""
import ctypes as C

import numpy as np
import pytest
import torch

from raygaussx_amd import scenes

pytestmark = pytest.mark.gpu

# north_star's gradient gates; equal inputs through the same kernels differ only in the order of the
# fp32 atomic adds, so the test holds the two entry points much closer than the gates
COS_MIN, REL_MAX = 0.9999, 1e-3
REL_SAME_KERNELS = 1e-5


def test_allocation_free_backward_matches_the_workspace_backward():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import gpu_common as gx
    from raygaussx_amd import _lib, optix_utils as u_ox
    from raygaussx_amd.render_optix import compute_rgb
    lib = _lib.lib()
    dev = gx.DEV
    stream = _lib.stream(dev)

    def one_call(config, n, width, height, seed, scale, with_record):
        sc = gx.to_dev(scenes.scene_to_numpy(scenes.make_scene(config, n=n, sh_degree=1, seed=seed)))
        cam = scenes.make_camera(config, 1, width=width, height=height)
        cs = u_ox.camera_struct(cam)
        cfg = scenes.CONFIGS[config]
        gas = u_ox.AccelerationStructure(n, dev).build_from_gaussians(sc["positions"], sc["scales"] * scale, sc["quaternions"], sc["densities"])
        rgb = compute_rgb(cam.camera_center, sc["positions"], sc["color_features"], None, None, None, 0, 1)
        prims = u_ox.pack_prims(gas, cs, sc["positions"], sc["scales"] * scale, sc["quaternions"], sc["densities"], rgb)
        rec = u_ox.new_records(cs, dev) if with_record else None
        img = u_ox.march_forward(gas, cs, prims, cfg["dt_step"], False, 512, True, records=rec)
        dloss = torch.from_numpy(np.random.default_rng(seed).normal(size=(width * height, 3)).astype(np.float32)).to(dev)
        want = u_ox.march_backward(gas, cs, prims, img, dloss, cfg["dt_step"], False, 512, True, records=rec)
        f = dict(dtype=torch.float32, device=dev)
        got = (torch.empty(n, **f), torch.empty(n, 3, **f), torch.empty(n, 3, **f), torch.empty(n, 3, **f), torch.empty(n, 4, **f))
        m = _lib.RgxMarch(cfg["dt_step"], 0, 512, 1, 1e-3)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(dev)[0]
        print(f"[gpu-step] rgx_march_backward_noalloc: n={n}, {width}x{height}, record {with_record}", flush=True)
        rc = lib.rgx_march_backward_noalloc(_lib.ptr(gas.ws), C.byref(cs), C.byref(m), _lib.ptr(prims), C.c_int64(n), _lib.ptr(img),
                                            _lib.ptr(dloss), *[_lib.ptr(g) for g in got], _lib.ptr(rec),
                                            C.c_size_t(0 if rec is None else rec.numel()), None, stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free_before          # nothing was allocated on the device
        for name, a, b in zip(("density", "rgb", "position", "scale", "quaternion"), got, want):
            cos, rel = gx.cos_rel(a.cpu().numpy(), b.cpu().numpy())
            assert float(b.abs().max()) > 0
            assert cos >= COS_MIN and rel <= REL_MAX and rel <= REL_SAME_KERNELS, (name, cos, rel)

    one_call(0, 20000, 200, 152, 5, 2.0, True)       # replays the forward's record; fills 1.28 MB of the gradient block
    one_call(0, 3000, 64, 48, 6, 3.0, True)          # smaller: the array still holds the first call's data beyond its own
    one_call(1, 5000, 96, 80, 7, 3.0, False)         # and without a record (the tree-searching backward)

    # beyond the array's limits: a clear error, before anything is launched
    cs = u_ox.camera_struct(scenes.make_camera(0, 0, width=64, height=64))
    m = _lib.RgxMarch(0.0025, 0, 512, 1, 1e-3)
    dummy = torch.zeros(64, device=dev)
    args = lambda n: (_lib.ptr(dummy), C.byref(cs), C.byref(m), _lib.ptr(dummy), C.c_int64(n), *[_lib.ptr(dummy)] * 7, None, C.c_size_t(0), None, stream)
    assert lib.rgx_march_backward_noalloc(*args((1 << 20) + 1)) == -4
    assert b"limit" in lib.rgx_strerror(-4)
    cs.width, cs.height = 4096, 1025                 # more than 2^22 rays
    assert lib.rgx_march_backward_noalloc(*args(1000)) == -4
    assert lib.rgx_march_backward_noalloc(*args(-1)) == -1
