"""The C-ABI library without a GPU: it loads, exports every function include/rgx.h declares, reports
the header's ABI version, answers the host-only queries (sizes, error strings) and rejects bad
arguments before touching the device.  Plus the host mirror's pure-Python parts."""
import ctypes as C
import math
import os
import re

import numpy as np
import pytest
import torch

from raygaussx_amd import _lib, scenes, optix_utils as u_ox

HEADER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "include", "rgx.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rgx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_function():
    lib = _lib.lib()
    names = _declared()
    assert len(names) >= 30 and "rgx_march_forward" in names and "rgx_dist2_knn3" in names
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_lib.SYMBOLS) == names            # the binding checks the same list at load time
    version = int(re.search(r"#define RGX_ABI_VERSION (\d+)", open(HEADER).read()).group(1))
    assert lib.rgx_abi_version() == version == _lib.ABI_VERSION


def test_error_strings_and_size_queries():
    lib = _lib.lib()
    msgs = {rc: lib.rgx_strerror(rc).decode() for rc in (0, -1, -2, -3, -99)}
    assert len(set(msgs.values())) >= 4 and all(msgs.values())
    out = C.c_size_t(0)
    sizes = []
    for n in (0, 1, 1000, 1_000_000):
        assert lib.rgx_build_workspace_bytes(C.c_int64(n), C.byref(out)) == 0
        sizes.append(out.value)
    assert sizes == sorted(sizes) and sizes[-1] >= 1_000_000 * 100 and all(s % 256 == 0 for s in sizes)
    assert lib.rgx_build_workspace_bytes(C.c_int64(-1), C.byref(out)) == -1
    assert lib.rgx_build_workspace_bytes(C.c_int64(5), None) == -1
    assert lib.rgx_march_workspace_bytes(C.c_int64(1000), C.c_int64(640000), C.c_int32(2048), C.byref(out)) == 0
    with_rays = out.value
    assert lib.rgx_march_workspace_bytes(C.c_int64(1000), C.c_int64(0), C.c_int32(2048), C.byref(out)) == 0
    # the gradient block (64 bytes per Gaussian) and, growing with the ray count, the tile order of the backward
    assert 1000 * 64 <= out.value < with_rays and with_rays % 256 == 0 and with_rays - out.value >= (640000 // 64) * 4
    assert lib.rgx_march_records_bytes(C.c_int32(800), C.c_int32(800), C.c_int32(16384), C.byref(out)) == 0
    assert out.value == 100 * 100 * 16384 * 4
    assert lib.rgx_march_records_bytes(C.c_int32(801), C.c_int32(9), C.c_int32(1024), C.byref(out)) == 0
    assert out.value == 101 * 2 * 1024 * 4
    # hit lists plus on average 64 slots of sample sums per tile (the Python mirror's default)
    assert lib.rgx_march_records_bytes(C.c_int32(800), C.c_int32(800), C.c_int32(u_ox.REC_TILE_WORDS), C.byref(out)) == 0
    assert u_ox.REC_TILE_WORDS == 16384 + 64 * 8192 and out.value == 100 * 100 * u_ox.REC_TILE_WORDS * 4
    assert lib.rgx_check_plain_arith(None, None, C.c_int64(4), None, None) == -1
    for bad in ((0, 8, 16384), (8, 8, 512), (8, 8, 1026)):     # empty image, region too small, not a multiple of 4
        assert lib.rgx_march_records_bytes(C.c_int32(bad[0]), C.c_int32(bad[1]), C.c_int32(bad[2]), C.byref(out)) == -1
    lay = (C.c_size_t * 6)()
    assert lib.rgx_build_layout(C.c_int64(1000), lay) == 0 and lib.rgx_build_layout(C.c_int64(-1), lay) == -1
    assert lib.rgx_build_workspace_bytes(C.c_int64(1000), C.byref(out)) == 0
    assert lay[5] == 0 and all(0 < lay[i] < out.value and lay[i] % 256 == 0 for i in range(5)) and len(set(lay)) == 6
    assert lib.rgx_morton_workspace_bytes(C.c_int64(1000), C.byref(out)) == 0 and out.value > 0
    assert lib.rgx_knn_workspace_bytes(C.c_int64(1000), C.byref(out)) == 0 and out.value >= 1000 * 16


def test_bad_arguments_are_rejected_before_any_launch():
    lib = _lib.lib()
    null = C.c_void_p(0)
    eye = (C.c_float * 3)(0, 0, 0)
    assert lib.rgx_sh_forward(eye, null, null, null, null, null, 0, 7, C.c_int64(10), null, null) == -1       # degree
    assert lib.rgx_sh_forward(eye, null, null, null, null, null, 0, 3, C.c_int64(10), null, null) == -1       # null tensors
    assert lib.rgx_sh_forward(eye, null, null, null, null, null, 0, 3, C.c_int64(0), null, null) == 0         # empty: nothing to do
    assert lib.rgx_build(null, null, null, null, C.c_int64(10), C.c_float(0.1), null, C.c_size_t(0), null) == -1
    assert lib.rgx_reduce_supersampling(null, 8, 8, 1, 1, 0, null, null, null) == -1
    assert lib.rgx_gather_rows(1, null, null, null, null, C.c_int64(4), null) == -1
    assert lib.rgx_dist2_knn3(null, C.c_int64(4), null, null, C.c_size_t(0), null) == -1
    cam = _lib.RgxCamera()
    march = _lib.RgxMarch(0.0025, 0, 2048, 1, 1e-3)
    assert lib.rgx_march_forward(null, C.byref(cam), C.byref(march), null, C.c_int64(0), null, null, C.c_size_t(0), null,
                                 C.c_size_t(0), null, null) == -1                                           # no tree
    with pytest.raises(_lib.RgxError):
        _lib.check(-2)


def test_refit_of_an_unbuilt_or_mismatched_structure_is_refused_on_the_host():
    """update_acceleration_structure walks the tree a build left in the workspace, so the mirror refuses it
    for a structure that was never built and for anything but one box per Gaussian of that build -- before
    any launch (the library's own device-side check of the workspace header backs this up)."""
    gas = u_ox.AccelerationStructure.__new__(u_ox.AccelerationStructure)
    gas.n, gas.device, gas.built, gas.ws = 100, "cpu", False, torch.zeros(256, dtype=torch.uint8)
    with pytest.raises(_lib.RgxError, match="never built"):
        gas.update(torch.zeros(100, 6))
    with pytest.raises(_lib.RgxError, match="never built"):
        u_ox.update_acceleration_structure(gas, torch.zeros(100, 6))
    gas.built = True
    for bad in (torch.zeros(99, 6), torch.zeros(100, 5), torch.zeros(600)):
        with pytest.raises(_lib.RgxError, match=r"\(100, 6\)"):
            gas.update(bad)
    with pytest.raises(_lib.RgxError, match=r"\(100, 6\)"):
        gas.build_from_boxes(torch.zeros(101, 6))
    lib = _lib.lib()
    null = C.c_void_p(0)
    assert lib.rgx_refit_aabbs(null, C.c_int64(10), null, C.c_size_t(0), null) == -1


def test_missing_library_is_an_error_not_a_fallback(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/librgx.so")
    with pytest.raises(_lib.RgxError, match="no fallback"):
        _lib.lib()


def test_camera_constants_and_settings_mirror_the_reference():
    from raygaussx_amd import optix_utils as u_ox
    from raygaussx_amd.render_optix import RenderOptixSettings, default_settings
    cam = scenes.make_camera(1, 3, width=120, height=80)
    cs = u_ox.camera_struct(cam, supersampling=(2, 3))
    assert (cs.width, cs.height) == (240, 240)                       # optix_utils.py:252-253: size x supersampling
    np.testing.assert_allclose(list(cs.eye), cam.camera_center.numpy(), rtol=0, atol=0)
    rot = cam.world_view_transform[:3, :3].numpy()
    np.testing.assert_array_equal(np.array([list(cs.u), list(cs.v), list(cs.w)], np.float32), rot.T)   # columns 0..2
    assert math.isclose(cs.tan_half_fov_x, math.tan(cam.FoVx / 2), rel_tol=1e-6)
    assert math.isclose(cs.tan_half_fov_y, math.tan(cam.FoVy / 2), rel_tol=1e-6)
    assert (cs.principal_x, cs.principal_y) == (0.5, 0.5)
    # the reference's 18 positional arguments, in its order (render_optix.py:67-89)
    s = RenderOptixSettings("ctx", False, None, "pg_f", "pl_f", "pg_b", "pl_b", 0.0025, True, cam, 2048, 0, 7, 0, 0,
                            (1, 1), True, None)
    assert (s.dt_step, s.dynamic_sampling, s.max_prim_slice, s.iteration, s.white_background) == (0.0025, True, 2048, 7, True)
    assert s.t_eps == u_ox.TRANSMITTANCE_EPSILON == 1e-3 and s.record_hits and s.rec_tile_words >= 1024
    d = default_settings(cam, 0.005, True, 512, t_eps=1e-4)
    assert d.viewpoint_cam is cam and d.t_eps == 1e-4 and d.supersampling == (1, 1)
    # OptiX set-up calls are inert handles; only the kernel stages that exist can be asked for
    ctx = u_ox.create_context(log=None)
    mod = u_ox.create_module(ctx, None, stage="forward")
    assert u_ox.create_sbt(u_ox.create_program_groups(ctx, mod)) is not None
    assert u_ox.create_pipeline(ctx, u_ox.create_program_groups(ctx, mod), None) is not None
    assert u_ox.create_module(ctx, None, stage="gui").stage == "gui"     # the viewer's kernels exist (march_viewer, sh_viewer)
    with pytest.raises(ValueError):
        u_ox.create_module(ctx, None, stage="raster")


def test_scenes_are_seeded_and_shaped_as_the_configs_say():
    a = scenes.make_scene(0, n=500, sh_degree=2, seed=3)
    b = scenes.make_scene(0, n=500, sh_degree=2, seed=3)
    for k in a:
        assert torch.equal(a[k], b[k]), k
    assert a["color_features"].shape == (500, 3, 9) and a["quaternions"].shape == (500, 4)
    np.testing.assert_allclose(a["quaternions"].norm(dim=1).numpy(), 1.0, atol=1e-6)
    assert (a["scales"] > 0).all() and (a["densities"] > 0).all()
    assert scenes.CONFIGS[3]["t_eps"] == 1e-4 and scenes.CONFIGS[4]["n"] == 1_000_000
    cam = scenes.make_camera(2, 10)
    assert (cam.image_width, cam.image_height) == (1237, 822)
    fwd = cam.world_view_transform[:3, 2]
    to_origin = -cam.camera_center / cam.camera_center.norm()
    assert float(fwd @ to_origin) > 0.999                            # look-at cameras face the scene centre



def test_record_size_fits_a_memory_budget():
    """optix_utils.fit_tile_words: the full record if it fits, else fewer sample-sum slots, else the
    hit lists alone, else no record (host arithmetic on the library's size query)."""
    cs = _lib.RgxCamera()
    cs.width, cs.height = 3840, 2160                      # 129 600 tiles
    full = u_ox.records_bytes(cs, u_ox.REC_TILE_WORDS)
    assert full == 129600 * u_ox.REC_TILE_WORDS * 4 > 250e9
    assert u_ox.fit_tile_words(cs, u_ox.REC_TILE_WORDS, full) == u_ox.REC_TILE_WORDS
    w = u_ox.fit_tile_words(cs, u_ox.REC_TILE_WORDS, 100 * 2**30)
    assert u_ox.REC_LIST_WORDS < w < u_ox.REC_TILE_WORDS and (w - u_ox.REC_LIST_WORDS) % u_ox.REC_SLOT_WORDS == 0
    assert u_ox.records_bytes(cs, w) <= 100 * 2**30 < u_ox.records_bytes(cs, w + u_ox.REC_SLOT_WORDS)
    assert u_ox.fit_tile_words(cs, u_ox.REC_TILE_WORDS, 10 * 2**30) == u_ox.REC_LIST_WORDS
    assert u_ox.fit_tile_words(cs, u_ox.REC_TILE_WORDS, 2**30) == 0
    assert u_ox.fit_tile_words(cs, 4096, 10 * 2**30) == 4096     # a caller's small record is left alone


def test_bench_finds_its_stored_profile_figures():
    """bench.py reports HBM traffic and VALU instructions per launch from the summaries under profiles/ (a run
    without the profiler cannot count them): the lines it looks for are there, for both timed workloads."""
    import importlib.util
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for workload, key in (("c4_1M_800x800", "march_forward"), ("c4_1M_800x800", "march_backward"),
                          ("c3_3M_1920x1080_fwd", "march_forward")):
        traffic, source = bench.stored_traffic(workload, key)
        assert traffic and traffic > 1e8 and source.startswith("profiles/") and os.path.exists(os.path.join(root, source))
        bench._valu_measured = dict(value=600.0)        # what the probe kernel would measure on the GPU
        issue = bench.valu_issue(workload, key, 7.0, "cpu")
        assert issue and issue["instructions_per_launch"] > 1e9 and 0.0 < issue["frac"] <= 1.0 and issue["peak"] == 600.0
        assert bench.valu_issue(workload, key, 0.01, "cpu")["above_peak"]       # an impossible pairing is flagged, frac capped
    assert bench.stored_traffic("c4_1M_800x800", "no_such_kernel") == (None, None)
