"""GPU tests at the benchmark's full size (1 M Gaussians, 800x800: the workload of bench.py).

The oracle's brute-force hit search cannot render 640 000 rays of this scene, so parity is checked
(a) against the oracle on a strided sample of rays -- colours, march counters and, with dL/dimage
zero outside the sample, all gradients -- and (b) through properties that hold at any size: the
forward is deterministic, the backward is linear in dL/dimage, renumbering the Gaussians permutes
the gradients and leaves the image alone, forward and backward march the same hits.
"""
import numpy as np
import pytest
import torch

from raygaussx_amd import scenes

pytestmark = pytest.mark.gpu

N, W, H = 1_000_000, 800, 800
IMG_TOL, COS_MIN, REL_MAX = 1e-4, 0.9999, 1e-3
PARAMS = ("positions", "scales", "quaternions", "densities", "color_features")


@pytest.fixture(scope="module")
def gx():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import gpu_common
    from raygaussx_amd import _lib
    _lib.lib()
    return gpu_common


@pytest.fixture(scope="module")
def big():
    sc = scenes.scene_to_numpy(scenes.make_scene(4, n=N))
    sc = {k: sc[k] for k in PARAMS}
    return sc, scenes.make_camera(4, 3, width=W, height=H), scenes.CONFIGS[4]


def _step(msg):
    print(f"[gpu-step] {msg}", flush=True)


def test_ray_sample_against_the_oracle(gx, orc, big):
    sc, cam, cfg = big
    ids = np.linspace(0, W * H - 1, 384).astype(np.int64)
    img, st, ctx = orc.render_forward(sc, cam, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"], ray_ids=ids)
    assert img.shape == (W * H, 3)          # the oracle fills the sampled rays of a full-size image
    dloss = np.zeros((W * H, 3), np.float32)
    dloss[ids] = np.random.default_rng(11).normal(size=(len(ids), 3)).astype(np.float32)
    og, ost = orc.render_backward(sc, ctx, img, dloss)
    _step("full size: forward + backward, gradient of a 384-ray sample")
    out = gx.gpu_render(sc, cam, cfg, want_grad=dloss)
    assert np.abs(out["image"][ids] - img[ids]).max() <= IMG_TOL
    assert st["hit_pairs"] > 50000
    assert out["stats_fwd"]["hit_pairs"] == out["stats_bwd"]["hit_pairs"] > 1e8
    assert out["stats_fwd"]["slabs"] == out["stats_bwd"]["slabs"]
    assert out["stats_fwd"]["overflow_rays"] == 0
    for k in PARAMS:
        cos, rel = gx.cos_rel(out["grads"][k], og[k])
        assert cos >= COS_MIN and rel <= REL_MAX, (k, cos, rel)


def test_forward_is_deterministic_and_backward_is_linear(gx, big):
    sc, cam, cfg = big
    rng = np.random.default_rng(12)
    g1 = rng.normal(size=(W * H, 3)).astype(np.float32)
    g2 = rng.normal(size=(W * H, 3)).astype(np.float32)
    _step("full size: three backward passes")
    a = gx.gpu_render(sc, cam, cfg, want_grad=g1)
    b = gx.gpu_render(sc, cam, cfg, want_grad=g2)
    c = gx.gpu_render(sc, cam, cfg, want_grad=(0.5 * g1 - 2.0 * g2).astype(np.float32))
    assert np.array_equal(a["image"], b["image"]) and np.array_equal(a["image"], c["image"])
    assert a["stats_fwd"] == b["stats_fwd"] == c["stats_fwd"]
    assert 0.0 < a["image"].min() and a["image"].max() <= 1.0 + 1e-5 and a["image"].std() > 0.01
    for k in PARAMS:
        want = 0.5 * a["grads"][k] - 2.0 * b["grads"][k]
        cos, rel = gx.cos_rel(c["grads"][k], want)
        assert cos >= 1 - 1e-6 and rel <= 1e-4, (k, cos, rel)     # fp32 sums in different orders


def test_renumbering_the_gaussians_permutes_the_gradients(gx, big):
    sc, cam, cfg = big
    rng = np.random.default_rng(13)
    perm = rng.permutation(N)
    g = rng.normal(size=(W * H, 3)).astype(np.float32)
    _step("full size: permuted scene")
    a = gx.gpu_render(sc, cam, cfg, want_grad=g)
    b = gx.gpu_render({k: np.ascontiguousarray(v[perm]) for k, v in sc.items()}, cam, cfg, want_grad=g)
    # same Gaussians, same rays: the same hits (the tree is built on sorted codes, ties aside)
    for k in ("hit_pairs", "slabs", "empty_slabs", "rays_hit"):
        assert a["stats_fwd"][k] == b["stats_fwd"][k], k
    assert np.abs(a["image"] - b["image"]).max() <= 2e-6
    for k in PARAMS:
        cos, rel = gx.cos_rel(b["grads"][k], a["grads"][k][perm])
        assert cos >= 1 - 1e-6 and rel <= 1e-4, (k, cos, rel)


def test_record_sizes_give_the_same_gradients(gx, big):
    """The backward must not depend on how much of the forward's work the record kept: hit lists and
    sample sums for every tile (the default), a pool of sample sums that runs out half way (tiles
    with and without sums in one launch), hit lists only, and no record at all."""
    sc, cam, cfg = big
    g = np.random.default_rng(14).normal(size=(W * H, 3)).astype(np.float32)
    _step("full size: default record")
    ref = gx.gpu_render(sc, cam, cfg, want_grad=g)
    assert ref["stats_bwd"]["nodes_visited"] == 0
    # "uncounted": launched without a statistics block, i.e. the kernel variants that carry no counters
    for label, kw in (("sample-sum pool of 20 slots per tile", dict(rec_tile_words=16384 + 20 * 8192)),
                      ("hit lists only", dict(rec_tile_words=16384)),
                      ("no record", dict(record_hits=False)),
                      ("default record, uncounted", dict(stats=False)),
                      ("hit lists only, uncounted", dict(rec_tile_words=16384, stats=False)),
                      ("no record, uncounted", dict(record_hits=False, stats=False))):
        _step("full size: " + label)
        out = gx.gpu_render(sc, cam, cfg, want_grad=g, **kw)
        assert np.abs(out["image"] - ref["image"]).max() <= 2e-6
        if "stats_bwd" in out:
            assert out["stats_bwd"]["hit_pairs"] == ref["stats_bwd"]["hit_pairs"]
            assert (out["stats_bwd"]["nodes_visited"] > 0) == (label == "no record")
        for k in PARAMS:
            cos, rel = gx.cos_rel(out["grads"][k], ref["grads"][k])
            assert cos >= 1 - 1e-6 and rel <= 1e-4, (label, k, cos, rel)


def test_large_image_of_a_small_scene(gx, orc):
    """Images beyond about a megapixel are dealt to the XCDs in 8x8-tile blocks instead of 4x4 (a
    ragged 1101x1003 image here: 138x126 tiles, the last column and row partly outside).  Colours and
    gradients of a ray sample spread over the whole image against the oracle; an unmapped or
    doubly mapped block of tiles would show in both."""
    w, h = 1101, 1003
    sc = scenes.scene_to_numpy(scenes.make_scene(1, n=20000, seed=5))
    sc = {k: sc[k] for k in PARAMS}
    sc["scales"] = sc["scales"] * 3.0
    cam, cfg = scenes.make_camera(1, 2, width=w, height=h), scenes.CONFIGS[1]
    ids = np.unique(np.random.default_rng(15).integers(0, w * h, 3000))
    img, st, ctx = orc.render_forward(sc, cam, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"], ray_ids=ids)
    dloss = np.zeros((w * h, 3), np.float32)
    dloss[ids] = np.random.default_rng(16).normal(size=(len(ids), 3)).astype(np.float32)
    og, ost = orc.render_backward(sc, ctx, img, dloss)
    _step("1101x1003 image, 20000 Gaussians")
    out = gx.gpu_render(sc, cam, cfg, want_grad=dloss)
    assert st["hit_pairs"] > 20000
    assert np.abs(out["image"][ids] - img[ids]).max() <= IMG_TOL
    # every pixel was written: colours in range, none left at the all-zero of fresh memory, background white
    assert 0.0 <= out["image"].min() and out["image"].max() <= 1.0 + 1e-5
    assert not np.any(np.all(out["image"] == 0.0, axis=1))
    assert np.all(out["image"] == 1.0, axis=1).mean() > 0.2
    assert out["stats_fwd"]["hit_pairs"] == out["stats_bwd"]["hit_pairs"]
    for k in PARAMS:
        cos, rel = gx.cos_rel(out["grads"][k], og[k])
        assert cos >= COS_MIN and rel <= REL_MAX, (k, cos, rel)


def test_heavy_tailed_scene_ray_sample_against_the_oracle(gx, orc):
    """The unbounded-scene generator (configs[2]: a dense core plus a shell of large background
    Gaussians) at 1 M Gaussians and its own image size: crowded slabs that need several candidate
    tables, rays that cross hundreds of Gaussians.

    Fixed step: the usual gates.  Adaptive step (the configuration's own setting): the step is
    dt_dist / cbrt(T), and where a slab ends decides which Gaussians it holds, whether it is empty,
    and with that where the march restarts -- the last bit of cbrt or of exp (libm on the CPU, the
    hardware's on the GPU) can re-phase all later samples of a ray.  The oracle itself moves by
    7e-4 .. 9e-4 (relative L2 of the gradients; 9e-5 in the image) on exactly this input when its
    own step is scaled by 1 + 2^-23 (oracle.set_step_scale), so for this mode the gradient gate here
    is four times the usual one; the library measures 1.1e-3 .. 1.3e-3 against the oracle."""
    n, w, h = 1_000_000, 1237, 822
    sc = scenes.scene_to_numpy(scenes.make_scene(2, n=n, seed=3))
    sc = {k: sc[k] for k in PARAMS}
    cam = scenes.make_camera(2, 1, width=w, height=h)
    ids = np.unique(np.random.default_rng(17).integers(0, w * h, 256))
    dloss = np.zeros((w * h, 3), np.float32)
    dloss[ids] = np.random.default_rng(18).normal(size=(len(ids), 3)).astype(np.float32)
    for adaptive, rel_max in ((False, REL_MAX), (True, 4 * REL_MAX)):
        cfg = dict(scenes.CONFIGS[2], dynamic_sampling=adaptive)
        img, st, ctx = orc.render_forward(sc, cam, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"], ray_ids=ids)
        og, ost = orc.render_backward(sc, ctx, img, dloss)
        _step(f"configs[2] scene, 1 M Gaussians, 1237x822, adaptive step {adaptive}")
        out = gx.gpu_render(sc, cam, cfg, want_grad=dloss)
        assert st["hit_pairs"] > 20000
        assert np.abs(out["image"][ids] - img[ids]).max() <= IMG_TOL
        assert out["stats_fwd"]["hit_pairs"] == out["stats_bwd"]["hit_pairs"]
        for k in PARAMS:
            cos, rel = gx.cos_rel(out["grads"][k], og[k])
            assert cos >= COS_MIN and rel <= rel_max, (adaptive, k, cos, rel)


def test_tile_cooperative_and_per_ray_queries_find_the_same_hits(gx, orc, big):
    """Two implementations of the collect query on the GPU, at the benchmark's size: the per-ray
    skip-link traversal (rgx_trace_segments: the plain `/` and sqrtf(), pinned against the oracle on
    small scenes) and the tile-cooperative one the march kernels use (rgx_collect_tiles: candidate
    tables, the short division and square-root sequences).  Same segments, same hit sets, for every
    pixel and at several depths -- some ten million ray-Gaussian hits."""
    from raygaussx_amd import optix_utils as u_ox
    from raygaussx_amd.render_optix import compute_rgb
    sc, cam, cfg = big
    d = gx.to_dev(sc)
    gas = u_ox.AccelerationStructure(N, gx.DEV).build_from_gaussians(d["positions"], d["scales"], d["quaternions"], d["densities"])
    eye = torch.as_tensor(np.asarray(cam.camera_center, np.float32))
    rgb = compute_rgb(eye.to(gx.DEV), d["positions"], d["color_features"], None, None, None, 0, 3)
    ps = u_ox.pack_prims(gas, eye, d["positions"], d["scales"], d["quaternions"], d["densities"], rgb)
    dirs = torch.from_numpy(orc.ray_dirs(orc.camera_struct(cam))).to(gx.DEV)
    cams = u_ox.camera_struct(cam)
    cap, total = 128, 0
    for t0 in (2.6, 3.4, 4.1, 5.0):
        tlo = torch.full((W * H,), t0, dtype=torch.float32, device=gx.DEV)
        thi = tlo + 0.08
        _step(f"both collect queries, slab at t = {t0}")
        c_tile, i_tile = u_ox.collect_tiles(gas, cams, ps, tlo, thi, cap)
        c_ray, i_ray = u_ox.trace_segments(gas, ps, eye, dirs, tlo, thi, cap)
        assert int(c_ray.min()) >= 0 and int(c_ray.max()) < cap          # no list was cut
        assert torch.equal(c_tile, c_ray)
        # -1 pads the unused tail of a row in both; sorted rows must agree
        assert torch.equal(torch.sort(i_tile, dim=1).values, torch.sort(i_ray, dim=1).values)
        total += int(c_ray.sum())
    assert total > 5_000_000
