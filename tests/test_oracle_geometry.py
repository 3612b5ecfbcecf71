"""Pins the geometric half of the CPU oracle against closed forms and float64 brute force."""
import math

import numpy as np
import torch

import f64ref
from raygaussx_amd import scenes


def _small_scene(n=200, seed=3):
    sc = scenes.make_scene(0, n=n, seed=seed)
    return scenes.scene_to_numpy(sc)


def test_aabb_closed_form_and_surface_samples(orc):
    sc = _small_scene(300)
    boxes, bmin, bmax = orc.aabb(sc["positions"], sc["scales"], sc["quaternions"], sc["densities"])
    q = torch.tensor(sc["quaternions"], dtype=torch.float64)
    R = f64ref.rot_from_quat(q).numpy()
    s = sc["scales"].astype(np.float64)
    rho = sc["densities"].astype(np.float64)
    k = np.sqrt(np.maximum(2.0 * np.log(rho / 0.1), 0.0))
    cov_diag = np.einsum("nij,nj,nij->ni", R, s * s, R)      # diag(R S^2 R^T)
    half = k[:, None] * np.sqrt(cov_diag)
    c = sc["positions"].astype(np.float64)
    np.testing.assert_allclose(boxes[:, :3], c - half, rtol=2e-5, atol=1e-6)
    np.testing.assert_allclose(boxes[:, 3:], c + half, rtol=2e-5, atol=1e-6)
    # dense surface samples of {x : |S^-1 R^T (x-c)| = k} stay inside and touch each face
    rng = np.random.default_rng(0)
    u = rng.normal(size=(20000, 3))
    u /= np.linalg.norm(u, axis=1, keepdims=True)
    for n in range(0, 300, 37):
        pts = c[n] + (R[n] @ (u * (k[n] * s[n])).T).T
        assert (pts >= boxes[n, :3] - 1e-6).all() and (pts <= boxes[n, 3:] + 1e-6).all()
        if k[n] > 0:
            ext = pts.max(0) - pts.min(0)
            np.testing.assert_allclose(ext, boxes[n, 3:] - boxes[n, :3], rtol=2e-3)
    np.testing.assert_array_equal(bmin, boxes[:, :3].min(0))
    np.testing.assert_array_equal(bmax, boxes[:, 3:].max(0))


def test_aabb_identity_quaternion_and_invisible(orc):
    pos = np.array([[0.5, -1.0, 2.0], [1.0, 1.0, 1.0]], np.float32)
    scale = np.array([[0.1, 0.2, 0.3], [0.5, 0.5, 0.5]], np.float32)
    quat = np.array([[1, 0, 0, 0], [1, 0, 0, 0]], np.float32)
    dens = np.array([0.8, 0.05], np.float32)     # second one is below the 0.1 threshold
    boxes, _, _ = orc.aabb(pos, scale, quat, dens)
    k = math.sqrt(2 * math.log(0.8 / 0.1))
    np.testing.assert_allclose(boxes[0], np.r_[pos[0] - k * scale[0], pos[0] + k * scale[0]], rtol=1e-6)
    np.testing.assert_array_equal(boxes[1], np.r_[pos[1], pos[1]])   # d clamped to 0


def test_pack_prims_layout_and_cutoff(orc):
    sc = _small_scene(100)
    eye = np.array([1.0, 2.0, 3.0], np.float32)
    rgb = np.random.default_rng(1).random((100, 3), dtype=np.float32)
    prims = orc.pack_prims(eye, sc["positions"], sc["scales"], sc["quaternions"], sc["densities"], rgb)
    rho = sc["densities"]
    k = prims[:, 7]
    vis = rho > 0.1
    # the Gaussian is truncated where rho * exp(-k^2/2) equals the threshold
    np.testing.assert_allclose(rho[vis] * np.exp(-0.5 * k[vis].astype(np.float64) ** 2), 0.1, rtol=1e-5)
    assert np.isnan(k[rho < 0.1]).all()
    np.testing.assert_array_equal(prims[:, :3], eye[None] - sc["positions"])
    np.testing.assert_array_equal(prims[:, 3], 0)
    np.testing.assert_allclose(prims[vis, 4:7] * k[vis, None] * sc["scales"][vis], 1.0, rtol=1e-6)
    np.testing.assert_array_equal(prims[:, 8:12], sc["quaternions"])
    np.testing.assert_allclose(prims[:, 12:15], rgb * rho[:, None], rtol=1e-7)
    np.testing.assert_array_equal(prims[:, 15], rho)


def test_ray_dirs_match_pinhole_model(orc):
    for cfg, idx in ((0, 0), (2, 17)):
        cam = scenes.make_camera(cfg, idx, width=61, height=37)
        cs = orc.camera_struct(cam)
        d = orc.ray_dirs(cs)
        ref = f64ref.ray_dirs_pinhole(cam)
        np.testing.assert_allclose(d, ref, atol=3e-7)
    cam = scenes.make_camera(0, 0, width=33, height=33)      # odd size: centre pixel looks along forward
    d = orc.ray_dirs(orc.camera_struct(cam), [16 * 33 + 16])
    np.testing.assert_allclose(d[0], cam.world_view_transform[:3, 2].numpy(), atol=1e-7)
    # pixel (0,0) is top-left: right-axis component negative, down-axis component negative
    d0 = orc.ray_dirs(orc.camera_struct(cam), [0])[0]
    assert d0 @ cam.world_view_transform[:3, 0].numpy() < 0 and d0 @ cam.world_view_transform[:3, 1].numpy() < 0


def test_supersampling_scales_the_ray_grid(orc):
    cam = scenes.make_camera(0, 0, width=8, height=4)
    cs = orc.camera_struct(cam, supersampling=(2, 3))
    assert (cs.width, cs.height) == (16, 12)


def _f64_hits(sc, eye, dirs, tlo, thi, margin=1e-4):
    valid, t_in, t_out, closest2 = f64ref.ellipsoid_roots(eye, dirs, sc["positions"], sc["scales"],
                                                         sc["quaternions"], sc["densities"])
    tlo = torch.as_tensor(tlo, dtype=torch.float64)[:, None]
    thi = torch.as_tensor(thi, dtype=torch.float64)[:, None]
    lo = torch.maximum(tlo, t_in)
    hi = torch.minimum(thi, t_out)
    hit = valid & (closest2 < 1 - 1e-7) & (lo <= hi)
    # pairs the fp32 predicate may legitimately decide either way
    fragile = (closest2 - 1).abs() < margin
    fragile |= ((lo - hi).abs() < margin * (1 + hi.abs()))
    return hit.numpy(), lo.numpy(), fragile.numpy()


def test_segment_hits_match_float64_closed_form(orc):
    sc = _small_scene(400, seed=5)
    sc["scales"] = sc["scales"] * 3.0        # fatter Gaussians: more (ray, prim) pairs to decide
    rng = np.random.default_rng(2)
    eye = np.array([2.5, 1.5, 2.0], np.float32)
    prims = orc.pack_prims(eye, sc["positions"], sc["scales"], sc["quaternions"], sc["densities"],
                           np.zeros((400, 3), np.float32))
    tgt = rng.uniform(-1, 1, size=(300, 3))
    dirs = tgt - eye[None]
    dirs = (dirs / np.linalg.norm(dirs, axis=1, keepdims=True)).astype(np.float32)
    tlo = rng.uniform(1.0, 4.0, 300).astype(np.float32)
    thi = (tlo + rng.uniform(0.05, 1.0, 300)).astype(np.float32)
    counts, ids = orc.trace_segments(prims, dirs, tlo, thi, cap=400)
    hit, lo, fragile = _f64_hits(sc, eye, dirs, tlo, thi)
    assert hit.sum() > 200
    for r in range(300):
        got = set(ids[r, :counts[r]].tolist())
        want = set(np.nonzero(hit[r])[0].tolist())
        diff = got ^ want
        assert all(fragile[r, p] for p in diff), (r, diff)
    # first-hit = smallest clipped entry root over the hit set, -1 when empty
    fh = orc.first_hit(prims, dirs, tlo, thi)
    for r in range(300):
        solid = hit[r] & ~fragile[r]
        if hit[r].sum() == 0 and not fragile[r].any():
            assert fh[r] == -1.0
        elif solid.any() and not (fragile[r] & ~solid).any():
            np.testing.assert_allclose(fh[r], lo[r][hit[r]].min(), rtol=2e-5, atol=2e-5)


def test_isotropic_gaussian_is_textbook_sphere(orc):
    # k*s sphere of radius rad at distance 5 straight ahead
    rho = 0.1 * math.exp(0.5 * 2.0 ** 2)                # k = 2
    s = 0.25
    rad = 2.0 * s
    pos = np.array([[5.0, 0.0, 0.0]], np.float32)
    prims = orc.pack_prims(np.zeros(3, np.float32), pos, np.full((1, 3), s, np.float32),
                           np.array([[0.6, 0.0, 0.8, 0.0]], np.float32), np.array([rho], np.float32),
                           np.zeros((1, 3), np.float32))
    offs = np.array([0.0, 0.3, 0.49, 0.51], np.float64)   # lateral offsets of the aim point
    dirs = np.stack([np.full(4, 5.0), offs, np.zeros(4)], 1)
    dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
    fh = orc.first_hit(prims, dirs.astype(np.float32), np.zeros(4, np.float32), np.full(4, 100, np.float32))
    for i in range(4):
        b = dirs[i] @ pos[0].astype(np.float64)
        disc = b * b - (25.0 - rad * rad)
        if disc > 0:
            np.testing.assert_allclose(fh[i], b - math.sqrt(disc), rtol=1e-5)
        else:
            assert fh[i] == -1.0
    # a ray that starts inside reports t = tmin; a segment entirely behind the exit misses
    inside = orc.first_hit(prims, dirs[:1].astype(np.float32), np.array([5.0], np.float32), np.array([9.0], np.float32))
    assert inside[0] == 5.0
    behind = orc.first_hit(prims, dirs[:1].astype(np.float32), np.array([5.6], np.float32), np.array([9.0], np.float32))
    assert behind[0] == -1.0


def test_rigid_motion_equivariance(orc):
    sc = _small_scene(150, seed=9)
    sc["scales"] = sc["scales"] * 3.0
    rng = np.random.default_rng(4)
    eye = np.array([3.0, 0.5, 1.0], np.float64)
    tgt = rng.uniform(-1, 1, size=(120, 3))
    dirs = tgt - eye
    dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
    tlo = np.full(120, 1.0, np.float32)
    thi = np.full(120, 6.0, np.float32)
    z = np.zeros((150, 3), np.float32)
    prims = orc.pack_prims(eye, sc["positions"], sc["scales"], sc["quaternions"], sc["densities"], z)
    c0, i0 = orc.trace_segments(prims, dirs, tlo, thi, 150)
    # rotate the world by a random rotation g and translate by tr
    g = torch.randn(4, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    g = g / g.norm()
    G = f64ref.rot_from_quat(g).numpy()
    tr = np.array([0.3, -2.0, 1.1])
    q = sc["quaternions"].astype(np.float64)
    gw, gx, gy, gz = g.numpy()
    qw, qx, qy, qz = q.T
    q2 = np.stack([gw * qw - gx * qx - gy * qy - gz * qz, gw * qx + gx * qw + gy * qz - gz * qy,
                   gw * qy - gx * qz + gy * qw + gz * qx, gw * qz + gx * qy - gy * qx + gz * qw], 1)
    pos2 = sc["positions"].astype(np.float64) @ G.T + tr
    prims2 = orc.pack_prims(G @ eye + tr, pos2, sc["scales"], q2, sc["densities"], z)
    c1, i1 = orc.trace_segments(prims2, dirs @ G.T, tlo, thi, 150)
    same = sum(set(i0[r, :c0[r]]) == set(i1[r, :c1[r]]) for r in range(120))
    assert same >= 117      # identical up to a few grazing pairs decided by rounding
    assert c0.sum() > 100


def test_invisible_prims_are_never_hit(orc):
    pos = np.zeros((3, 3), np.float32)
    scale = np.full((3, 3), 0.5, np.float32)
    quat = np.tile(np.array([[1, 0, 0, 0]], np.float32), (3, 1))
    dens = np.array([0.05, 0.1, 0.0], np.float32)      # below, at, and zero
    prims = orc.pack_prims(np.array([0, 0, -3], np.float32), pos, scale, quat, dens, np.zeros((3, 3), np.float32))
    d = np.array([[0, 0, 1]], np.float32)
    c, _ = orc.trace_segments(prims, d, np.array([0], np.float32), np.array([10], np.float32), 8)
    assert c[0] == 0


def test_collect_truncation_is_reported(orc):
    n = 12
    pos = np.zeros((n, 3), np.float32)
    pos[:, 2] = np.linspace(1, 2, n)
    prims = orc.pack_prims(np.zeros(3, np.float32), pos, np.full((n, 3), 0.2, np.float32),
                           np.tile(np.array([[1, 0, 0, 0]], np.float32), (n, 1)), np.full(n, 1.0, np.float32),
                           np.zeros((n, 3), np.float32))
    d = np.array([[0, 0, 1]], np.float32)
    c, ids = orc.trace_segments(prims, d, np.array([0], np.float32), np.array([10], np.float32), 5)
    assert c[0] == -5 and ids[0].tolist() == [0, 1, 2, 3, 4]
    c, _ = orc.trace_segments(prims, d, np.array([0], np.float32), np.array([10], np.float32), n)
    assert c[0] == n


def test_morton_codes_match_naive_bit_loop(orc):
    rng = np.random.default_rng(11)
    pos = rng.normal(size=(5000, 3)).astype(np.float32)
    codes = orc.morton_codes(pos)
    mn, mx = pos.min(0), pos.max(0)
    scale = (np.float32(1023.0) / ((mx - mn) + np.float32(1e-9))).astype(np.float32)
    q = ((pos - mn) * scale).astype(np.int32)
    want = np.zeros(5000, np.int64)
    for i in range(10):
        for a in range(3):
            want |= ((q[:, a] >> i) & 1).astype(np.int64) << (3 * i + a)
    np.testing.assert_array_equal(codes, want)
    assert q.max() <= 1023 and q.min() == 0
    order = orc.morton_order(pos)
    assert sorted(order.tolist()) == list(range(5000))
    assert (np.diff(codes[order]) >= 0).all()
    # x is the lowest interleaved bit: moving only along x by one cell flips bit 0
    two = np.array([[0, 0, 0], [1, 1, 1], [1.0 / 1023 * 1.0001, 0, 0]], np.float32)
    c = orc.morton_codes(two)
    assert c[0] == 0 and c[2] == 1 and c[1] == (1 << 30) - 1


def test_reduce_supersampling_is_the_block_mean(orc):
    """utils/general_utils.py:489-502: each output pixel is the mean of its fx x fy block of rays
    (checked against a reshape-mean in float64), and factor (1, 1) is the identity."""
    rng = np.random.default_rng(0)
    W, H = 7, 5
    for fx, fy in ((1, 1), (2, 1), (1, 3), (2, 2), (3, 2)):
        rays = rng.random((W * fx * H * fy, 3), dtype=np.float32)
        got = orc.reduce_supersampling(W, H, rays, (fx, fy))
        want = rays.astype(np.float64).reshape(H, fy, W, fx, 3).mean(axis=(1, 3))
        assert got.shape == (H, W, 3) and got.dtype == np.float32
        np.testing.assert_allclose(got, want, rtol=0, atol=2e-7)
        if (fx, fy) == (1, 1):
            np.testing.assert_array_equal(got.reshape(-1, 3), rays)


def test_knn3_mean_distance_matches_a_kd_tree(orc):
    """distCUDA2 (simple_knn.cu:137-184) against scipy's cKDTree in float64 (k = 4: the point itself
    and its three nearest), with duplicated points and fewer than four points."""
    from scipy.spatial import cKDTree
    rng = np.random.default_rng(3)
    for n in (4, 50, 3000):
        p = rng.normal(size=(n, 3)).astype(np.float32)
        if n == 50:
            p[10] = p[11]                       # a duplicate is a neighbour at distance 0
        d, _ = cKDTree(p.astype(np.float64)).query(p.astype(np.float64), k=4)
        want = (d[:, 1:] ** 2).mean(1)
        np.testing.assert_allclose(orc.dist2_knn3(p), want, rtol=2e-6, atol=1e-12)
    two = orc.dist2_knn3(np.array([[0, 0, 0], [1, 0, 0]], np.float32))
    assert np.isinf(two).all()                 # (1 + FLT_MAX + FLT_MAX) / 3 overflows, as in the reference


def test_culled_candidate_search_equals_the_brute_force(orc):
    """The bounding-volume tree the timed CPU baseline uses (orc_cull_build) must change nothing: the
    candidate lists are those of the loop over all primitives, so images, counters, hit lists and
    gradients are equal in every bit -- for an object scene, for the heavy-tailed one with the camera
    inside the cloud, with invisible Gaussians (k undefined) and with axis-parallel rays."""
    from raygaussx_amd import scenes
    for config, n, w, h, mult in ((0, 3000, 40, 32, 2.0), (2, 8000, 36, 28, 3.0), (1, 5000, 33, 33, 4.0)):
        sc = scenes.scene_to_numpy(scenes.make_scene(config, n=n, sh_degree=1, seed=50 + config))
        sc["scales"] = sc["scales"] * mult
        sc["densities"][::7] = 0.05                                  # below the threshold: never hit
        cam = scenes.look_at_camera((3.0, 0.0, 0.0), fov_x_deg=30, width=w, height=h) if config == 1 else \
            scenes.make_camera(config, 2, width=w, height=h)
        cfg = scenes.CONFIGS[config]
        img, st, ctx = orc.render_forward(sc, cam, cfg["dt_step"], cfg["dynamic_sampling"], 512)
        dloss = np.random.default_rng(config).normal(size=img.shape).astype(np.float32)
        g, _ = orc.march_backward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], img, dloss)
        slabs, _ = orc.march_trace(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], (h // 2) * w + w // 2)
        orc.cull_build(ctx["prims"])
        try:
            img2, st2 = orc.march_forward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"])
            g2, _ = orc.march_backward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], img, dloss)
            slabs2, _ = orc.march_trace(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], (h // 2) * w + w // 2)
        finally:
            orc.cull_free()
        assert st == st2 and st["hit_pairs"] > 2000
        assert np.array_equal(img, img2)
        for k in g:
            assert np.array_equal(g[k], g2[k]), k
        assert len(slabs) == len(slabs2) and all(a[:4] == b[:4] and np.array_equal(a[4], b[4]) for a, b in zip(slabs, slabs2))
