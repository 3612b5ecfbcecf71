"""Pins the marching half of the CPU oracle: analytic optical depth, compositing
identities, an independent float64 march, torch.autograd and central differences."""
import math

import numpy as np
import torch

import f64ref
from raygaussx_amd import scenes


def _axis_camera(width=9, height=9, dist=4.0):
    return scenes.look_at_camera((dist, 0.0, 0.0), fov_x_deg=10.0, width=width, height=height)


def _render(orc, sc, cam, dt, dynamic=False, cap=256, white=True, eps=1e-3, ray_ids=None):
    return orc.render_forward(sc, cam, dt, dynamic, cap, white_background=white, t_eps=eps, ray_ids=ray_ids)


def _one_gaussian(rho, s, rgb, pos=(0.0, 0.0, 0.0)):
    sh = np.zeros((1, 3, 1), np.float32)
    sh[0, :, 0] = (np.asarray(rgb) - 0.5) / 0.28209479177387814   # degree-0 colour = 0.5 + C0*sh
    return dict(positions=np.array([pos], np.float32), scales=np.full((1, 3), s, np.float32),
                quaternions=np.array([[1, 0, 0, 0]], np.float32), densities=np.array([rho], np.float32),
                color_features=sh)


def test_single_isotropic_gaussian_matches_erf_optical_depth(orc):
    rho, s, rgb = 3.0, 0.05, (0.2, 0.6, 0.9)
    k = math.sqrt(2 * math.log(rho / 0.1))
    tau = rho * s * math.sqrt(2 * math.pi) * math.erf(k / math.sqrt(2))
    want = np.array(rgb) * (1 - math.exp(-tau)) + math.exp(-tau)         # white background
    cam = _axis_camera()
    centre = 4 * 9 + 4
    errs = []
    for dt in (0.004, 0.002, 0.001):
        img, st, _ = _render(orc, _one_gaussian(rho, s, rgb), cam, dt)
        errs.append(np.abs(img[centre] - want).max())
        assert st["overflow_rays"] == 0
        # midpoint rule is O(dt^2) inside the support; the 0.1 density jump at each of the two
        # truncation boundaries adds at most 0.1*dt/2 of optical depth
        assert errs[-1] < 0.1 * dt + 1e-5
    assert errs[2] < 2e-5
    # black background drops the transmitted term only
    img_b, _, _ = _render(orc, _one_gaussian(rho, s, rgb), cam, 0.001, white=False)
    np.testing.assert_allclose(img_b[centre], np.array(rgb) * (1 - math.exp(-tau)), atol=3e-5)


def test_empty_and_missed_scenes_return_background(orc):
    cam = _axis_camera()
    img, st, _ = _render(orc, _one_gaussian(0.05, 0.05, (0.1, 0.2, 0.3)), cam, 0.002)   # below threshold
    np.testing.assert_array_equal(img, 1.0)
    assert st["rays_hit"] == 0
    img, _, _ = _render(orc, _one_gaussian(0.05, 0.05, (0.1, 0.2, 0.3)), cam, 0.002, white=False)
    np.testing.assert_array_equal(img, 0.0)
    # a Gaussian behind the camera is inside the scene bbox but no ray reaches it
    img, st, _ = _render(orc, _one_gaussian(2.0, 0.05, (0.1, 0.2, 0.3), pos=(8.0, 0, 0)), cam, 0.002)
    np.testing.assert_array_equal(img, 1.0)


def test_two_disjoint_gaussians_composite_front_to_back(orc):
    cam = _axis_camera()
    centre = 4 * 9 + 4
    a = _one_gaussian(1.5, 0.04, (0.9, 0.1, 0.2), pos=(0.6, 0, 0))     # nearer to the camera at x=4
    b = _one_gaussian(2.5, 0.05, (0.1, 0.8, 0.3), pos=(-0.7, 0, 0))
    both = {k: np.concatenate([a[k], b[k]]) for k in a}
    dt = 0.001
    ia, _, _ = _render(orc, a, cam, dt, white=False)
    ib, _, _ = _render(orc, b, cam, dt, white=False)
    iab, st, _ = _render(orc, both, cam, dt, white=False)
    ta = math.exp(-1.5 * 0.04 * math.sqrt(2 * math.pi) * math.erf(math.sqrt(2 * math.log(15.0)) / math.sqrt(2)))
    np.testing.assert_allclose(iab[centre], ia[centre] + ta * ib[centre], atol=3e-5)
    assert st["empty_slabs"] >= 1        # the gap between them is skipped by a first-hit query


def _f64_march_image(sc, cam, dt, ids, eps=1e-3):
    """Independent fixed-step march in float64: sample i of the ray sits at
    t_first + (i + 0.5) dt on a grid anchored at the first hit, restarted after
    every empty slab at the next hit; 32-sample slabs, termination every 16."""
    eye = cam.camera_center.double().numpy()
    dirs = f64ref.ray_dirs_pinhole(cam, ids)
    pos, scale, quat, dens = (sc[k].astype(np.float64) for k in ("positions", "scales", "quaternions", "densities"))
    rgb = 0.5 + 0.28209479177387814 * sc["color_features"][:, :, 0].astype(np.float64)
    valid, t_in, t_out, closest2 = f64ref.ellipsoid_roots(eye, dirs, pos, scale, quat, dens)
    valid = (valid & (closest2 < 1 - 1e-7)).numpy()
    t_in, t_out = t_in.numpy(), t_out.numpy()
    R = f64ref.rot_from_quat(torch.tensor(quat)).numpy()
    kk = 2 * np.log(dens / 0.1)
    out = np.ones((len(ids), 3))
    for r in range(len(ids)):
        cand = np.nonzero(valid[r] & (t_out[r] >= 0))[0]
        if len(cand) == 0:
            continue
        tb = max(t_in[r, cand].min(), 0.0)
        tend = t_out[r, cand].max()
        T, C = 1.0, np.zeros(3)
        L = 32 * dt
        while tb <= tend and T > eps:
            hit = cand[(t_in[r, cand] <= tb + L) & (t_out[r, cand] >= tb)]
            if len(hit) == 0:
                nxt = cand[t_out[r, cand] >= tb + L]
                if len(nxt) == 0:
                    break
                tb = max(t_in[r, nxt].min(), tb + L)
                continue
            t = tb + dt * (np.arange(32) + 0.5)
            x = eye[None] + t[:, None] * dirs[r][None]
            loc = np.einsum("hji,hsj->hsi", R[hit], x[None] - pos[hit][:, None]) / scale[hit][:, None]
            power = (loc ** 2).sum(-1)
            w = np.exp(-0.5 * power) * (power < kk[hit][:, None])
            sig = (dens[hit][:, None] * w).sum(0)
            col = ((dens[hit][:, None] * w)[:, :, None] * rgb[hit][:, None]).sum(0)
            for base in (0, 16):
                if T <= eps:
                    break
                for i in range(base, base + 16):
                    xx = sig[i] * dt
                    ww = math.exp(-xx)
                    C += T * dt * (1 - ww) / max(xx, 1e-6) * col[i]
                    T *= ww
            tb += L
        out[r] = C + T
    return out


def _f64_march_adaptive(sc, cam, dt0, ids, eps=1e-3, dynamic=True):
    """Independent float64 march with the step rule of gaussians_aabb.cu:266-273 recomputed from its OWN
    transmittance and position: dt = min(max(t / 1024, dt0) * T^(-1/3), 4 dt0), slab = 32 dt; every
    sample's Mahalanobis distance evaluated directly.  Returns the image, per ray the blended slabs
    [(t, dt, sorted ids)], and per ray a margin: the smallest relative distance between a decision the
    march took (a Gaussian's entry or exit against a slab boundary, T against eps) and its flipping
    point.  A float32 march of the same rule can only differ in its slab sequence on rays whose margin
    is of the order of float32 rounding."""
    eye = cam.camera_center.double().numpy()
    dirs = f64ref.ray_dirs_pinhole(cam, ids)
    pos, scale, quat, dens = (sc[k].astype(np.float64) for k in ("positions", "scales", "quaternions", "densities"))
    rgb = 0.5 + 0.28209479177387814 * sc["color_features"][:, :, 0].astype(np.float64)
    valid, t_in, t_out, closest2 = f64ref.ellipsoid_roots(eye, dirs, pos, scale, quat, dens)
    near_graze = ((closest2 - (1 - 1e-7)).abs() < 1e-5).numpy()     # the predicate's disc > 1e-7 test
    valid = (valid & (closest2 < 1 - 1e-7)).numpy()
    t_in, t_out = t_in.numpy(), t_out.numpy()
    R = f64ref.rot_from_quat(torch.tensor(quat)).numpy()
    kk = 2 * np.log(dens / 0.1)
    out = np.ones((len(ids), 3))
    seqs, margins = [], []
    for r in range(len(ids)):
        cand = np.nonzero(valid[r] & (t_out[r] >= 0))[0]
        seq, margin = [], np.inf
        if near_graze[r].any():
            margin = 0.0
        if len(cand):
            tb = max(t_in[r, cand].min(), 0.0)
            tend = t_out[r, cand].max()
            T, C = 1.0, np.zeros(3)
            dt = dt0
            while tb <= tend and T > eps:
                margin = min(margin, abs(T - eps) / eps)
                if dynamic:
                    dt = min(max(tb / 1024.0, dt0) * T ** (-1.0 / 3.0), 4.0 * dt0)
                L = 32 * dt
                ci, co = t_in[r, cand], t_out[r, cand]
                margin = min(margin, np.abs(ci - (tb + L)).min() / (tb + L), np.abs(co - tb).min() / tb)
                hit = cand[(ci <= tb + L) & (co >= tb)]
                if len(hit) == 0:
                    nxt = cand[co >= tb + L]
                    if len(nxt) == 0:
                        break
                    tb = max(t_in[r, nxt].min(), tb + L)
                    continue
                seq.append((tb, dt, np.sort(hit)))
                t = tb + dt * (np.arange(32) + 0.5)
                x = eye[None] + t[:, None] * dirs[r][None]
                loc = np.einsum("hji,hsj->hsi", R[hit], x[None] - pos[hit][:, None]) / scale[hit][:, None]
                power = (loc ** 2).sum(-1)
                w = np.exp(-0.5 * power) * (power < kk[hit][:, None])
                sig = (dens[hit][:, None] * w).sum(0)
                col = ((dens[hit][:, None] * w)[:, :, None] * rgb[hit][:, None]).sum(0)
                for base in (0, 16):
                    if T <= eps:
                        break
                    if base:
                        margin = min(margin, abs(T - eps) / eps)
                    for i in range(base, base + 16):
                        xx = sig[i] * dt
                        ww = math.exp(-xx)
                        C += T * dt * (1 - ww) / max(xx, 1e-6) * col[i]
                        T *= ww
                tb += L
            margin = min(margin, abs(T - eps) / eps)
            out[r] = C + T
        seqs.append(seq)
        margins.append(margin)
    return out, seqs, np.array(margins)


def test_adaptive_step_matches_independent_float64_march(orc):
    """Pins the dynamic_sampling branch (gaussians_aabb.cu:266-273).  The float64 march above recomputes
    every step from its own transmittance; on rays where none of its decisions sits within 1e-4 of
    flipping, the oracle must have marched the same slabs -- same count, same (t, dt) to float32
    accuracy, same hit sets -- and produced the same colour.  A cbrt for the rcbrt, a dropped
    4 dt0 cap, a wrong 1024 or a step taken from the previous slab's T all change dt by far more."""
    checked = 0
    for seed, n, mult, res in ((3, 1500, 3.0, 20), (8, 4000, 2.0, 16)):
        sc = scenes.scene_to_numpy(scenes.make_scene(2, n=n, sh_degree=0, seed=seed))
        sc["scales"] = sc["scales"] * mult
        cam = scenes.make_camera(2, 1, width=res, height=res)
        ids = np.arange(res * res)
        dt0 = 0.005
        img, st, ctx = _render(orc, sc, cam, dt0, dynamic=True, cap=n)
        want, seqs, margins = _f64_march_adaptive(sc, cam, dt0, ids)
        robust = margins > 1e-4
        assert robust.mean() > 0.8 and st["overflow_rays"] == 0
        steps_seen = set()
        for r in np.nonzero(robust)[0]:
            slabs, _ = orc.march_trace(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], int(r))
            got = [(tb, dt, np.sort(i)) for tb, dt, lo, hi, i in slabs if len(i)]
            assert len(got) == len(seqs[r]), (seed, r, len(got), len(seqs[r]))
            for (tb, dt, hit), (tb64, dt64, hit64) in zip(got, seqs[r]):
                assert abs(tb - tb64) <= 2e-5 * tb64 and abs(dt - dt64) <= 2e-5 * dt64, (seed, r, tb, tb64, dt, dt64)
                assert np.array_equal(hit, hit64), (seed, r)
                steps_seen.add(round(dt64 / dt0, 2))
            checked += len(got)
        # the steps met span the rule's whole range: dt0 (T = 1 near the camera) up to the 4 dt0 cap
        assert min(steps_seen) < 1.05 and max(steps_seen) == 4.0 and len(steps_seen) > 20
        err = np.abs(img[ids] - want).max(1)[robust]
        assert np.quantile(err, 0.98) < 2e-5 and err.max() < 6e-4     # one flipped cut-off sample costs <= 0.1 * 4 dt0 * |dc|
    assert checked > 1500


def test_adaptive_step_closed_forms_on_one_gaussian(orc):
    """The step rule against what the mathematics fixes, on one isotropic Gaussian on the ray axis
    (transmittance known in closed form through erf):
    (i) the first slab has T = 1, so dt = max(t_enter / 1024, dt0) exactly -- the distance term alone,
        on both sides of its max and up to where it alone reaches the cap;
    (ii) further in, dt = dt_dist * T(t)^(-1/3) with the analytic T(t);
    (iii) once T < 1/64 the step is the cap 4 dt0 exactly, until T < eps ends the ray."""
    dt0, s = 0.005, 0.3
    # (a tiny eps keeps the dense cases marching after T < 1/64, where the cap is the whole rule)
    for rho, dist, eps in ((3.0, 4.0, 1e-3), (3.0, 12.0, 1e-3), (3.0, 40.0, 1e-3), (30.0, 4.0, 1e-9), (80.0, 9.0, 1e-9)):
        k = math.sqrt(2 * math.log(rho / 0.1))
        cam = _axis_camera(dist=dist)
        img, st, ctx = _render(orc, _one_gaussian(rho, s, (0.2, 0.6, 0.9)), cam, dt0, dynamic=True, eps=eps)
        slabs, _ = orc.march_trace(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], 4 * 9 + 4)
        slabs = [sl for sl in slabs if len(sl[4])]
        assert len(slabs) >= 2
        t_enter = dist - k * s
        assert abs(slabs[0][0] - t_enter) < 1e-4
        # (i): float32 arithmetic of the rule with T = 1 (rcbrt(1) = 1)
        first = min(max(np.float32(slabs[0][0]) / np.float32(1024.0), np.float32(dt0)), np.float32(4.0) * np.float32(dt0))
        assert np.float32(slabs[0][1]) == first, (rho, dist, slabs[0][1], first)

        def T_analytic(t):      # exp(-int_{t_enter}^{t} rho exp(-(u - dist)^2 / (2 s^2)) du)
            a, b = (t_enter - dist) / (s * math.sqrt(2)), (min(t, dist + k * s) - dist) / (s * math.sqrt(2))
            return math.exp(-rho * s * math.sqrt(math.pi / 2) * (math.erf(b) - math.erf(a)))

        saturated = grew = 0
        for tb, dt, lo, hi, _ in slabs[1:]:
            T = T_analytic(tb)
            want = min(max(tb / 1024.0, dt0) * T ** (-1.0 / 3.0), 4 * dt0)
            # the oracle's T is a midpoint-rule product: O(dt^2) off the analytic one, plus the 0.1 density
            # jump at the truncation boundary
            assert abs(dt - want) <= 2e-3 * want, (rho, dist, tb, dt, want)
            if T < 1.0 / 64.0 * 0.98:
                assert np.float32(dt) == np.float32(4.0) * np.float32(dt0)      # (iii): the cap, exactly
                saturated += 1
            grew += dt > slabs[0][1] * 1.01
        if rho >= 30.0:
            assert saturated >= 1
        if dist <= 12.0:
            assert grew >= 1            # (ii): the step really grows with falling T


def test_forward_matches_independent_float64_march(orc):
    sc = scenes.scene_to_numpy(scenes.make_scene(0, n=600, sh_degree=0, seed=21))
    sc["scales"] = sc["scales"] * 2.5
    cam = scenes.make_camera(0, 0, width=24, height=24)
    ids = np.arange(24 * 24)
    img, st, _ = _render(orc, sc, cam, 0.0025, cap=600)
    want = _f64_march_image(sc, cam, 0.0025, ids)
    assert st["rays_hit"] > 200 and st["hit_pairs"] > 2000
    # a fp32-vs-fp64 flip of one `power < k^2` sample moves a colour by <= 0.1*dt*|dc| ~ 2.5e-4
    err = np.abs(img - want).max(1)
    assert np.quantile(err, 0.98) < 2e-5
    assert err.max() < 6e-4


def _slabs_for_autograd(orc, ctx, ray):
    slabs, rgb = orc.march_trace(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], ray)
    return [(tb, dt, ids) for tb, dt, tlo, thi, ids in slabs if len(ids)], rgb


def _autograd_grads(orc, sc, cam, ctx, rays, dloss, rgb_np, eps=1e-3, dynamic=False):
    params = {k: torch.tensor(sc[k].astype(np.float64), requires_grad=True)
              for k in ("positions", "scales", "quaternions", "densities")}
    params["rgb"] = torch.tensor(rgb_np.astype(np.float64), requires_grad=True)
    dirs = orc.ray_dirs(ctx["cs"], rays).astype(np.float64)
    slabs = []
    for r in rays:
        s, _ = _slabs_for_autograd(orc, ctx, int(r))
        slabs.append(s)
    img = f64ref.march_torch(params, cam.camera_center.double().numpy(), dirs, slabs, eps)
    loss = (img * torch.tensor(dloss[rays].astype(np.float64))).sum()
    loss.backward()
    return {k: v.grad.numpy() for k, v in params.items()}, img.detach().numpy()


def _cos_rel(a, b):
    a = a.astype(np.float64).ravel()
    b = b.astype(np.float64).ravel()
    return a @ b / (np.linalg.norm(a) * np.linalg.norm(b) + 1e-300), np.linalg.norm(a - b) / (np.linalg.norm(b) + 1e-300)


def test_backward_matches_autograd_with_frozen_hit_sets(orc):
    for dynamic, seed in ((False, 31), (True, 32)):
        sc = scenes.scene_to_numpy(scenes.make_scene(0, n=64, sh_degree=0, seed=seed))
        sc["scales"] = sc["scales"] * 6.0
        sc["densities"] = sc["densities"] * 3.0 + 0.3
        sc["positions"][63] = 6.0 / np.sqrt(3.0)          # behind the camera: never touched
        cam = scenes.make_camera(0, 0, width=12, height=12)
        img, st, ctx = orc.render_forward(sc, cam, 0.0025, dynamic, 64)
        rng = np.random.default_rng(seed)
        dloss = rng.normal(size=img.shape).astype(np.float32)
        g, st_b = orc.march_backward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], img, dloss)
        assert st_b["hit_pairs"] == st["hit_pairs"] and st["hit_pairs"] > 500
        rays = np.arange(144)
        ag, img64 = _autograd_grads(orc, sc, cam, ctx, rays, dloss, ctx["rgb"], dynamic=dynamic)
        err = np.abs(img - img64).max(1)      # a fp32/fp64 flip of one cut-off sample costs <= 2.5e-4
        assert np.quantile(err, 0.95) < 2e-5 and err.max() < 6e-4
        for name, key in (("ddens", "densities"), ("drgb", "rgb"), ("dpos", "positions"),
                          ("dscale", "scales"), ("dquat", "quaternions")):
            cos, rel = _cos_rel(g[name], ag[key])
            assert cos > 0.99999 and rel < 2e-3, (dynamic, name, cos, rel)
        # prims no ray touched get exactly zero
        touched = np.zeros(64, bool)
        for r in rays:
            for _, _, ids in _slabs_for_autograd(orc, ctx, int(r))[0]:
                touched[ids] = True
        assert (~touched).any()
        for name in ("ddens", "drgb", "dpos", "dscale", "dquat"):
            assert not g[name][~touched].any()


def test_backward_is_linear_in_the_image_gradient(orc):
    sc = scenes.scene_to_numpy(scenes.make_scene(0, n=64, sh_degree=0, seed=33))
    sc["scales"] = sc["scales"] * 6.0
    cam = scenes.make_camera(0, 0, width=10, height=10)
    img, _, ctx = orc.render_forward(sc, cam, 0.0025, False, 64)
    rng = np.random.default_rng(5)
    a = rng.normal(size=img.shape).astype(np.float32)
    b = rng.normal(size=img.shape).astype(np.float32)
    args = (ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], img)
    ga, _ = orc.march_backward(*args, a)
    gb, _ = orc.march_backward(*args, b)
    gab, _ = orc.march_backward(*args, (2 * a - 3 * b).astype(np.float32))
    for k in ga:
        np.testing.assert_allclose(gab[k], 2 * ga[k] - 3 * gb[k], rtol=2e-3, atol=2e-6 * np.abs(gab[k]).max() + 1e-9)
    # restricting to a ray subset equals zeroing the other rays' gradient
    sub = np.arange(0, 100, 3)
    masked = np.zeros_like(a)
    masked[sub] = a[sub]
    g1, _ = orc.march_backward(*args, a, ray_ids=sub)
    g2, _ = orc.march_backward(*args, masked)
    for k in g1:
        np.testing.assert_allclose(g1[k], g2[k], rtol=1e-5, atol=1e-9)


def test_backward_matches_central_differences_through_whole_operator(orc):
    """End-to-end check incl. SH colour: d loss / d density and d loss / d position
    by float64-stepped central differences of the fp32 oracle forward."""
    sc = scenes.scene_to_numpy(scenes.make_scene(0, n=24, sh_degree=2, seed=41))
    sc["scales"] = sc["scales"] * 8.0
    sc["densities"] = sc["densities"] + 0.5
    cam = scenes.make_camera(0, 0, width=10, height=10)
    img, _, ctx = orc.render_forward(sc, cam, 0.0025, False, 64)
    rng = np.random.default_rng(6)
    dloss = rng.normal(size=img.shape).astype(np.float32)
    g, _ = orc.render_backward(sc, ctx, img, dloss)

    def loss(scn):
        im, _, _ = orc.render_forward(scn, cam, 0.0025, False, 64)
        return float((im.astype(np.float64) * dloss).sum())

    num = np.zeros(24)
    h = 2e-3
    for n in range(24):
        p, m = {k: v.copy() for k, v in sc.items()}, {k: v.copy() for k, v in sc.items()}
        p["color_features"][n, 1, 0] += h
        m["color_features"][n, 1, 0] -= h
        num[n] = (loss(p) - loss(m)) / (2 * h)
    ana = g["color_features"][:, 1, 0]
    cos, rel = _cos_rel(ana, num)
    assert cos > 0.999 and rel < 3e-2, (cos, rel)


def test_viewer_depth_and_quantised_colours(orc):
    """The viewer's outputs (cuda_gui/gaussians_aabb.cu): expected depth sum T (1 - w) t and
    uchar4 colours on a black background.  (i) One isotropic Gaussian on the ray axis against a
    float64 quadrature of int t sigma(t) exp(-tau(t)) dt with the truncated density; (ii) with
    colour 1 the image is 1 - T, so depth / colour is a weighted mean distance that must lie inside
    the Gaussian; (iii) in a scene, depth / (1 - T) lies between the box entry and exit and the
    frame is the colours' quantisation, with the known values 0 -> 0, 0.5 -> 128, 1 -> 255."""
    rho, s, dist = 3.0, 0.05, 4.0
    k = math.sqrt(2 * math.log(rho / 0.1))
    cam = _axis_camera(dist=dist)
    centre = 4 * 9 + 4
    sc = _one_gaussian(rho, s, (1.0, 1.0, 1.0))
    t = np.linspace(dist - k * s, dist + k * s, 400001)
    sigma = rho * np.exp(-0.5 * ((t - dist) / s) ** 2)
    tau = np.concatenate([[0.0], np.cumsum(0.5 * (sigma[1:] + sigma[:-1]) * np.diff(t))])
    f = t * sigma * np.exp(-tau)
    want_depth = float(np.sum(0.5 * (f[1:] + f[:-1]) * np.diff(t)))
    want_alpha = 1.0 - math.exp(-tau[-1])
    for dt in (0.002, 0.001):
        _, _, ctx = _render(orc, sc, cam, dt, white=False)
        frame, depth, colors = orc.march_gui(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"])
        assert abs(colors[centre, 0] - want_alpha) < 0.1 * dt + 1e-5
        # depth carries the same O(dt) truncation-boundary error as the optical depth, times t
        assert abs(depth[centre] - want_depth) < dist * (0.1 * dt + 1e-5) + dt * want_alpha
        mean_t = depth[centre] / colors[centre, 0]
        assert dist - k * s < mean_t < dist            # absorption weights the near side
        assert depth[0] == 0.0 and (frame[0] == (0, 0, 0, 255)).all()      # a ray that misses
    # (iii) a scene
    scn = scenes.scene_to_numpy(scenes.make_scene(0, n=800, sh_degree=0, seed=5))
    scn["scales"] = scn["scales"] * 2.5
    scn["color_features"][:] = (1.0 - 0.5) / 0.28209479177387814          # colour exactly 1
    cam2 = scenes.make_camera(0, 0, width=32, height=32)
    img, st, ctx = _render(orc, scn, cam2, 0.0025, cap=800, white=False)
    frame, depth, colors = orc.march_gui(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"])
    np.testing.assert_array_equal(colors, img)                            # same march as the forward
    hit = colors[:, 0] > 1e-3
    assert hit.sum() > 300
    eye = cam2.camera_center.numpy().astype(np.float64)
    dirs = orc.ray_dirs(ctx["cs"], np.arange(32 * 32)).astype(np.float64)
    lo = (ctx["bmin"].astype(np.float64) - eye) / dirs
    hi = (ctx["bmax"].astype(np.float64) - eye) / dirs
    tenter = np.minimum(lo, hi).max(1)
    texit = np.maximum(lo, hi).min(1)
    mean_t = depth[hit] / colors[hit, 0]
    assert (mean_t > tenter[hit] - 1e-3).all() and (mean_t < texit[hit] + 1e-3).all()
    np.testing.assert_array_equal(frame[:, :3], np.minimum(np.floor(np.clip(colors, 0, 1) * 256.0), 255).astype(np.uint8))
    assert (frame[:, 3] == 255).all()
    one = _one_gaussian(60.0, 0.2, (0.5, 1.0, 0.0))                       # opaque: colours reach (0.5, 1, 0)
    _, _, ctx1 = _render(orc, one, cam, 0.002, white=False)
    f1, _, c1 = orc.march_gui(ctx1["cs"], ctx1["ms"], ctx1["bmin"], ctx1["bmax"], ctx1["prims"])
    assert abs(c1[centre, 1] - 1.0) < 2e-3 and f1[centre, 2] == 0 and f1[centre, 1] >= 254 and 127 <= f1[centre, 0] <= 128


def test_step_scale_probe_is_exact_at_one_and_moves_the_adaptive_march(orc):
    """oracle.set_step_scale(1.0) is the reference's arithmetic bit for bit; scaling the adaptive
    step by one ulp moves image and gradients (the probe behind the looser adaptive-step gate of the
    full-size GPU test, where a re-phased ray costs far more than it does in this small scene)."""
    sc = scenes.scene_to_numpy(scenes.make_scene(2, n=20000, seed=3))
    cam, cfg = scenes.make_camera(2, 1, width=96, height=64), scenes.CONFIGS[2]
    dloss = np.random.default_rng(18).normal(size=(96 * 64, 3)).astype(np.float32)

    def run(scale):
        orc.set_step_scale(scale)
        try:
            img, st, ctx = orc.render_forward(sc, cam, cfg["dt_step"], True, cfg["max_prim_slice"])
            g, _ = orc.render_backward(sc, ctx, img, dloss)
        finally:
            orc.set_step_scale(1.0)
        return img, g

    img_a, g_a = run(1.0)
    img_b, g_b = run(1.0)
    assert np.array_equal(img_a, img_b) and all(np.array_equal(g_a[k], g_b[k]) for k in g_a if g_a[k] is not None)
    img_c, g_c = run(1.0 + 2.0 ** -23)
    assert 0.0 < np.abs(img_c - img_a).max() < 1e-4
    rel = np.linalg.norm(g_c["positions"] - g_a["positions"]) / np.linalg.norm(g_a["positions"])
    assert 1e-7 < rel < 1e-3
    # the fixed step does not use the coefficient at all
    orc.set_step_scale(1.5)
    try:
        img_d, _, _ = orc.render_forward(sc, cam, cfg["dt_step"], False, cfg["max_prim_slice"])
    finally:
        orc.set_step_scale(1.0)
    img_e, _, _ = orc.render_forward(sc, cam, cfg["dt_step"], False, cfg["max_prim_slice"])
    assert np.array_equal(img_d, img_e)


def test_cutoff_probes_of_the_backward(orc):
    """orc_march_backward_in_cut / orc_set_backward_mask_form: the per-ray count of samples the backward's
    gradient loop takes as inside a cut-off equals a float64 count over the same slabs on every ray without a
    sample within rounding of a cut-off; the count of samples on which the forward's and the backward's
    arrangements of the power disagree is zero on almost every ray, and never more than the float64 count's
    near-edge samples; deciding by the forward's arrangement changes the gradients of no Gaussian that no
    disagreeing ray touches, and leaves everything alone when no ray disagrees."""
    sc = scenes.scene_to_numpy(scenes.make_scene(0, n=500, sh_degree=0, seed=41))
    sc["scales"] = sc["scales"] * 2.0
    sc["densities"] = sc["densities"] * 0.25 + 0.12          # faint: no ray saturates, every blended sample counts
    cam = scenes.make_camera(0, 0, width=20, height=20)
    img, st, ctx = orc.render_forward(sc, cam, 0.0025, False, 500)
    args = (ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"])
    counts = orc.march_backward_in_cut(*args, img)
    assert counts.shape == (400, 2) and counts[:, 0].sum() > 20000
    eye = cam.camera_center.double().numpy()
    dirs = f64ref.ray_dirs_pinhole(cam)
    R = f64ref.rot_from_quat(torch.tensor(sc["quaternions"].astype(np.float64))).numpy()
    pos, scale = sc["positions"].astype(np.float64), sc["scales"].astype(np.float64)
    kk = 2.0 * np.log(sc["densities"].astype(np.float64) / 0.1)
    want, near = np.zeros(400, np.int64), np.zeros(400, np.int64)
    touched = [set() for _ in range(400)]
    for r in range(400):
        slabs, _ = orc.march_trace(*args, r)
        for tb, dt, tlo, thi, ids in slabs:
            if not len(ids):
                continue
            touched[r].update(int(i) for i in ids)
            t = tb + dt * (np.arange(32) + 0.5)
            x = eye[None] + t[:, None] * dirs[r][None]
            loc = np.einsum("hji,hsj->hsi", R[ids], x[None] - pos[ids][:, None]) / scale[ids][:, None]
            power = (loc ** 2).sum(-1)
            want[r] += int((power < kk[ids][:, None]).sum())
            near[r] += int((np.abs(power / kk[ids][:, None] - 1.0) < 2e-4).sum())     # one ulp of t moves a thin Gaussian's power by 1e-4
    clear = near == 0
    assert clear.mean() > 0.8
    assert np.array_equal(counts[clear, 0], want[clear])                 # the count itself, against float64
    assert np.all(np.abs(counts[:, 0] - want) <= near)
    assert np.all(counts[:, 1] <= near) and (counts[:, 1] == 0).mean() > 0.97
    # the two forms of the decision
    rng = np.random.default_rng(42)
    dloss = rng.normal(size=img.shape).astype(np.float32)
    g0, _ = orc.march_backward(*args, img, dloss)
    orc.set_backward_mask_form(1)
    try:
        g1, _ = orc.march_backward(*args, img, dloss)
        again = orc.march_backward_in_cut(*args, img)
    finally:
        orc.set_backward_mask_form(0)
    assert np.array_equal(again, counts)                                 # the probe reports both forms whichever decides
    disagreeing = np.nonzero(counts[:, 1] > 0)[0]
    suspects = set().union(*[touched[r] for r in disagreeing]) if len(disagreeing) else set()
    same = np.ones(500, bool)
    same[list(suspects)] = False
    for k in g0:
        assert np.array_equal(g0[k][same], g1[k][same]), k
    quiet = dloss.copy()
    quiet[disagreeing] = 0.0
    h0, _ = orc.march_backward(*args, img, quiet)
    orc.set_backward_mask_form(1)
    try:
        h1, _ = orc.march_backward(*args, img, quiet)
    finally:
        orc.set_backward_mask_form(0)
    for k in h0:
        assert np.array_equal(h0[k], h1[k]), k                          # without the disagreeing rays: the same backward, bit for bit
