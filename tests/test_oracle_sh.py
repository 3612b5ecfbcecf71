"""Pins the SH colour kernels of the CPU oracle: scipy's spherical harmonics for the
basis, torch.autograd for the gradients, and the one place the reference departs
from calculus (utils/sh_utils.cu:367) isolated exactly."""
import math

import numpy as np
import torch
from scipy.special import sph_harm_y

C0 = 0.28209479177387814


def real_sh_basis_scipy(d):
    """Real SH with the Condon-Shortley phase (the 3DGS convention), order l^2 + l + m."""
    x, y, z = d[:, 0], d[:, 1], d[:, 2]
    theta = np.arccos(np.clip(z, -1, 1))
    phi = np.arctan2(y, x)
    out = []
    for l in range(4):
        for m in range(-l, l + 1):
            Y = sph_harm_y(l, abs(m), theta, phi)
            out.append(Y.real if m == 0 else math.sqrt(2) * (Y.real if m > 0 else Y.imag))
    return np.stack(out, 1)


def basis_torch(d):
    x, y, z = d[..., 0], d[..., 1], d[..., 2]
    xx, yy, zz, xy, yz, xz = x * x, y * y, z * z, x * y, y * z, x * z
    C1 = 0.4886025119029199
    C2 = [1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792, 0.5462742152960396]
    C3 = [-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154,
          -0.4570457994644658, 1.445305721320277, -0.5900435899266435]
    return torch.stack([
        torch.full_like(x, C0), -C1 * y, C1 * z, -C1 * x,
        C2[0] * xy, C2[1] * yz, C2[2] * (2 * zz - xx - yy), C2[3] * xz, C2[4] * (xx - yy),
        C3[0] * y * (3 * xx - yy), C3[1] * xy * z, C3[2] * y * (4 * zz - xx - yy),
        C3[3] * z * (2 * zz - 3 * xx - 3 * yy), C3[4] * x * (4 * zz - xx - yy), C3[5] * z * (xx - yy),
        C3[6] * x * (xx - 3 * yy)], -1)


def _inputs(n, K, G, seed):
    rng = np.random.default_rng(seed)
    pos = rng.normal(size=(n, 3)).astype(np.float32) * 2
    eye = np.array([0.3, -4.0, 1.0], np.float32)
    sh = rng.normal(size=(n, 3, K)).astype(np.float32)
    sg = rng.normal(size=(n, 3, G)).astype(np.float32)
    sharp = rng.uniform(0.5, 4, size=(n, G)).astype(np.float32)
    axis = rng.normal(size=(n, G, 3)).astype(np.float32)
    axis /= np.linalg.norm(axis, axis=2, keepdims=True) + 1e-9
    return eye, pos, sh, sg, sharp, axis


def test_basis_matches_scipy_spherical_harmonics(orc):
    rng = np.random.default_rng(0)
    pos = rng.normal(size=(50, 3)).astype(np.float32)
    eye = np.zeros(3, np.float32)
    d = pos / np.linalg.norm(pos, axis=1, keepdims=True)
    want = real_sh_basis_scipy(d.astype(np.float64))
    np.testing.assert_allclose(basis_torch(torch.tensor(d, dtype=torch.float64)).numpy(), want, atol=1e-6)
    for j in range(16):
        sh = np.zeros((50, 3, 16), np.float32)
        sh[:, 1, j] = 1.0
        rgb = orc.sh_forward(eye, pos, sh)
        np.testing.assert_allclose(rgb[:, 1] - 0.5, want[:, j], atol=2e-6)
        np.testing.assert_array_equal(rgb[:, 0], 0.5)


def test_degree_zero_is_rgb2sh_inverse_and_unclamped(orc):
    eye, pos, sh, *_ = _inputs(20, 1, 0, 1)
    rgb = orc.sh_forward(eye, pos, sh)
    np.testing.assert_allclose(rgb, 0.5 + C0 * sh[:, :, 0], rtol=1e-6)
    assert (rgb < 0).any()          # negative colours are legal: there is no clamp


def _torch_forward(eye, pos, sh, sg, sharp, axis):
    v = pos - eye
    d = v / v.norm(dim=1, keepdim=True)
    K = sh.shape[2]
    rgb = 0.5 + (basis_torch(d)[:, None, :K] * sh).sum(-1)
    if sg.shape[2]:
        g = torch.exp(sharp * ((d[:, None] * axis).sum(-1) - 1.0))       # (n,G)
        rgb = rgb + (sg * g[:, None]).sum(-1)
    return rgb


def test_forward_and_backward_match_autograd_all_degrees_with_lobes(orc):
    for degree, G in ((0, 0), (1, 2), (2, 0), (3, 3), (3, 0)):
        K = (degree + 1) ** 2
        eye, pos, sh, sg, sharp, axis = _inputs(40, K, G, 10 + degree)
        drgb = np.random.default_rng(3).normal(size=(40, 3)).astype(np.float32)
        drgb[7] = 0.0                                            # early-out row (sh_utils.cu:226)
        kw = dict(sg=sg, sharp=sharp, axis=axis) if G else {}
        rgb = orc.sh_forward(eye, pos, sh, **kw)
        t = [torch.tensor(a.astype(np.float64), requires_grad=True) for a in (pos, sh, sg, sharp, axis)]
        out = _torch_forward(torch.tensor(eye.astype(np.float64)), *t)
        np.testing.assert_allclose(rgb, out.detach().numpy(), atol=3e-6, rtol=2e-5)
        (out * torch.tensor(drgb.astype(np.float64))).sum().backward()
        for exact in (True, False):
            dsh, dpos, dsg, dsharp, daxis = orc.sh_backward(eye, pos, sh, drgb, exact_dy9=exact, **kw)
            np.testing.assert_allclose(dsh, t[1].grad.numpy(), atol=3e-6, rtol=2e-5)
            assert not dsh[7].any() and not dpos[7].any()
            if G:
                np.testing.assert_allclose(dsg, t[2].grad.numpy(), atol=3e-6, rtol=2e-5)
                np.testing.assert_allclose(dsharp, t[3].grad.numpy(), atol=3e-6, rtol=2e-5)
                np.testing.assert_allclose(daxis, t[4].grad.numpy(), atol=3e-6, rtol=2e-5)
            else:
                assert dsg is None and dsharp is None and daxis is None
            if exact or degree < 3:
                np.testing.assert_allclose(dpos, t[0].grad.numpy(), atol=5e-6, rtol=2e-5)
            else:
                # the reference's d/dy of basis 9 is C3[0]*(3xx - yy) instead of C3[0]*3(xx - yy):
                # dL/ddir.y is off by C3[0] * 2yy * sum_c drgb_c sh[c,9], then projected by the
                # Jacobian of the normalisation.  Nothing else differs.
                v = (pos - eye).astype(np.float64)
                r = np.linalg.norm(v, axis=1)
                d = v / r[:, None]
                extra_y = -0.5900435899266435 * 2 * d[:, 1] ** 2 * (drgb.astype(np.float64) * sh[:, :, 9]).sum(1)
                ddir = np.zeros_like(v)
                ddir[:, 1] = extra_y
                proj = (ddir - d * (d * ddir).sum(1, keepdims=True)) / r[:, None]
                np.testing.assert_allclose(dpos, t[0].grad.numpy() + proj, atol=5e-6, rtol=2e-5)
                assert np.abs(proj).max() > 1e-3
