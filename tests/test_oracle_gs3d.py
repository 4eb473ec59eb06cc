"""Pins the oracle's 3D-Gaussian (EWA) path (oracle/gs3d.cpp) without the reference: textbook forms in numpy for the
covariances, the conic, the projection and the compositing, and central finite differences in fp64 for both backward
passes. CPU only."""
import numpy as np
import pytest
import torch
from scipy.spatial.transform import Rotation

import oracle as O
from fast_sp_gs_amd import scenes


def _scene(P=400, size=96, seed=0):
    scene, cam = scenes.config0(P=P, size=size, seed=seed)
    n = lambda t: np.ascontiguousarray(t.double().numpy())
    g = np.random.default_rng(seed + 1)
    s = dict(means3D=n(scene.means3D), rotations=n(scene.rotations), opacities=n(scene.opacities), shs=n(scene.shs),
             scales=np.ascontiguousarray(np.concatenate([n(scene.scales) * 3, n(scene.scales[:, :1]) * g.uniform(0.5, 4, (P, 1))], 1)),
             Tw2v=n(cam.Tw2v), Tv2c=n(cam.Tv2c), campos=n(cam.campos))
    s['rotations'] = np.ascontiguousarray(s['rotations'] / np.linalg.norm(s['rotations'], axis=1, keepdims=True))
    tan_fov = (cam.W / 2 / float(cam.Tv2s[0, 0]), cam.H / 2 / float(cam.Tv2s[1, 1]))
    return s, cam, tan_fov


def _forward(s, cam, tan_fov, **over):
    a = {**s, **over}
    return O.gs3d_preprocess_forward(cam.W, cam.H, 3, False, a['means3D'], a['scales'], a['rotations'], a['opacities'],
                                     a['shs'], None, a['Tw2v'], a['Tv2c'], a['campos'], tan_fov)


def test_preprocess_forward_textbook_forms():
    s, cam, tan_fov = _scene()
    W, H = cam.W, cam.H
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    vis = rad > 0
    assert vis.sum() > 300
    fx, fy = 0.5 * W / tan_fov[0], 0.5 * H / tan_fov[1]
    for i in np.flatnonzero(vis)[:60]:
        R = Rotation.from_quat(s['rotations'][i]).as_matrix()  # the scene's quaternions are unit (x, y, z, w)
        S = np.diag(s['scales'][i] ** 2)
        Sigma = R @ S @ R.T
        assert np.allclose([Sigma[0, 0], Sigma[0, 1], Sigma[0, 2], Sigma[1, 1], Sigma[1, 2], Sigma[2, 2]], c3[i], rtol=1e-10, atol=1e-16)
        t = s['Tw2v'][:3, :3] @ s['means3D'][i] + s['Tw2v'][:3, 3]
        assert t[2] > 0.2 and abs(t[0]) < 1.3 * tan_fov[0] * t[2]  # inside the clamp, so J is the plain Jacobian
        J = np.array([[fx / t[2], 0, -fx * t[0] / t[2] ** 2], [0, fy / t[2], -fy * t[1] / t[2] ** 2]])
        Wm = s['Tw2v'][:3, :3]
        cov = J @ Wm @ Sigma @ Wm.T @ J.T + 0.3 * np.eye(2)
        conic = np.linalg.inv(cov)
        assert np.allclose([conic[0, 0], conic[0, 1], conic[1, 1]], co[i, :3], rtol=1e-9)
        assert co[i, 3] == s['opacities'][i, 0] and dep[i] == pytest.approx(t[2], rel=1e-12)
        clip = s['Tv2c'] @ np.append(t, 1.0)
        ndc = clip[:2] / clip[3]
        assert np.allclose(m2[i], [(ndc[0] + 1) * 0.5 * W - 0.5, (ndc[1] + 1) * 0.5 * H - 0.5], atol=1e-5)
        lam = np.linalg.eigvalsh(cov).max()
        assert rad[i] in (int(np.ceil(3 * np.sqrt(lam))), int(np.ceil(3 * np.sqrt(lam))) + 1)  # the 0.1 floor under the root
        x0, x1 = np.clip([int((m2[i, 0] - rad[i]) / 16), int((m2[i, 0] + rad[i] + 15) / 16)], 0, (W + 15) // 16)
        y0, y1 = np.clip([int((m2[i, 1] - rad[i]) / 16), int((m2[i, 1] + rad[i] + 15) / 16)], 0, (H + 15) // 16)
        assert tt[i] == (x1 - x0) * (y1 - y0)
    # rejected rows stay zero; a culling mask rejects
    behind = dict(means3D=s['means3D'] + np.array([0, 0, 50.0]))
    out = _forward(s, cam, tan_fov, **behind)
    assert not out[3].any() and not out[0].any() and not out[6].any()
    cull = np.zeros(len(rad), bool)
    cull[::2] = True
    out = O.gs3d_preprocess_forward(W, H, 3, False, s['means3D'], s['scales'], s['rotations'], s['opacities'], s['shs'],
                                    None, s['Tw2v'], s['Tv2c'], s['campos'], tan_fov, culling=cull)
    assert not out[3][::2].any() and np.array_equal(out[3][1::2], rad[1::2])


def _composite_numpy(W, H, m2, co, col, ex, pl, ranges):
    img, opa = np.zeros((3, H, W)), np.zeros((H, W))
    ext = np.zeros((ex.shape[1], H, W))
    gx = (W + 15) // 16
    for py in range(H):
        for px in range(W):
            r0, r1 = ranges[(py // 16) * gx + px // 16]
            ids = pl[r0:r1]
            d = m2[ids] - np.array([px, py], float)
            power = -0.5 * (co[ids, 0] * d[:, 0] ** 2 + co[ids, 2] * d[:, 1] ** 2) - co[ids, 1] * d[:, 0] * d[:, 1]
            alpha = np.minimum(0.99, co[ids, 3] * np.exp(power))
            alpha[(power > 0) | (alpha < 1 / 255)] = 0
            T = 1.0
            for k in range(len(ids)):
                if alpha[k] == 0:
                    continue
                if T * (1 - alpha[k]) < 1e-4:
                    break
                img[:, py, px] += col[ids[k]] * alpha[k] * T
                ext[:, py, px] += ex[ids[k]] * alpha[k] * T
                T *= 1 - alpha[k]
            opa[py, px] = 1 - T
    return img, opa, ext


def test_render_forward_closed_form_and_compositor():
    # one Gaussian: image = alpha * colour with alpha = min(0.99, o * exp(-0.5 d^T Q d))
    W = H = 32
    m2 = np.array([[13.3, 17.8]])
    co = np.array([[0.08, 0.02, 0.05, 0.8]])
    col, ex = np.array([[0.2, 0.5, 0.9]]), np.array([[2.0, -1.0]])
    ranges = np.zeros((4, 2), np.int64)
    ranges[:, 1] = 1  # every tile lists the Gaussian
    pl = np.zeros(1, np.int32)
    oc, oo, oe, nc = O.gs3d_render_forward(W, H, m2, co, col, ex, pl, ranges)
    yy, xx = np.mgrid[0:H, 0:W].astype(float)
    dx, dy = m2[0, 0] - xx, m2[0, 1] - yy
    alpha = np.minimum(0.99, 0.8 * np.exp(-0.5 * (0.08 * dx * dx + 0.05 * dy * dy) - 0.02 * dx * dy))
    alpha[alpha < 1 / 255] = 0
    assert np.abs(oo - alpha).max() < 1e-14 and np.abs(oc - alpha[None] * col[0][:, None, None]).max() < 1e-14
    assert np.abs(oe - alpha[None] * ex[0][:, None, None]).max() < 1e-14
    assert np.array_equal(nc, (alpha > 0).astype(np.int32))
    # a scene: independent per-pixel numpy compositor
    s, cam, tan_fov = _scene(P=600, size=64, seed=3)
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    ex = np.random.default_rng(1).normal(size=(len(rad), 2))
    ranges, pl = O.prepare(cam.W, cam.H, m2.astype(np.float32), dep.astype(np.float32), rad, tt)
    acc_w, acc_n, acc_max = np.zeros(len(rad)), np.zeros(len(rad), np.int32), np.zeros(len(rad), np.int32)
    oc, oo, oe, nc = O.gs3d_render_forward(cam.W, cam.H, m2, co, col, ex, pl, ranges, acc_max, acc_w, acc_n)
    img, opa, ext = _composite_numpy(cam.W, cam.H, m2, co, col, ex, pl, ranges)
    assert np.abs(oc - img).max() < 1e-12 and np.abs(oo - opa).max() < 1e-12 and np.abs(oe - ext).max() < 1e-12
    assert oo.max() > 0.5 and abs(acc_w.sum() - oo.sum()) < 1e-9  # blend weights sum to the opacity image
    assert acc_max.sum() == int((oo > 0).sum()) and acc_n.sum() >= acc_max.sum()


def test_topk_weights_are_the_largest_blend_weights():
    """gaussian_topk_weights against an independent per-pixel pass: collect every contributing (w, id) front to back,
    sort by weight (a later Gaussian first among equals), keep k."""
    s, cam, tan_fov = _scene(P=500, size=48, seed=5)
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    ranges, pl = O.prepare(cam.W, cam.H, m2.astype(np.float32), dep.astype(np.float32), rad, tt)
    K, W, H = 3, cam.W, cam.H
    ti, tw = O.gs3d_topk_weights(K, W, H, m2, co, ranges, pl)
    assert (np.diff(tw, axis=-1) <= 0).all() and ((ti == -1) == (tw == 0)).all()
    gx, crowded = (W + 15) // 16, 0
    for y in range(H):
        for x in range(W):
            r0, r1 = ranges[(y // 16) * gx + x // 16]
            T, ws = 1.0, []
            for order, e in enumerate(range(r0, r1)):
                i = pl[e]
                dx, dy = m2[i, 0] - x, m2[i, 1] - y
                power = -0.5 * (co[i, 0] * dx * dx + co[i, 2] * dy * dy) - co[i, 1] * dx * dy
                if power > 0:
                    continue
                a = min(0.99, co[i, 3] * np.exp(power))
                if a < 1 / 255:
                    continue
                if T * (1 - a) < 1e-4:
                    break
                ws.append((a * T, order, i))
                T *= 1 - a
            ws.sort(key=lambda t: (-t[0], -t[1]))
            top = [(w, i) for w, _, i in ws[:K]] + [(0.0, -1)] * (K - len(ws[:K]))
            assert np.allclose(tw[y, x], [t[0] for t in top], atol=1e-13)
            assert list(ti[y, x]) == [t[1] for t in top]
            crowded += len(ws) > K
    assert crowded > 20


def test_render_backward_finite_differences():
    s, cam, tan_fov = _scene(P=150, size=48, seed=5)
    W, H = cam.W, cam.H
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    P = len(rad)
    rng = np.random.default_rng(2)
    ex = rng.normal(size=(P, 3))
    ranges, pl = O.prepare(W, H, m2.astype(np.float32), dep.astype(np.float32), rad, tt)
    gi, go, ge = rng.normal(size=(3, H, W)), rng.normal(size=(H, W)), rng.normal(size=(3, H, W))

    def loss(m2_, co_, col_, ex_):
        oc, oo, oe, _ = O.gs3d_render_forward(W, H, m2_, co_, col_, ex_, pl, ranges)
        return (oc * gi).sum() + (oo * go).sum() + (oe * ge).sum()

    oc, oo, oe, nc = O.gs3d_render_forward(W, H, m2, co, col, ex, pl, ranges)
    g_col, g_ex, g_m2, g_co = O.gs3d_render_backward(W, H, m2, co, col, ex, oo, nc, gi, ge, go, pl, ranges)
    vis = np.flatnonzero(rad > 0)
    h = 1e-6
    checked = 0
    for i in vis[rng.permutation(len(vis))[:25]]:
        for name, arr, grad, cols in (("means2D", m2, g_m2, 2), ("conic_opacity", co, g_co, 4), ("colors", col, g_col, 3),
                                      ("extras", ex, g_ex, 3)):
            for c in range(cols):
                a, b = arr.copy(), arr.copy()
                a[i, c] += h
                b[i, c] -= h
                args = {"means2D": (m2, co, col, ex), }
                if name == "means2D":
                    fd = (loss(a, co, col, ex) - loss(b, co, col, ex)) / (2 * h)
                elif name == "conic_opacity":
                    fd = (loss(m2, a, col, ex) - loss(m2, b, col, ex)) / (2 * h)
                elif name == "colors":
                    fd = (loss(m2, co, a, ex) - loss(m2, co, b, ex)) / (2 * h)
                else:
                    fd = (loss(m2, co, col, a) - loss(m2, co, col, b)) / (2 * h)
                scale = max(abs(fd), np.abs(grad).max() * 1e-3, 1e-6)
                # thresholds (alpha = 1/255, T = 1e-4, the 0.99 clamp) make the image piecewise smooth: a step that
                # crosses one shows up as a large mismatch; those are rare and skipped by the count below
                if abs(fd - grad[i, c]) <= 2e-4 * scale:
                    checked += 1
    assert checked >= 0.97 * 25 * 12


def test_preprocess_backward_finite_differences():
    s, cam, tan_fov = _scene(P=60, size=64, seed=7)
    W, H = cam.W, cam.H
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    P = len(rad)
    rng = np.random.default_rng(4)
    g_m2, g_col, g_co = rng.normal(size=(P, 2)), rng.normal(size=(P, 3)), rng.normal(size=(P, 4))

    def loss(**over):
        o = _forward(s, cam, tan_fov, **over)
        return (o[0] * g_m2).sum() + (o[2] * g_col).sum() + (o[6] * g_co).sum()

    g3, gs, gq, gop, gsh, _, gcov, gm2_out = O.gs3d_preprocess_backward(
        W, H, 3, False, s['means3D'], s['scales'], s['rotations'], s['shs'], None, s['Tw2v'], s['Tv2c'], s['campos'],
        tan_fov, rad, col, c3, g_m2, g_col, g_co)
    assert np.allclose(gm2_out[rad > 0], g_m2[rad > 0] * np.array([0.5 * W, 0.5 * H]))
    assert np.array_equal(gop[rad > 0, 0], g_co[rad > 0, 3])
    h = 1e-6
    vis = np.flatnonzero(rad > 0)
    for name, grad in (("means3D", g3), ("scales", gs), ("rotations", gq), ("shs", gsh)):
        base = s[name]
        worst = 0.0
        for i in vis[:12]:
            idxs = [(c,) for c in range(base.shape[1])] if base.ndim == 2 else [(k, c) for k in (0, 3, 9, 15) for c in range(3)]
            for ix in idxs:
                a, b = base.copy(), base.copy()
                a[(i,) + ix] += h
                b[(i,) + ix] -= h
                fd = (loss(**{name: a}) - loss(**{name: b})) / (2 * h)
                worst = max(worst, abs(fd - grad[(i,) + ix]) / max(np.abs(grad[vis[:12]]).max(), 1e-9))
        assert worst < 2e-5, (name, worst)


def _ref_cov3D(scaling, rotation):
    """The reference's own torch formulation, renderer/gaussian_render.py:389-424 (build_rotation without normalising,
    L = R S, L L^T, upper triangle), in the dtype of its arguments."""
    x, y, z, r = rotation.unbind(-1)
    R = torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y),
                     2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x),
                     2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], -1).view(-1, 3, 3)
    Lm = R @ torch.diag_embed(scaling)
    C = Lm @ Lm.transpose(1, 2)
    return torch.stack([C[:, 0, 0], C[:, 0, 1], C[:, 0, 2], C[:, 1, 1], C[:, 1, 2], C[:, 2, 2]], -1)


def _ref_cov2D(means, cov3D, Tw2v, fx, fy, tx, ty):
    """renderer/gaussian_render.py:450-493 of the reference, line by line."""
    P = means.shape[0]
    R = Tw2v[:3, :3]
    p = torch.einsum('pi,ji->pj', means, R) + Tw2v[:3, 3]
    x, y, z = p.unbind(-1)
    limit_x, limit_y = z.detach() * 1.3 * tx, z.detach() * 1.3 * ty
    x = torch.minimum(torch.maximum(x, -limit_x), limit_x)
    y = torch.minimum(torch.maximum(y, -limit_y), limit_y)
    v0 = torch.zeros_like(z)
    J = torch.stack([fx / z, v0, -(fx * x) / (z * z), v0, fy / z, -(fy * y) / (z * z)], -1).view(P, 2, 3)
    T = J @ R
    V = torch.stack([cov3D[:, 0], cov3D[:, 1], cov3D[:, 2], cov3D[:, 1], cov3D[:, 3], cov3D[:, 4],
                     cov3D[:, 2], cov3D[:, 4], cov3D[:, 5]], -1).view(-1, 3, 3)
    V_ = T @ V @ T.transpose(-1, -2)
    return torch.stack([V_[:, 0, 0] + 0.3, V_[:, 0, 1], V_[:, 1, 1] + 0.3], -1)


def test_covariance_operators_match_the_reference_formulation():
    """gs_compute_cov3D_* / gs_compute_cov2D_*: the oracle in fp64 against the reference's torch fallbacks and their
    autograd, with points inside and outside the 1.3 x field-of-view clamp."""
    import torch
    g = torch.Generator().manual_seed(3)
    N = 300
    q = torch.randn(N, 4, generator=g, dtype=torch.float64)            # not normalised on purpose
    s = torch.rand(N, 3, generator=g, dtype=torch.float64) * 0.3 + 0.01
    gc = torch.randn(N, 6, generator=g, dtype=torch.float64)
    qa, sa = q.clone().requires_grad_(True), s.clone().requires_grad_(True)
    want = _ref_cov3D(sa, qa)
    want.backward(gc)
    got = O.gs3d_compute_cov3D(q.numpy(), s.numpy())
    np.testing.assert_allclose(got, want.detach().numpy(), rtol=1e-12, atol=1e-14)
    gq, gs = O.gs3d_compute_cov3D_backward(q.numpy(), s.numpy(), gc.numpy())
    np.testing.assert_allclose(gq, qa.grad.numpy(), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(gs, sa.grad.numpy(), rtol=1e-11, atol=1e-13)

    Tw2v = torch.eye(4, dtype=torch.float64)
    ang = 0.4
    Tw2v[:3, :3] = torch.tensor([[np.cos(ang), 0, np.sin(ang)], [0.1, 0.99, -0.05], [-np.sin(ang), 0.05, np.cos(ang)]])
    Tw2v[:3, 3] = torch.tensor([0.2, -0.1, 4.0])
    means = torch.randn(N, 3, generator=g, dtype=torch.float64) * torch.tensor([3.0, 3.0, 0.8])  # many beyond the clamp
    cov3D = want.detach()
    fx, fy, tx, ty = 500.0, 480.0, 0.4, 0.35
    pv = means @ Tw2v[:3, :3].T + Tw2v[:3, 3]
    keep = pv[:, 2] > 0.5  # in front of the camera, as every Gaussian that reaches this step is
    means, cov3D, pv, N = means[keep], cov3D[keep], pv[keep], int(keep.sum())
    assert N > 200
    outside = (pv[:, 0].abs() > 1.3 * tx * pv[:, 2]) | (pv[:, 1].abs() > 1.3 * ty * pv[:, 2])
    assert outside.any() and (~outside).any()
    ma, ca = means.clone().requires_grad_(True), cov3D.clone().requires_grad_(True)
    want2 = _ref_cov2D(ma, ca, Tw2v, fx, fy, tx, ty)
    g2 = torch.randn(N, 3, generator=g, dtype=torch.float64)
    want2.backward(g2)
    got2 = O.gs3d_compute_cov2D(cov3D.numpy(), means.numpy(), Tw2v.numpy(), fx, fy, tx, ty)
    np.testing.assert_allclose(got2, want2.detach().numpy(), rtol=1e-11, atol=1e-12)
    g_cov3D, g_mean = O.gs3d_compute_cov2D_backward(cov3D.numpy(), means.numpy(), Tw2v.numpy(), fx, fy, tx, ty,
                                                    g2.numpy())
    np.testing.assert_allclose(g_cov3D, ca.grad.numpy(), rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(g_mean, ma.grad.numpy(), rtol=1e-9, atol=1e-9 * float(ma.grad.abs().max()))


def test_extra_channels_forward_and_backward():
    """gaussian_rasterize_extra_*: 20 channels (two of the reference's groups of 16). Forward against the independent
    numpy compositor and, with a shortened n_contrib, against a per-pixel pass cut at that list position; backward
    against the finite-difference-pinned main backward fed zero colour / opacity gradients, and against central
    differences of the extra forward itself."""
    s, cam, tan_fov = _scene(P=300, size=48, seed=9)
    W, H = cam.W, cam.H
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    P, E = len(rad), 20
    rng = np.random.default_rng(4)
    ex = rng.normal(size=(P, E))
    ranges, pl = O.prepare(W, H, m2.astype(np.float32), dep.astype(np.float32), rad, tt)
    oc, oo, _, nc = O.gs3d_render_forward(W, H, m2, co, col, np.ascontiguousarray(ex[:, :1]), pl, ranges)
    out = O.gs3d_extra_forward(W, H, ex, m2, co, ranges, pl, nc)
    assert out.shape == (H, W, E)
    _, _, ext = _composite_numpy(W, H, m2, co, col, ex, pl, ranges)
    assert np.abs(out - ext.transpose(1, 2, 0)).max() < 1e-12 and np.abs(out).max() > 0.5

    cut = nc // 2  # stop each pixel half way down its list
    out_cut = O.gs3d_extra_forward(W, H, ex, m2, co, ranges, pl, cut)
    gx, shortened = (W + 15) // 16, 0
    for y in range(0, H, 3):
        for x in range(0, W, 3):
            r0, _ = ranges[(y // 16) * gx + x // 16]
            T, acc = 1.0, np.zeros(E)
            for e in range(r0, r0 + cut[y, x]):
                i = pl[e]
                dx, dy = m2[i, 0] - x, m2[i, 1] - y
                power = -0.5 * (co[i, 0] * dx * dx + co[i, 2] * dy * dy) - co[i, 1] * dx * dy
                a = min(0.99, co[i, 3] * np.exp(power))
                if power > 0 or a < 1 / 255:
                    continue
                acc += ex[i] * a * T
                T *= 1 - a
            assert np.abs(out_cut[y, x] - acc).max() < 1e-12
            shortened += np.abs(out_cut[y, x] - out[y, x]).max() > 1e-6
    assert shortened > 20

    g = rng.normal(size=(H, W, E))
    ge, gm, gc = O.gs3d_extra_backward(W, H, ex, oo, g, m2, co, ranges, pl, nc)
    z3, z1 = np.zeros((3, H, W)), np.zeros((H, W))
    r_col, r_ex, r_m2, r_co = O.gs3d_render_backward(W, H, m2, co, col, ex, oo, nc, z3,
                                                     np.ascontiguousarray(g.transpose(2, 0, 1)), z1, pl, ranges)
    for mine, ref in ((ge, r_ex), (gm, r_m2), (gc, r_co)):
        assert np.abs(mine - ref).max() <= 1e-12 * max(1.0, np.abs(ref).max()) and np.abs(ref).max() > 1e-3
    assert np.abs(r_col).max() == 0
    only_e = O.gs3d_extra_backward(W, H, ex, oo, g, m2, co, ranges, pl, nc, want=(True, False, False))
    assert np.array_equal(only_e[0], ge) and only_e[1] is None and only_e[2] is None
    only_g = O.gs3d_extra_backward(W, H, ex, oo, g, m2, co, ranges, pl, nc, want=(False, True, True))
    assert only_g[0] is None and np.array_equal(only_g[1], gm) and np.array_equal(only_g[2], gc)

    def loss(m2_, co_, ex_):
        return (O.gs3d_extra_forward(W, H, ex_, m2_, co_, ranges, pl, nc) * g).sum()

    h, ok, n = 1e-6, 0, 0
    vis = np.flatnonzero(rad > 0)
    for i in vis[rng.permutation(len(vis))[:12]]:
        for which, arr, grad, cols in ((0, m2, gm, (0, 1)), (1, co, gc, (0, 1, 2, 3)), (2, ex, ge, (0, 7, 19))):
            for c in cols:
                a, b = arr.copy(), arr.copy()
                a[i, c] += h
                b[i, c] -= h
                args_a, args_b = [m2, co, ex], [m2, co, ex]
                args_a[which], args_b[which] = a, b
                fd = (loss(*args_a) - loss(*args_b)) / (2 * h)
                n += 1
                ok += abs(fd - grad[i, c]) <= 2e-4 * max(abs(fd), np.abs(grad).max() * 1e-3, 1e-6)
    assert ok >= 0.97 * n  # a step that crosses the alpha = 1/255 threshold is the rare miss


def test_precomputed_covariances_and_camera_gradients():
    """Pre-computed cov3D / cov2D inputs (gaussian_preprocess.cu:76-92): feeding the covariances the stand-alone
    operators give reproduces the ordinary forward; their gradients (the conic's derivative for cov2D, :293-301; the
    [P,6] gradient for cov3D) against central differences. Camera gradients (:271, :318-355 and
    gaussian_compute_cov2D.cu:163-183): dL/dTw2v rows 0-2 and dL/dcampos against central differences of the forward in
    the view matrix and the camera position (points inside 1.3 x FoV, where the reference's formula is exact)."""
    s, cam, tan_fov = _scene(P=60, size=64, seed=7)
    W, H = cam.W, cam.H
    base = _forward(s, cam, tan_fov)
    m2, dep, col, rad, tt, c3, co = base
    P = len(rad)
    vis = np.flatnonzero(rad > 0)
    fx, fy = 0.5 * W / tan_fov[0], 0.5 * H / tan_fov[1]
    cov3 = O.gs3d_compute_cov3D(s['rotations'], s['scales'])
    cov2 = O.gs3d_compute_cov2D(cov3, s['means3D'], s['Tw2v'], fx, fy, *tan_fov)

    def fwd(**over):
        a = {**s, **{k: v for k, v in over.items() if k in s}}
        return O.gs3d_preprocess_forward(W, H, 3, False, a['means3D'], a['scales'], a['rotations'], a['opacities'],
                                         a['shs'], None, a['Tw2v'], a['Tv2c'], a['campos'], tan_fov,
                                         cov3D_precomp=over.get('cov3D'), cov2D_precomp=over.get('cov2D'))

    o3 = fwd(cov3D=cov3.copy())
    o2 = fwd(cov2D=cov2.copy())
    for o in (o3, o2):
        assert np.array_equal(o[3], rad) and np.array_equal(o[4], tt)
        assert np.abs(o[6] - co).max() < 1e-12 * max(1, np.abs(co).max()) and np.abs(o[0] - m2).max() < 1e-12
    assert o3[5] is not None and np.abs(o3[5] - cov3).max() == 0

    rng = np.random.default_rng(4)
    g_m2, g_col, g_co = rng.normal(size=(P, 2)), rng.normal(size=(P, 3)), rng.normal(size=(P, 4))
    loss = lambda o: (o[0] * g_m2).sum() + (o[2] * g_col).sum() + (o[6] * g_co).sum()
    args = (W, H, 3, False, s['means3D'], s['scales'], s['rotations'], s['shs'], None, s['Tw2v'], s['Tv2c'],
            s['campos'], tan_fov, rad, col)
    h = 1e-6
    # cov2D pre-computed: [P,3] gradient, nothing reaches the means through the covariance, no scale / rotation outputs
    r2 = O.gs3d_preprocess_backward(*args, c3, g_m2, g_col, g_co, cov2D=cov2)
    assert r2[1] is None and r2[2] is None and r2[6].shape == (P, 3)
    r3 = O.gs3d_preprocess_backward(*args, cov3, g_m2, g_col, g_co, precomputed=True)
    assert r3[1] is None and r3[6].shape == (P, 6)
    full = O.gs3d_preprocess_backward(*args, c3, g_m2, g_col, g_co)
    assert np.abs(r3[0] - full[0]).max() < 1e-12 and np.abs(r3[6] - full[6]).max() < 1e-12
    for name, arr, grad in (('cov2D', cov2, r2[6]), ('cov3D', cov3, r3[6])):
        worst = 0.0
        for i in vis[:10]:
            for c in range(arr.shape[1]):
                a, b = arr.copy(), arr.copy()
                a[i, c] += h
                b[i, c] -= h
                fd = (loss(fwd(**{name: a})) - loss(fwd(**{name: b}))) / (2 * h)
                worst = max(worst, abs(fd - grad[i, c]) / max(np.abs(grad[vis[:10]]).max(), 1e-9))
        assert worst < 2e-5, (name, worst)
    # the means' gradient with cov2D given is the projection's and the colours' alone
    assert np.abs(r2[0] - full[0]).max() > 1e-3 * np.abs(full[0]).max()

    # camera gradients: accumulate into the caller's buffers, rows 0-2 of the view matrix
    out = O.gs3d_preprocess_backward(*args, c3, g_m2, g_col, g_co, camera=True)
    g_vm, g_cam = out[-2], out[-1]
    assert not g_vm[3].any() and np.abs(g_vm[:3]).max() > 0 and np.abs(g_cam).max() > 0
    for a_ in range(3):
        for b_ in range(4):
            p, m = s['Tw2v'].copy(), s['Tw2v'].copy()
            p[a_, b_] += h
            m[a_, b_] -= h
            fd = (loss(fwd(Tw2v=p)) - loss(fwd(Tw2v=m))) / (2 * h)
            assert abs(fd - g_vm[a_, b_]) < 2e-5 * max(1.0, np.abs(g_vm).max()), (a_, b_, fd, g_vm[a_, b_])
    for a_ in range(3):
        p, m = s['campos'].copy(), s['campos'].copy()
        p[a_] += h
        m[a_] -= h
        fd = (loss(fwd(campos=p)) - loss(fwd(campos=m))) / (2 * h)
        assert abs(fd - g_cam[a_]) < 2e-5 * max(1.0, np.abs(g_cam).max())
    # the stand-alone cov2D operator's view-matrix gradient (added to the caller's buffer)
    g2 = rng.normal(size=(P, 3))
    gvm = np.ones((4, 4))
    O.gs3d_compute_cov2D_backward(cov3, s['means3D'], s['Tw2v'], fx, fy, *tan_fov, g2, gvm)
    assert np.all(gvm[3] == 1.0)
    for a_ in range(3):
        for b_ in range(4):
            p, m = s['Tw2v'].copy(), s['Tw2v'].copy()
            p[a_, b_] += h
            m[a_, b_] -= h
            fd = ((O.gs3d_compute_cov2D(cov3, s['means3D'], p, fx, fy, *tan_fov) * g2).sum() -
                  (O.gs3d_compute_cov2D(cov3, s['means3D'], m, fx, fy, *tan_fov) * g2).sum()) / (2 * h)
            assert abs(fd - (gvm[a_, b_] - 1.0)) < 2e-5 * max(1.0, np.abs(gvm).max()), (a_, b_)


def test_bucket_snapshots_and_per_gaussian_backward():
    """gaussian_rasterize_forward's snapshots (state before every 32nd list entry) and gaussian_rasterize_fast_backward
    (gaussian_render.cu:540-694), restated bucket by bucket from those snapshots: the same derivative as the
    back-to-front backward (pinned by finite differences above), so the two must agree to rounding."""
    s, cam, tan_fov = _scene(P=900, size=48, seed=5)
    s['scales'] = s['scales'] * 2.5
    W, H = cam.W, cam.H
    m2, dep, col, rad, tt, c3, co = _forward(s, cam, tan_fov)
    P = len(rad)
    rng = np.random.default_rng(2)
    ranges, pl = O.prepare(W, H, m2.astype(np.float32), dep.astype(np.float32), rad, tt)
    lens = ranges[:, 1] - ranges[:, 0]
    assert lens.max() > 70
    offset = np.ascontiguousarray(np.cumsum((lens + 31) // 32).astype(np.int64))
    for E in (0, 2):
        ex = rng.normal(size=(P, E)) if E else None
        oc, oo, oe, nc, max_c, b2t, sT, sar = O.gs3d_render_forward(W, H, m2, co, col, ex, pl, ranges,
                                                                    bucket_offset=offset)
        plain = O.gs3d_render_forward(W, H, m2, co, col, ex, pl, ranges)
        assert np.array_equal(oc, plain[0]) and np.array_equal(nc, plain[3])
        assert np.array_equal(b2t, np.repeat(np.arange(len(lens)), (lens + 31) // 32)) and sar.shape[1] == 3 + E
        gx = (W + 15) // 16
        for t in np.flatnonzero(lens > 0):
            ty, tx = divmod(int(t), gx)
            assert max_c[t] == nc[ty * 16:ty * 16 + 16, tx * 16:tx * 16 + 16].max()
            b0 = 0 if t == 0 else int(offset[t - 1])
            hh, ww = min(16, H - ty * 16), min(16, W - tx * 16)
            assert np.all(sT[b0].reshape(16, 16)[:hh, :ww] == 1.0) and not sar[b0].any()
            # a later bucket holds the image of the list cut in front of it, where the pixel was still blending
            for k in range(1, int((lens[t] + 31) // 32)):
                cut = ranges.copy()
                cut[:, 1] = cut[:, 0]
                cut[t, 1] = cut[t, 0] + 32 * k
                pc, po, pe, _ = O.gs3d_render_forward(W, H, m2, co, col, ex, pl, cut)
                live = sT[b0 + k].reshape(16, 16)[:hh, :ww] > 0
                blk = lambda a: a[..., ty * 16:ty * 16 + hh, tx * 16:tx * 16 + ww]
                assert np.abs((sT[b0 + k].reshape(16, 16)[:hh, :ww] - (1 - blk(po)))[live]).max(initial=0) < 1e-12
                for c in range(3):
                    assert np.abs((sar[b0 + k, c].reshape(16, 16)[:hh, :ww] - blk(pc)[c])[live]).max(initial=0) < 1e-12
                for c in range(E):
                    assert np.abs((sar[b0 + k, 3 + c].reshape(16, 16)[:hh, :ww] - blk(pe)[c])[live]).max(initial=0) < 1e-12
        gi, go = rng.normal(size=(3, H, W)), rng.normal(size=(H, W))
        ge = rng.normal(size=(E, H, W)) if E else None
        slow = O.gs3d_render_backward(W, H, m2, co, col, ex, oo, nc, gi, ge, go, pl, ranges)
        fast = O.gs3d_render_fast_backward(W, H, m2, co, col, ex, oc, oe, oo, nc, max_c, offset, b2t, sT, sar, gi, ge,
                                           go, pl, ranges)
        for a, b in zip(slow, fast):
            assert (a is None) == (b is None)
            if a is not None:
                assert np.abs(a - b).max() < 1e-9 * max(1.0, np.abs(a).max()) and np.abs(a).max() > 0
