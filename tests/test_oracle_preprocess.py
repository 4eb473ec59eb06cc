"""Pins the oracle's surfel preprocess (oracle/gs2d.cpp: compute_transmat, compute_aabb, preprocess_forward/backward)
with checks that do not retype its formulas:
  * the ray-splat matrix maps tangent-plane points to the pixels a textbook projection gives (closed form through the
    reference's own camera conventions), and the reference's literal single-surfel case projects its centre there;
  * the 3-sigma bound really bounds the projected ellipse (brute force over the ellipse boundary), the radius / tile
    rectangle / tiles_touched follow from it, rejected surfels produce zeros;
  * the backward pass equals central finite differences of the double-precision forward;
  * the float and double instantiations agree.
"""
import json
from pathlib import Path

import numpy as np
import pytest

GOLD = json.loads((Path(__file__).parent / "golden" / "single_surfel_inputs.json").read_text())


def quat_R(q):
    x, y, z, w = q
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (y * w + x * z)],
                     [2 * (x * y + z * w), 1 - 2 * (x * x + z * z), 2 * (y * z - x * w)],
                     [2 * (x * z - y * w), 2 * (x * w + y * z), 1 - 2 * (x * x + y * y)]])


def project(Tw2v, Tv2c, W, H, pw):
    """Textbook pipeline: world -> view -> clip -> NDC -> pixel centre coordinates ((ndc+1)*W/2 - 0.5)."""
    ph = np.append(pw, 1.0)
    clip = Tv2c @ (Tw2v @ ph)
    ndc = clip[:2] / clip[3]
    return np.array([(ndc[0] + 1) * W / 2 - 0.5, (ndc[1] + 1) * H / 2 - 0.5]), clip[3]


def _scene(P=200, seed=0, dtype=np.float64, W=200, H=120):
    import torch
    from fast_sp_gs_amd import scenes
    sc, _ = scenes.config0(P=P, size=64, seed=seed)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]), at=torch.tensor([0.1, 0.0, 0.0]))
    f = lambda t: np.ascontiguousarray(t.numpy().astype(dtype))
    s = dict(means3D=f(sc.means3D), scales=f(sc.scales) * 8, rotations=f(sc.rotations), opacities=f(sc.opacities),
             shs=f(sc.shs), Tw2v=f(cam.Tw2v), Tv2c=f(cam.Tv2c), campos=f(cam.campos), W=W, H=H)
    return s


def _fwd(O, s, **kw):
    return O.preprocess_forward(s['W'], s['H'], 3, s['means3D'], s['scales'], s['rotations'], s['opacities'], s['shs'],
                                None, s['Tw2v'], s['Tv2c'], s['campos'], **kw)


def test_transmat_maps_tangent_plane_to_pixels(oracle_mod):
    s = _scene()
    m2, colors, tm, no, dep, radii, tt = _fwd(oracle_mod, s)
    rng = np.random.default_rng(1)
    for i in np.flatnonzero(radii > 0)[:50]:
        R = quat_R(s['rotations'][i])
        for _ in range(4):
            u, v = rng.uniform(-2, 2, 2)
            pw = s['means3D'][i] + R[:, 0] * s['scales'][i, 0] * u + R[:, 1] * s['scales'][i, 1] * v
            pix, w = project(s['Tw2v'], s['Tv2c'], s['W'], s['H'], pw)
            h = tm[i] @ np.array([u, v, 1.0])
            assert np.allclose(h[:2] / h[2], pix, atol=1e-9) and abs(h[2] - w) < 1e-12
        # normal = view-space third column of R, flipped to face the camera; depth = view z
        n_view = s['Tw2v'][:3, :3] @ R[:, 2]
        p_view = s['Tw2v'][:3, :3] @ s['means3D'][i] + s['Tw2v'][:3, 3]
        sign = 1.0 if -(p_view @ n_view) > 0 else -1.0
        assert np.allclose(no[i, :3], sign * n_view, atol=1e-12)
        assert abs(dep[i] - p_view[2]) < 1e-12 and abs(no[i, 3] - s['opacities'][i, 0]) == 0


def test_reference_literal_surfel_projects_its_centre(oracle_mod):
    O = oracle_mod
    for case in GOLD['cases']:
        a = lambda k: np.ascontiguousarray(np.array(case[k] if k in case else GOLD[k], np.float64))
        W, H = GOLD['W'], GOLD['H']
        shs = a('shs').reshape(1, 1, 3)
        out = O.preprocess_forward(W, H, 0, a('means3D'), a('scales'), a('rotations'), a('opacity'), shs, None,
                                   a('Tw2v'), a('Tv2c'), a('campos'))
        m2, colors, tm, no, dep, radii, tt = out
        assert radii[0] > 0
        centre = tm[0] @ np.array([0, 0, 1.0])
        pix, _ = project(a('Tw2v'), a('Tv2c'), W, H, a('means3D')[0])
        assert np.allclose(centre[:2] / centre[2], pix, atol=1e-9)
        # (ndc2pix @ Tv2c)[:3,:3] are the intrinsics of the fixture: the standard and the "fast" transforms coincide
        ndc2pix = np.array([[W / 2, 0, 0, (W - 1) / 2], [0, H / 2, 0, (H - 1) / 2], [0, 0, 0, 1.0]])
        assert np.allclose((ndc2pix @ a('Tv2c'))[:, [0, 1, 2]], a('Tv2s'), atol=1e-9)
        assert abs(colors[0, 0] - max(0.0, 0.5 + 0.28209479177387814 * case['shs'][0][0])) < 1e-12


def test_bound_radius_rect(oracle_mod):
    s = _scene(P=300, seed=3)
    m2, colors, tm, no, dep, radii, tt = _fwd(oracle_mod, s)
    gx, gy = (s['W'] + 15) // 16, (s['H'] + 15) // 16
    th = np.linspace(0, 2 * np.pi, 721)
    n_checked = 0
    for i in range(300):
        if radii[i] == 0:
            assert tt[i] == 0 and not m2[i].any() and not tm[i].any() and not no[i].any() and dep[i] == 0
            continue
        M = tm[i]
        h = M @ np.stack([3 * np.cos(th), 3 * np.sin(th), np.ones_like(th)])
        if (h[2] <= 0).any():
            continue  # ellipse crosses the camera plane: no finite box
        xy = h[:2] / h[2]
        lo, hi = xy.min(1), xy.max(1)
        ext = (hi - lo) / 2
        assert np.allclose((hi + lo) / 2, m2[i], atol=1e-3 * max(1, ext.max()))
        expect_r = np.ceil(max(ext.max(), 3 * 0.707106))
        assert abs(radii[i] - expect_r) <= 1 and radii[i] >= np.floor(ext.max())
        r = radii[i]
        x0 = min(gx, max(0, int((m2[i, 0] - r) / 16))); x1 = min(gx, max(0, int((m2[i, 0] + r + 15) / 16)))
        y0 = min(gy, max(0, int((m2[i, 1] - r) / 16))); y1 = min(gy, max(0, int((m2[i, 1] + r + 15) / 16)))
        assert tt[i] == (x1 - x0) * (y1 - y0) and tt[i] > 0
        n_checked += 1
    assert n_checked > 100


def test_rejections(oracle_mod):
    s = _scene(P=64, seed=5)
    s['means3D'][:8, 2] = 3.9  # view z = 4 - 3.9 + ... <= 0.2: behind the near cut
    s['means3D'][8:16, 0] = 50.0  # far off screen: empty rectangle
    cull = np.zeros(64, bool)
    cull[16:24] = True
    m2_in = np.full((64, 2), 7.0)
    m2, colors, tm, no, dep, radii, tt = _fwd(oracle_mod, s, culling=cull, means2D=m2_in)
    assert not radii[:24].any() and not tt[:24].any() and radii[24:].all()
    assert (m2[:24] == 7.0).all()  # caller-supplied means2D rows of rejected surfels are left alone
    assert not colors[:24].any() and not tm[:24].any()


def test_float_matches_double(oracle_mod):
    s64, s32 = _scene(dtype=np.float64), _scene(dtype=np.float32)
    o64, o32 = _fwd(oracle_mod, s64), _fwd(oracle_mod, s32)
    same = o64[5] == o32[5]
    assert same.mean() > 0.97  # radii can differ by one when an extent sits on an integer
    for a, b in zip(o64[:5], o32[:5]):
        assert np.abs(a[same] - b[same]).max() < 2e-3 * max(1.0, np.abs(a).max())


def test_backward_matches_finite_differences(oracle_mod):
    O = oracle_mod
    s = _scene(P=24, seed=11)
    W, H = s['W'], s['H']
    rng = np.random.default_rng(0)
    m2, colors, tm, no, dep, radii, tt = _fwd(O, s)
    vis = radii > 0
    assert vis.sum() >= 12
    P = 24
    w_m2, w_tm, w_no, w_c = rng.normal(size=(P, 2)), rng.normal(size=(P, 3, 3)), rng.normal(size=(P, 4)), rng.normal(size=(P, 3))

    def loss(**over):
        t = dict(s)
        t.update(over)
        o = _fwd(O, t)
        return (o[0] * w_m2).sum() + (o[2] * w_tm).sum() + (o[3] * w_no).sum() + (o[1] * w_c).sum()

    g3, gs, gr, gop, gsh, _, gm2_after = O.preprocess_backward(
        W, H, 3, s['means3D'], s['scales'], s['rotations'], s['shs'], None, s['Tw2v'], s['Tv2c'], s['campos'], tm,
        radii, colors, np.ascontiguousarray(w_m2), np.ascontiguousarray(w_tm), np.ascontiguousarray(w_c),
        np.ascontiguousarray(w_no))
    eps = 1e-6
    for name, grad in (('means3D', g3), ('scales', gs), ('rotations', gr)):
        for i in np.flatnonzero(vis)[:8]:
            for a in range(grad.shape[1]):
                p, m = s[name].copy(), s[name].copy()
                p[i, a] += eps
                m[i, a] -= eps
                fd = (loss(**{name: p}) - loss(**{name: m})) / (2 * eps)
                assert abs(fd - grad[i, a]) < 1e-5 * max(1.0, abs(fd)), (name, i, a, fd, grad[i, a])
    for (i, l, c) in [(int(np.flatnonzero(vis)[0]), 0, 0), (int(np.flatnonzero(vis)[1]), 7, 2), (int(np.flatnonzero(vis)[2]), 15, 1)]:
        p, m = s['shs'].copy(), s['shs'].copy()
        p[i, l, c] += eps
        m[i, l, c] -= eps
        fd = (loss(shs=p) - loss(shs=m)) / (2 * eps)
        assert abs(fd - gsh[i, l, c]) < 1e-6
    # opacity gradient is the 4th component of the normal_opacity gradient; invisible rows stay zero
    assert np.array_equal(gop[vis, 0], w_no[vis, 3]) and not gop[~vis].any() and not g3[~vis].any()
    # densification proxy written over grad_mean2D (gs_2d_preprocess.cu:325-328)
    expect = np.stack([w_tm[:, 0, 2] * tm[:, 2, 2] * 0.5 * W, w_tm[:, 1, 2] * tm[:, 2, 2] * 0.5 * H], 1)
    assert np.allclose(gm2_after[vis], expect[vis], rtol=1e-12) and np.array_equal(gm2_after[~vis], w_m2[~vis])


def test_transmat_ops_agree_with_preprocess(oracle_mod):
    O = oracle_mod
    s = _scene(P=30, seed=2)
    P, W, H = 30, s['W'], s['H']
    Tw2c = np.ascontiguousarray(s['Tv2c'] @ s['Tw2v'])
    tm, nrm = np.zeros((P, 3, 3)), np.zeros((P, 3))
    assert O.call("gs_2d_compute_transmat_forward_f64", P, W, H, s['means3D'], s['scales'], s['rotations'], s['Tw2v'],
                  Tw2c, tm, nrm) == 0
    out = _fwd(O, s)
    vis = out[5] > 0
    assert np.allclose(tm[vis], out[2][vis], rtol=1e-12)
    rng = np.random.default_rng(4)
    gM, gN = np.ascontiguousarray(rng.normal(size=(P, 3, 3))), np.ascontiguousarray(rng.normal(size=(P, 3)))
    g3, gs, gr = np.zeros((P, 3)), np.zeros((P, 2)), np.zeros((P, 4))
    assert O.call("gs_2d_compute_transmat_backward_f64", P, W, H, s['means3D'], s['scales'], s['rotations'],
                  s['Tw2v'], Tw2c, gM, gN, g3, gs, gr) == 0

    def loss(**over):
        t = dict(s)
        t.update(over)
        tm_, n_ = np.zeros((P, 3, 3)), np.zeros((P, 3))
        O.call("gs_2d_compute_transmat_forward_f64", P, W, H, t['means3D'], t['scales'], t['rotations'], t['Tw2v'],
               Tw2c, tm_, n_)
        return (tm_ * gM).sum() + (n_ * gN).sum()

    eps = 1e-6
    for name, grad in (('means3D', g3), ('scales', gs), ('rotations', gr)):
        for i in range(0, P, 6):
            for a in range(grad.shape[1]):
                p, m = s[name].copy(), s[name].copy()
                p[i, a] += eps
                m[i, a] -= eps
                fd = (loss(**{name: p}) - loss(**{name: m})) / (2 * eps)
                assert abs(fd - grad[i, a]) < 1e-6 * max(1.0, abs(fd))
