"""Pins the oracle's alpha blend (oracle/gs2d.cpp: render_forward / render_backward / topk_weights):
  * single-surfel closed form on the reference's literal known-answer inputs: alpha = min(.99, o exp(-min(u^2+v^2,
    2|d|^2)/2)) with (u, v) from an independent 2x2 linear solve, thresholded at 1/255 (the relation the reference's
    own tests check, gs_2d_render.py:1073-1079 / gs_2d_fast_render.py:1050-1064);
  * an independent numpy per-pixel compositor on a small scene (front-to-back products instead of running state);
  * invariants: opacity = 1 - prod(1 - alpha), extras[8] = sum w = opacity, n_contrib bounds;
  * backward = central finite differences of the double-precision forward for image, opacity, depth, normal, median
    depth and distortion channels.
"""
import json
from pathlib import Path

import numpy as np
import pytest

GOLD = json.loads((Path(__file__).parent / "golden" / "single_surfel_inputs.json").read_text())


def _small_scene(O, P=40, W=48, H=32, seed=0, scale_mul=6.0, dtype=np.float64):
    import torch
    from fast_sp_gs_amd import scenes
    sc, _ = scenes.config0(P=P, size=64, seed=seed)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    f = lambda t: np.ascontiguousarray(t.numpy().astype(dtype))
    pre = O.preprocess_forward(W, H, 3, f(sc.means3D) * 0.5, f(sc.scales) * scale_mul, f(sc.rotations), f(sc.opacities),
                               f(sc.shs), None, f(cam.Tw2v), f(cam.Tv2c), f(cam.campos))
    m2, colors, tm, no, dep, radii, tt = pre
    ranges, pl = O.prepare(W, H, m2.astype(np.float32), dep.astype(np.float32), radii, tt)
    return dict(W=W, H=H, means2D=m2, colors=colors, trans_mat=tm, normal_opacity=no, ranges=ranges, point_list=pl,
                near=0.2, far=100.0, depths=dep)


def _uv(M, x, y):
    A = np.array([M[0, :2] - x * M[2, :2], M[1, :2] - y * M[2, :2]])
    b = -np.array([M[0, 2] - x * M[2, 2], M[1, 2] - y * M[2, 2]])
    return np.linalg.solve(A, b)


def _compose(s):
    """Independent compositor: per pixel, list all alphas first, then use cumulative products."""
    W, H = s['W'], s['H']
    gx = (W + 15) // 16
    img, opa, wsum, depth, last = np.zeros((3, H, W)), np.zeros((H, W)), np.zeros((H, W)), np.zeros((H, W)), np.zeros((H, W), int)
    for y in range(H):
        for x in range(W):
            t = (y // 16) * gx + x // 16
            r0, r1 = s['ranges'][t]
            alphas, cols, zs, pos = [], [], [], []
            for e in range(r0, r1):
                i = s['point_list'][e]
                M = s['trans_mat'][i]
                try:
                    u, v = _uv(M, x, y)
                except np.linalg.LinAlgError:
                    continue
                d = s['means2D'][i] - np.array([x, y])
                rho = min(u * u + v * v, 2 * (d @ d))
                z = u * M[2, 0] + v * M[2, 1] + M[2, 2]
                if z < s['near']:
                    continue
                a = min(0.99, s['normal_opacity'][i, 3] * np.exp(-0.5 * rho))
                if a < 1 / 255:
                    continue
                alphas.append(a), cols.append(s['colors'][i]), zs.append(z), pos.append(e - r0 + 1)
            T = 1.0
            for a, c, z, p in zip(alphas, cols, zs, pos):
                if T * (1 - a) < 1e-4:
                    break
                img[:, y, x] += a * T * c
                depth[y, x] += a * T * z
                wsum[y, x] += a * T
                T *= 1 - a
                last[y, x] = p
            opa[y, x] = 1 - T
    return img, opa, wsum, depth, last


def test_single_surfel_closed_form(oracle_mod):
    O = oracle_mod
    W, H = GOLD['W'], GOLD['H']
    for case in GOLD['cases']:
        a = lambda k: np.ascontiguousarray(np.array(case[k] if k in case else GOLD[k], np.float64))
        m2, colors, tm, no, dep, radii, tt = O.preprocess_forward(W, H, 0, a('means3D'), a('scales'), a('rotations'),
                                                                  a('opacity'), a('shs').reshape(1, 1, 3), None,
                                                                  a('Tw2v'), a('Tv2c'), a('campos'))
        ranges, pl = O.prepare(W, H, m2.astype(np.float32), dep.astype(np.float32), radii, tt)
        oc, oo, oe, _, nc = O.render_forward(W, H, m2, colors, no, tm, pl, ranges, 0.2, 100.0, False)
        expect = np.zeros((H, W))
        for y in range(0, H, 3):
            for x in range(0, W, 3):
                u, v = _uv(tm[0], x, y)
                d = m2[0] - np.array([x, y])
                al = min(0.99, case['opacity'][0][0] * np.exp(-0.5 * min(u * u + v * v, 2 * d @ d)))
                z = u * tm[0, 2, 0] + v * tm[0, 2, 1] + tm[0, 2, 2]
                expect[y, x] = al if (al >= 1 / 255 and z >= 0.2) else 0.0
                assert abs(oo[y, x] - expect[y, x]) < 1e-9
                assert np.abs(oc[:, y, x] - expect[y, x] * colors[0]).max() < 1e-9
        assert (expect > 0).sum() > 50  # the surfel is actually visible in the sampled pixels


def test_matches_independent_compositor_and_invariants(oracle_mod):
    O = oracle_mod
    s = _small_scene(O)
    oc, oo, oe, _, nc = O.render_forward(s['W'], s['H'], s['means2D'], s['colors'], s['normal_opacity'],
                                         s['trans_mat'], s['point_list'], s['ranges'], s['near'], s['far'], False)
    img, opa, wsum, depth, last = _compose(s)
    assert np.abs(oc - img).max() < 1e-9 and np.abs(oo - opa).max() < 1e-9
    assert np.abs(oe[0] - depth).max() < 1e-8 and np.abs(oe[8] - wsum).max() < 1e-9
    assert np.array_equal(nc[0], last)
    assert np.abs(oe[8] - oo).max() < 1e-9  # telescoping: sum of weights == accumulated opacity
    assert (oo > 0.3).any() and (nc[0] > 3).any()
    only = O.render_forward(s['W'], s['H'], s['means2D'], s['colors'], s['normal_opacity'], s['trans_mat'],
                            s['point_list'], s['ranges'], s['near'], s['far'], True)
    assert only[2] is None and np.array_equal(only[0], oc) and not only[4][1].any()
    # median contributor: last splat seen while T > 0.5, else -1
    assert ((nc[1] == -1) == (nc[0] == 0)).all()


def test_float_matches_double(oracle_mod):
    O = oracle_mod
    s = _small_scene(O)
    f32 = lambda a: np.ascontiguousarray(a.astype(np.float32))
    o64 = O.render_forward(s['W'], s['H'], s['means2D'], s['colors'], s['normal_opacity'], s['trans_mat'],
                           s['point_list'], s['ranges'], s['near'], s['far'], False)
    o32 = O.render_forward(s['W'], s['H'], f32(s['means2D']), f32(s['colors']), f32(s['normal_opacity']),
                           f32(s['trans_mat']), s['point_list'], s['ranges'], s['near'], s['far'], False)
    assert np.abs(o64[0] - o32[0]).max() < 1e-4 and np.abs(o64[1] - o32[1]).max() < 1e-4


def _never_filtered(s, i):
    """True if no contributing pixel of surfel i takes the screen-space low-pass branch (rho2d < rho3d)."""
    M = s['trans_mat'][i]
    for y in range(s['H']):
        for x in range(s['W']):
            try:
                u, v = _uv(M, x, y)
            except np.linalg.LinAlgError:
                return False
            d = s['means2D'][i] - np.array([x, y])
            r3, r2 = u * u + v * v, 2 * d @ d
            if s['normal_opacity'][i, 3] * np.exp(-0.5 * min(r3, r2)) >= 1 / 255 and r2 < r3:
                return False
    return True


@pytest.mark.parametrize("channels", ["image_opacity_normal", "depth_median_distortion"])
def test_backward_matches_finite_differences(oracle_mod, channels):
    """Image, opacity and normal gradients are exact derivatives for every surfel. For the depth-type channels the
    reference drops the d(depth)/d(intersection) chain for pixels where the low-pass filter wins
    (gs_2d_redner.cu:524-533 only adds dL_dz * (s, 1) to the third row there), and the oracle follows it; those
    channels are therefore checked on surfels that never take that branch, where the gradient is exact."""
    O = oracle_mod
    depth_like = channels == "depth_median_distortion"
    s = _small_scene(O, P=30, W=32, H=32, seed=4, scale_mul=40.0 if depth_like else 6.0)
    W, H = s['W'], s['H']
    rng = np.random.default_rng(1)
    g_img, g_opa, g_ext = np.zeros((3, H, W)), np.zeros((H, W)), np.zeros((9, H, W))
    if depth_like:
        g_ext[0], g_ext[4], g_ext[5] = rng.normal(size=(3, H, W))
    else:
        g_img, g_opa = rng.normal(size=(3, H, W)), rng.normal(size=(H, W))
        g_ext[1:4] = rng.normal(size=(3, H, W))

    def fwd(**over):
        t = dict(s)
        t.update(over)
        return O.render_forward(W, H, t['means2D'], t['colors'], t['normal_opacity'], t['trans_mat'], t['point_list'],
                                t['ranges'], t['near'], t['far'], False)

    def loss(**over):
        oc, oo, oe, _, _ = fwd(**over)
        return (oc * g_img).sum() + (oo * g_opa).sum() + (oe * g_ext).sum()

    oc, oo, oe, _, nc = fwd()
    gc, gm, gt, gn = O.render_backward(s['means2D'], s['normal_opacity'], s['colors'], s['trans_mat'], None, oo, oe,
                                       None, np.ascontiguousarray(g_img), np.ascontiguousarray(g_opa),
                                       np.ascontiguousarray(g_ext), None, s['ranges'], s['point_list'], nc, s['near'],
                                       s['far'])
    used = list(np.unique(s['point_list']))
    if depth_like:
        used = [i for i in used if _never_filtered(s, i)]
        assert len(used) >= 4
    eps = 1e-6
    checked = 0
    l0 = loss()
    for name, grad in (('colors', gc), ('trans_mat', gt), ('normal_opacity', gn), ('means2D', gm)):
        flat = grad.reshape(grad.shape[0], -1)
        for i in used[:8]:
            for a in range(flat.shape[1]):
                p, m = s[name].copy(), s[name].copy()
                p.reshape(p.shape[0], -1)[i, a] += eps
                m.reshape(m.shape[0], -1)[i, a] -= eps
                lp, lm = loss(**{name: p}), loss(**{name: m})
                if abs((lp - l0) - (l0 - lm)) > 1e-9:
                    continue  # a discrete event (threshold crossing, median switch) sits inside the FD stencil
                fd = (lp - lm) / (2 * eps)
                assert abs(fd - flat[i, a]) < 1e-5 * max(1.0, abs(fd)), (name, i, a, fd, flat[i, a])
                checked += 1
    assert checked > 80


def test_topk_weights_are_the_largest_blend_weights(oracle_mod):
    """Per-pixel top-k of w = alpha * T against an independent numpy pass. The top-k kernel tests `near` against the
    surfel's centre depth when the low-pass filter wins (gaussian_topk.cu:180-181), unlike the render kernels."""
    O = oracle_mod
    s = _small_scene(O, P=60, seed=2)
    W, H, K = s['W'], s['H'], 3
    ti, tw = np.zeros((H, W, K), np.int32), np.zeros((H, W, K))
    assert O.call("gs_2d_topk_weights_f64", K, W, H, s['near'], s['far'], s['means2D'], s['normal_opacity'],
                  s['trans_mat'], s['ranges'], s['point_list'], ti, tw) == 0
    assert (np.diff(tw, axis=-1) <= 0).all()  # descending
    assert ((ti == -1) == (tw == 0)).all()
    gx = (W + 15) // 16
    nonempty = 0
    for y in range(H):
        for x in range(W):
            r0, r1 = s['ranges'][(y // 16) * gx + x // 16]
            T, ws = 1.0, []
            for e in range(r0, r1):
                i = s['point_list'][e]
                M = s['trans_mat'][i]
                u, v = _uv(M, x, y)
                d = s['means2D'][i] - np.array([x, y])
                r3, r2 = u * u + v * v, 2 * (d @ d)
                z = (u * M[2, 0] + v * M[2, 1] + M[2, 2]) if r3 <= r2 else M[2, 2]
                if z < s['near']:
                    continue
                a = min(0.99, s['normal_opacity'][i, 3] * np.exp(-0.5 * min(r3, r2)))
                if a < 1 / 255:
                    continue
                if T * (1 - a) < 1e-4:
                    break
                ws.append((a * T, i))
                T *= 1 - a
            ws.sort(key=lambda t: -t[0])
            top = ws[:K] + [(0.0, -1)] * (K - len(ws[:K]))
            assert np.allclose(tw[y, x], [t[0] for t in top], atol=1e-12)
            assert list(ti[y, x]) == [t[1] for t in top]
            nonempty += len(ws) > K
    assert nonempty > 20
