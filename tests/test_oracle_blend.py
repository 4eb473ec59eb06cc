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


def _pixel_entries(s, x, y):
    """Every list entry of pixel (x, y) that passes the alpha and near tests, in list order, BEFORE the transmittance
    cut: (alpha, z, surfel id, 1-based list position, (u, v))."""
    gx = (s['W'] + 15) // 16
    r0, r1 = s['ranges'][(y // 16) * gx + x // 16]
    out = []
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
        out.append((a, z, int(i), e - r0 + 1, (u, v)))
    return out


def _compose(s, trans_mat_t2=None, flow_by_opacity=False):
    """Independent compositor: per pixel, list all alphas first, then work from closed forms on the whole list
    (cumulative products for T, explicit sums, an explicit pair sum for the distortion, an explicit running arg-max for
    the max-weight counter) instead of the kernel's running state."""
    W, H, P = s['W'], s['H'], s['normal_opacity'].shape[0]
    near, far = s['near'], s['far']
    o = dict(image=np.zeros((3, H, W)), opacity=np.zeros((H, W)), wsum=np.zeros((H, W)), depth=np.zeros((H, W)),
             last=np.zeros((H, W), int), normal=np.zeros((3, H, W)), median_depth=np.zeros((H, W)),
             median_pos=np.full((H, W), -1), M1=np.zeros((H, W)), M2=np.zeros((H, W)), distortion=np.zeros((H, W)),
             flow=np.zeros((H, W, 2)), accum_max_count=np.zeros(P, np.int64), accum_weights_p=np.zeros(P),
             accum_weights_count=np.zeros(P, np.int64))
    for y in range(H):
        for x in range(W):
            ent = _pixel_entries(s, x, y)
            # transmittance in front of each entry; the list is cut at the first entry that would leave T < 1e-4
            kept, T = [], 1.0
            for a, z, i, pos, uv in ent:
                if T * (1 - a) < 1e-4:
                    break
                kept.append((a, z, i, pos, uv, T))
                T *= 1 - a
            o['opacity'][y, x] = 1 - T
            if not kept:
                continue
            al = np.array([k[0] for k in kept])
            zs = np.array([k[1] for k in kept])
            ids = [k[2] for k in kept]
            Ts = np.array([k[5] for k in kept])
            assert np.allclose(Ts, np.concatenate([[1.0], np.cumprod(1 - al)[:-1]]))
            w = al * Ts
            m = far / (far - near) * (1 - near / zs)
            o['image'][:, y, x] = (w[:, None] * s['colors'][ids]).sum(0)
            o['normal'][:, y, x] = (w[:, None] * s['normal_opacity'][ids, :3]).sum(0)
            o['depth'][y, x], o['wsum'][y, x] = (w * zs).sum(), w.sum()
            o['M1'][y, x], o['M2'][y, x] = (w * m).sum(), (w * m * m).sum()
            o['distortion'][y, x] = sum(w[a] * w[b] * (m[a] - m[b]) ** 2 for a in range(len(w)) for b in range(a))
            o['last'][y, x] = kept[-1][3]
            half = np.nonzero(Ts > 0.5)[0][-1]  # T in front of the first entry is 1, so there always is one
            o['median_depth'][y, x], o['median_pos'][y, x] = zs[half], kept[half][3]
            for n in range(len(w)):
                o['accum_weights_p'][ids[n]] += w[n]
                o['accum_weights_count'][ids[n]] += 1
                o['accum_max_count'][ids[int(np.argmax(w[:n + 1]))]] += 1  # first of equal maxima, as `weight_max < w`
            if trans_mat_t2 is not None:
                raw = np.zeros(2)
                for n, k in enumerate(kept):
                    q = trans_mat_t2[k[2]] @ np.array([k[4][0], k[4][1], 1.0])
                    q2 = q[2] if abs(q[2]) >= 1e-5 else 1e-5
                    raw += w[n] * (q[:2] / q2 - np.array([x, y]))
                o['flow'][y, x] = raw / (o['opacity'][y, x] if flow_by_opacity else w.sum())
    return o


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
    c = _compose(s)
    assert np.abs(oc - c['image']).max() < 1e-9 and np.abs(oo - c['opacity']).max() < 1e-9
    assert np.abs(oe[0] - c['depth']).max() < 1e-8 and np.abs(oe[8] - c['wsum']).max() < 1e-9
    assert np.array_equal(nc[0], c['last'])
    assert np.abs(oe[8] - oo).max() < 1e-9  # telescoping: sum of weights == accumulated opacity
    assert (oo > 0.3).any() and (nc[0] > 3).any()
    only = O.render_forward(s['W'], s['H'], s['means2D'], s['colors'], s['normal_opacity'], s['trans_mat'],
                            s['point_list'], s['ranges'], s['near'], s['far'], True)
    assert only[2] is None and np.array_equal(only[0], oc) and not only[4][1].any()
    # median contributor: last splat seen while T > 0.5, else -1
    assert ((nc[1] == -1) == (nc[0] == 0)).all()


@pytest.mark.parametrize("seed,scale_mul", [(0, 6.0), (3, 25.0)])
def test_every_forward_output_matches_independent_compositor(oracle_mod, seed, scale_mul):
    """Normals, median depth and median contributor, M1, M2, the distortion as the explicit pair sum
    sum_i sum_{j<i} w_i w_j (m_i - m_j)^2 (what the recurrence of gs_2d_redner.cu:163-168 telescopes to), optical flow
    with the sum-of-weights normalisation (:230-233) and the three accum_* side outputs, the max-weight counter as a
    per-pixel replay of a running arg-max whose flag is never reset (:180-197): none of these is restated from the
    kernel's running-state form."""
    O = oracle_mod
    s = _small_scene(O, P=60, seed=seed, scale_mul=scale_mul)
    W, H, P = s['W'], s['H'], s['normal_opacity'].shape[0]
    rng = np.random.default_rng(seed)
    t2 = s['trans_mat'] + 0.05 * rng.normal(size=s['trans_mat'].shape) * np.abs(s['trans_mat']).mean()
    amc, awp, awc = np.zeros(P, np.int32), np.zeros(P), np.zeros(P, np.int32)
    oc, oo, oe, of, nc = O.render_forward(W, H, s['means2D'], s['colors'], s['normal_opacity'], s['trans_mat'],
                                          s['point_list'], s['ranges'], s['near'], s['far'], False,
                                          np.ascontiguousarray(t2), amc, awp, awc)
    c = _compose(s, trans_mat_t2=t2)
    assert (c['last'] >= 3).sum() > 50 and (c['median_pos'] != c['last']).sum() > 20  # deep lists, median not last
    assert np.abs(oe[1:4] - c['normal']).max() < 1e-9
    assert np.abs(oe[4] - c['median_depth']).max() < 1e-9 and np.array_equal(nc[1], c['median_pos'])
    assert np.abs(oe[6] - c['M1']).max() < 1e-9 and np.abs(oe[7] - c['M2']).max() < 1e-9
    assert np.abs(oe[5] - c['distortion']).max() < 1e-9 and c['distortion'].max() > 1e-6
    assert np.abs(of - c['flow']).max() < 1e-7 * max(1.0, np.abs(c['flow']).max()) and np.abs(c['flow']).max() > 1e-2
    assert np.array_equal(awc, c['accum_weights_count']) and np.abs(awp - c['accum_weights_p']).max() < 1e-9
    assert np.array_equal(amc, c['accum_max_count'])
    assert amc.sum() == awc.sum() and (amc != awc).any()  # one count per contributing pair, credited to the arg-max
    # without auxiliary outputs the kernel keeps no running maximum: only the image and opacity are produced and the
    # max-weight counter is not touched (the flag lives in the auxiliary branch, :172-184)
    amc2 = np.zeros(P, np.int32)
    only = O.render_forward(W, H, s['means2D'], s['colors'], s['normal_opacity'], s['trans_mat'], s['point_list'],
                            s['ranges'], s['near'], s['far'], True, None, amc2, None, None)
    assert not amc2.any() and np.array_equal(only[0], oc) and np.array_equal(only[1], oo)
    # accumulation: a second call adds to the caller's buffers
    O.render_forward(W, H, s['means2D'], s['colors'], s['normal_opacity'], s['trans_mat'], s['point_list'], s['ranges'],
                     s['near'], s['far'], False, None, amc, awp, awc)
    assert np.array_equal(amc, 2 * c['accum_max_count']) and np.array_equal(awc, 2 * c['accum_weights_count'])


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


@pytest.mark.parametrize("channels", ["image_opacity_normal", "depth_median_distortion", "flow"])
def test_backward_matches_finite_differences(oracle_mod, channels):
    """Image, opacity and normal gradients are exact derivatives for every surfel. For the depth-type channels and the
    optical flow the reference drops the chain through the intersection point for pixels where the low-pass filter wins
    (gs_2d_redner.cu:524-533 only adds dL_dz * (s, 1) to the third row there), and the oracle follows it; those
    channels are therefore checked on surfels that never take that branch, where the gradient is exact.
    Optical flow: the reference's gradient of the normalisation flow = raw / sum_w is NOT the derivative of that
    quotient: it takes dL/dsum_w = -(g . flow) / sum_w^2 (:328-332), one division by sum_w more than the quotient rule
    gives. The check therefore differentiates the surrogate  sum_pix (g / sw0) . raw(theta) + c0 * sum_w(theta)  with
    sw0 and c0 = -(g . flow0) / sw0^2 frozen at the base point, which has exactly the reference's gradient."""
    O = oracle_mod
    depth_like = channels != "image_opacity_normal"
    s = _small_scene(O, P=30, W=32, H=32, seed=4, scale_mul=40.0 if depth_like else 6.0)
    W, H = s['W'], s['H']
    rng = np.random.default_rng(1)
    g_img, g_opa, g_ext, g_flow, t2 = np.zeros((3, H, W)), np.zeros((H, W)), np.zeros((9, H, W)), None, None
    if channels == "depth_median_distortion":
        g_ext[0], g_ext[4], g_ext[5] = rng.normal(size=(3, H, W))
    elif channels == "flow":
        g_flow = np.ascontiguousarray(rng.normal(size=(H, W, 2)))
        t2 = np.ascontiguousarray(s['trans_mat'] + 0.05 * rng.normal(size=s['trans_mat'].shape)
                                  * np.abs(s['trans_mat']).mean())
    else:
        g_img, g_opa = rng.normal(size=(3, H, W)), rng.normal(size=(H, W))
        g_ext[1:4] = rng.normal(size=(3, H, W))

    def fwd(**over):
        t = dict(s)
        t.update(over)
        return O.render_forward(W, H, t['means2D'], t['colors'], t['normal_opacity'], t['trans_mat'], t['point_list'],
                                t['ranges'], t['near'], t['far'], False, t2)

    oc, oo, oe, of, nc = fwd()
    if g_flow is not None:
        sw0 = np.where(oe[8] == 0, 1.0, oe[8])
        c0 = -(g_flow * of).sum(-1) / sw0 ** 2
        g_raw = g_flow / sw0[..., None]

    def loss(**over):
        oc, oo, oe, of, _ = fwd(**over)
        val = (oc * g_img).sum() + (oo * g_opa).sum() + (oe * g_ext).sum()
        if g_flow is not None:
            val += (g_raw * (of * oe[8][..., None])).sum() + (c0 * oe[8]).sum()
        return val

    gc, gm, gt, gn = O.render_backward(s['means2D'], s['normal_opacity'], s['colors'], s['trans_mat'], t2, oo, oe,
                                       of, np.ascontiguousarray(g_img), np.ascontiguousarray(g_opa),
                                       np.ascontiguousarray(g_ext), g_flow, s['ranges'], s['point_list'], nc, s['near'],
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
                if abs((lp - l0) - (l0 - lm)) > 1e-9 * max(1.0, abs(l0)):
                    continue  # a discrete event (threshold crossing, median switch) sits inside the FD stencil
                fd = (lp - lm) / (2 * eps)
                assert abs(fd - flat[i, a]) < 1e-5 * max(1.0, abs(fd)), (name, i, a, fd, flat[i, a])
                checked += 1
    assert checked > 80
    if channels == "flow":
        assert np.abs(gt).max() > 1e-3 and np.abs(gn[:, 3]).max() > 1e-3


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
