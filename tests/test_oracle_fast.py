"""Pins the oracle's "fast" surfel path (oracle/gs2d_fast.cpp) against the independently pinned standard path and by
brute force:
  * with intrinsics Tv2s = (ndc2pix @ Tv2c)[:3,:3] and a view matrix without x/y translation the fast transform equals
    the standard one (the relation the reference's own test checks, gs_2d_fast_render.py:908-961), the adjugate solves
    the same plane-plane intersection, so images and all gradients must agree with the standard path through the chain
    rule d(adj)/dM;
  * the fused binning keeps exactly the tiles of the rectangle whose corner test passes (double-precision brute force,
    near-ties excluded), pads the rest with (T << 32, -1) and orders x-major within a surfel;
  * the per-splat formulation differs from the per-pixel one only in its channel set (finite differences);
  * snapshots are the running state before every 32nd list entry.
"""
import numpy as np
import pytest
import torch


def _setup(O, P=60, W=64, H=48, seed=0, scale_mul=8.0, dtype=np.float64):
    from fast_sp_gs_amd import scenes
    sc, _ = scenes.config0(P=P, size=64, seed=seed)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    f = lambda t: np.ascontiguousarray(t.numpy().astype(dtype))
    s = dict(means3D=f(sc.means3D) * 0.6, scales=f(sc.scales) * scale_mul, rotations=f(sc.rotations),
             opacities=f(sc.opacities), shs=f(sc.shs), Tw2v=f(cam.Tw2v), Tv2c=f(cam.Tv2c), campos=f(cam.campos), W=W,
             H=H)
    ndc2pix = np.array([[W / 2, 0, 0, (W - 1) / 2], [0, H / 2, 0, (H - 1) / 2], [0, 0, 0, 1.0]])
    s['Tv2s'] = np.ascontiguousarray((ndc2pix @ s['Tv2c'].astype(np.float64))[:, [0, 1, 2]].astype(dtype))
    return s


def _std(O, s):
    return O.preprocess_forward(s['W'], s['H'], 3, s['means3D'], s['scales'], s['rotations'], s['opacities'], s['shs'],
                                None, s['Tw2v'], s['Tv2c'], s['campos'])


def _fast(O, s):
    return O.fast_preprocess_forward(s['W'], s['H'], 3, s['means3D'], s['scales'], s['rotations'], s['opacities'],
                                     s['shs'], None, s['Tw2v'], s['Tv2s'], s['campos'])


def test_fast_transform_equals_standard_and_adjugate(oracle_mod):
    O = oracle_mod
    s = _setup(O)
    m2, colors, tm, no, dep, radii, tt = _std(O, s)
    fm2, fcolors, ftm, fim, fno, fdep, fradii, ftt = _fast(O, s)
    assert np.array_equal(radii, fradii) and np.array_equal(tt, ftt)
    for a, b in ((m2, fm2), (colors, fcolors), (tm, ftm), (no, fno), (dep, fdep)):
        assert np.abs(a - b).max() < 1e-9 * max(1.0, np.abs(a).max())
    vis = radii > 0
    for i in np.flatnonzero(vis)[:20]:
        M = ftm[i]
        assert np.allclose(fim[i] @ M, np.linalg.det(M) * np.eye(3), atol=1e-9 * np.abs(fim[i]).max() * np.abs(M).max())
        # p = IM (x, y, 1) is the intersection of the two pixel planes: k x l
        x, y = 13.0, 29.0
        k, l = x * M[2] - M[0], y * M[2] - M[1]
        assert np.allclose(fim[i] @ np.array([x, y, 1.0]), np.cross(k, l), rtol=1e-9, atol=1e-9 * np.abs(fim[i]).max())
    assert not fim[~vis].any()


def test_fast_transmat_ops_and_backward(oracle_mod):
    O = oracle_mod
    s = _setup(O, P=20)
    P = 20
    tm, nrm = np.zeros((P, 3, 3)), np.zeros((P, 3))
    assert O.call("gs_2d_fast_compute_transmat_forward_f64", P, s['means3D'], s['scales'], s['rotations'], s['Tw2v'],
                  s['Tv2s'], tm, nrm) == 0
    Tw2c = np.ascontiguousarray(s['Tv2c'] @ s['Tw2v'])
    tm_std, n_std = np.zeros((P, 3, 3)), np.zeros((P, 3))
    O.call("gs_2d_compute_transmat_forward_f64", P, s['W'], s['H'], s['means3D'], s['scales'], s['rotations'],
           s['Tw2v'], Tw2c, tm_std, n_std)
    assert np.abs(tm - tm_std).max() < 1e-9 * np.abs(tm).max() and np.abs(nrm - n_std).max() < 1e-12
    rng = np.random.default_rng(0)
    gM, gN = np.ascontiguousarray(rng.normal(size=(P, 3, 3))), np.ascontiguousarray(rng.normal(size=(P, 3)))
    out = [np.zeros((P, 3)), np.zeros((P, 2)), np.zeros((P, 4))]
    O.call("gs_2d_fast_compute_transmat_backward_f64", P, s['means3D'], s['scales'], s['rotations'], s['Tw2v'],
           s['Tv2s'], gM, gN, *out)
    ref = [np.zeros((P, 3)), np.zeros((P, 2)), np.zeros((P, 4))]
    O.call("gs_2d_compute_transmat_backward_f64", P, s['W'], s['H'], s['means3D'], s['scales'], s['rotations'],
           s['Tw2v'], Tw2c, gM, gN, *ref)
    for a, b in zip(out, ref):
        assert np.abs(a - b).max() < 1e-9 * max(1.0, np.abs(b).max())


def test_fused_binning_corner_test(oracle_mod):
    O = oracle_mod
    s32 = _setup(O, P=300, W=160, H=96, seed=2, dtype=np.float32)
    fm2, fcolors, ftm, fim, fno, fdep, fradii, ftt = _fast(O, s32)
    W, H = s32['W'], s32['H']
    gx, gy = (W + 15) // 16, (H + 15) // 16
    T = gx * gy
    ranges, pl, keys = O.fast_prepare(W, H, fm2, fim, fdep, s32['opacities'], fradii, ftt, return_keys=True)
    assert pl.size == ftt.sum()
    # expected membership by a double-precision corner test; near-ties (|W| tiny relative to its terms) are skipped
    lib = O.lib()
    n_pad = int((pl == -1).sum())
    assert n_pad > 0 and (keys[pl == -1] >> 32 == T).all() and (pl[-n_pad:] == -1).all()
    tiles_of = {}
    for t in range(T):
        for e in range(ranges[t, 0], ranges[t, 1]):
            assert keys[e] >> 32 == t
            tiles_of.setdefault(int(pl[e]), set()).add(t)
    assert ranges[:, 1].max() == pl.size - n_pad
    checked = kept = 0
    for i in np.flatnonzero(fradii > 0):
        r = fradii[i]
        x0 = min(gx, max(0, int((fm2[i, 0] - r) / 16))); x1 = min(gx, max(0, int((fm2[i, 0] + r + 15) / 16)))
        y0 = min(gy, max(0, int((fm2[i, 1] - r) / 16))); y1 = min(gy, max(0, int((fm2[i, 1] + r + 15) / 16)))
        im64 = np.ascontiguousarray(fim[i].astype(np.float64))
        d = -2 * np.log(2.0) * (7.9886846867721655 + np.log2(float(s32['opacities'][i, 0])))
        for x in range(x0, x1):
            for y in range(y0, y1):
                vals = []
                for (u, v) in ((x, y), (x + 1, y), (x, y + 1), (x + 1, y + 1)):
                    p = im64 @ np.array([16.0 * u, 16.0 * v, 1.0])
                    vals.append(p[0] ** 2 + p[1] ** 2 + d * p[2] ** 2)
                scale = max(abs(d) * (im64[2] @ np.array([16.0 * x, 16.0 * y, 1.0])) ** 2, 1e-30)
                if min(abs(v) for v in vals) < 1e-4 * scale:
                    continue  # too close to the conic for a float/double comparison
                expect = min(vals) <= 0
                assert expect == bool(lib.oracle_fast_corner_test_f64(O._p(im64), float(s32['opacities'][i, 0]), x, y))
                assert expect == ((y * gx + x) in tiles_of.get(int(i), set())), (i, x, y, vals)
                checked += 1
                kept += expect
    assert checked > 300 and 0 < kept < checked
    # within a tile: ascending depth bits, ties by index; overall x-major emission does not matter after the sort
    bits = fdep.view(np.uint32)
    for t in range(T):
        seg = pl[ranges[t, 0]:ranges[t, 1]]
        k = [(int(bits[i]), int(i)) for i in seg]
        assert k == sorted(k)


def _render_pair(O, s):
    m2, colors, tm, no, dep, radii, tt = _std(O, s)
    fm2, fcolors, ftm, fim, fno, fdep, fradii, ftt = _fast(O, s)
    ranges, pl = O.prepare(s['W'], s['H'], m2.astype(np.float32), dep.astype(np.float32), radii, tt)
    return (m2, colors, tm, no), (fm2, fcolors, ftm, fim, fno), ranges, pl


def test_fast_blend_matches_standard_blend(oracle_mod):
    O = oracle_mod
    s = _setup(O, P=50, W=48, H=32)
    W, H = s['W'], s['H']
    (m2, colors, tm, no), (fm2, fcolors, ftm, fim, fno), ranges, pl = _render_pair(O, s)
    oc, oo, oe, _, nc = O.render_forward(W, H, m2, colors, no, tm, pl, ranges, 0.2, 100.0, False)
    foc, foo, foe, fnc = O.fast_render_forward(W, H, 0.2, 100.0, False, fm2, fcolors, fno, ftm, fim, pl, ranges)[:4]
    assert np.abs(oc - foc).max() < 1e-9 and np.abs(oo - foo).max() < 1e-9 and np.array_equal(nc, fnc)
    assert np.abs(oe[:8] - foe).max() < 1e-8
    # backward: standard dL/dM == fast dL/dM + adjugate chain rule applied to dL/d(adj); other gradients identical
    rng = np.random.default_rng(0)
    g_img, g_opa = rng.normal(size=(3, H, W)), rng.normal(size=(H, W))
    g_ext9 = np.zeros((9, H, W))
    g_ext9[:6] = rng.normal(size=(6, H, W))
    gc, gm, gt, gn = O.render_backward(m2, no, colors, tm, None, oo, oe, None, g_img, g_opa, g_ext9, None, ranges, pl,
                                       nc, 0.2, 100.0)
    fgc, fgm, fgt, fgi, fgn = O.fast_render_backward(0.2, 100.0, 0, fm2, fno, fcolors, ftm, fim, foo, foe, g_img, g_opa,
                                                     np.ascontiguousarray(g_ext9[:8]), ranges, pl, fnc)
    for a, b in ((gc, fgc), (gm, fgm), (gn, fgn)):
        assert np.abs(a - b).max() < 1e-8 * max(1.0, np.abs(a).max())
    # chain rule through adj(M) by finite differences of the adjugate itself
    total = fgt.copy()
    eps = 1e-7
    for i in np.unique(pl):
        for a in range(9):
            Mp, Mm = ftm[i].reshape(-1).copy(), ftm[i].reshape(-1).copy()
            Mp[a] += eps
            Mm[a] -= eps
            adj = lambda M: np.stack([np.cross(M[1], M[2]), np.cross(M[2], M[0]), np.cross(M[0], M[1])], 1)
            d_adj = (adj(Mp.reshape(3, 3)) - adj(Mm.reshape(3, 3))) / (2 * eps)
            total[i].reshape(-1)[a] += (d_adj * fgi[i]).sum()
    assert np.abs(total - gt).max() < 1e-5 * max(1.0, np.abs(gt).max())
    # ... and the fast preprocess backward folds exactly that chain rule into dL/dM before continuing as the standard
    g3, gs, gr, go, gsh, _, gm2 = O.preprocess_backward(W, H, 3, s['means3D'], s['scales'], s['rotations'], s['shs'],
                                                        None, s['Tw2v'], s['Tv2c'], s['campos'], tm, _std(O, s)[5],
                                                        colors, gm, gt, gc, gn)
    fr = O.fast_preprocess_backward(W, H, 3, s['means3D'], s['scales'], s['rotations'], s['shs'], None, s['Tw2v'],
                                    s['Tv2s'], s['campos'], ftm, _fast(O, s)[6], fcolors, fgm, fgt, fgi, fgc, fgn)
    for a, b in zip((g3, gs, gr, go, gsh), fr[:5]):
        assert np.abs(a - b).max() < 1e-5 * max(1.0, np.abs(a).max())
    # densification proxy: the fast path uses the ACCUMULATED dL/dM (gs_2d_fast_preprocess.cu:606-608)
    vis = _fast(O, s)[6] > 0
    assert vis.any() and not np.allclose(fr[6][vis], gm2[vis])


def test_per_splat_form_and_snapshots(oracle_mod):
    O = oracle_mod
    s = _setup(O, P=50, W=48, H=32, scale_mul=40.0)
    W, H = s['W'], s['H']
    _, (fm2, fcolors, ftm, fim, fno), ranges, pl = _render_pair(O, s)
    lens = ranges[:, 1] - ranges[:, 0]
    bucket_offset = np.ascontiguousarray(np.cumsum((lens + 31) // 32).astype(np.int64))
    out = O.fast_render_forward(W, H, 0.2, 100.0, False, fm2, fcolors, fno, ftm, fim, pl, ranges, bucket_offset)
    foc, foo, foe, fnc, max_contrib, b2t, sT, sacc, saux = out
    gx = (W + 15) // 16
    assert np.array_equal(b2t, np.repeat(np.arange(len(lens)), (lens + 31) // 32))
    for t in np.flatnonzero(lens > 0):
        ty, tx = divmod(t, gx)
        blk = fnc[0, ty * 16:ty * 16 + 16, tx * 16:tx * 16 + 16]
        assert max_contrib[t] == blk.max()
        b0 = 0 if t == 0 else bucket_offset[t - 1]
        assert np.all(sT[b0].reshape(16, 16)[:blk.shape[0], :blk.shape[1]] == 1.0)  # first snapshot: untouched state
        assert not sacc[b0].any()
    # channel set of the per-splat form: no distortion gradient, M1/M2 as weighted sums (M1 without its depth term)
    rng = np.random.default_rng(3)
    zero8 = np.zeros((8, H, W))
    def grads(form, ch):
        ge = zero8.copy()
        ge[ch] = rng.normal(size=(H, W))
        return O.fast_render_backward(0.2, 100.0, form, fm2, fno, fcolors, ftm, fim, foo, foe, np.zeros((3, H, W)),
                                      np.zeros((H, W)), ge, ranges, pl, fnc)
    assert not any(np.abs(g).max() > 0 for g in grads(1, 5))        # distortion ignored
    assert any(np.abs(g).max() > 0 for g in grads(0, 5))
    assert not any(np.abs(g).max() > 0 for g in grads(0, 6))        # per-pixel form ignores M1 / M2
    assert any(np.abs(g).max() > 0 for g in grads(1, 7))
    # M2 map gradient of the per-splat form is the true derivative (surfels that never take the low-pass branch)
    g_M2 = rng.normal(size=(H, W))
    ge = zero8.copy()
    ge[7] = g_M2
    fgc, fgm, fgt, fgi, fgn = O.fast_render_backward(0.2, 100.0, 1, fm2, fno, fcolors, ftm, fim, foo, foe,
                                                     np.zeros((3, H, W)), np.zeros((H, W)), ge, ranges, pl, fnc)
    def loss(no_):
        o = O.fast_render_forward(W, H, 0.2, 100.0, False, fm2, fcolors, no_, ftm, fim, pl, ranges)
        return (o[2][7] * g_M2).sum()
    eps, checked = 1e-6, 0
    l0 = loss(fno)
    for i in np.unique(pl)[:12]:
        p, m = fno.copy(), fno.copy()
        p[i, 3] += eps
        m[i, 3] -= eps
        lp, lm = loss(p), loss(m)
        if abs((lp - l0) - (l0 - lm)) > 1e-9:
            continue
        assert abs((lp - lm) / (2 * eps) - fgn[i, 3]) < 1e-5 * max(1.0, abs(fgn[i, 3]))
        checked += 1
    assert checked >= 6


def _flow_case(O, seed=0, scale_mul=25.0, P=50, W=48, H=32):
    s = _setup(O, P=P, W=W, H=H, seed=seed, scale_mul=scale_mul)
    (m2, colors, tm, no), (fm2, fcolors, ftm, fim, fno), ranges, pl = _render_pair(O, s)
    rng = np.random.default_rng(seed + 11)
    t2 = np.ascontiguousarray(ftm + 0.05 * rng.normal(size=ftm.shape) * np.abs(ftm).mean())
    std = dict(W=W, H=H, means2D=m2, colors=colors, trans_mat=tm, normal_opacity=no, ranges=ranges, point_list=pl,
               near=0.2, far=100.0)
    return s, std, (fm2, fcolors, ftm, fim, fno), ranges, pl, t2, rng


def test_fast_flow_accum_and_snapshots_forward(oracle_mod):
    """Fast-path optical flow (normalised by the final opacity, gs_2d_fast_redner.cu:259-263), the accum_* side outputs
    and the 10-channel snapshots. With matched intrinsics the fast intersection equals the standard one, so the
    independent per-pixel compositor of test_oracle_blend.py (closed forms on the whole list, pair sums, running
    arg-max replay) applies with its flow divided by the opacity instead of the weight sum."""
    from test_oracle_blend import _compose
    O = oracle_mod
    s, std, (fm2, fcolors, ftm, fim, fno), ranges, pl, t2, rng = _flow_case(O)
    W, H, P = s['W'], s['H'], fno.shape[0]
    lens = ranges[:, 1] - ranges[:, 0]
    bucket_offset = np.ascontiguousarray(np.cumsum((lens + 31) // 32).astype(np.int64))
    amc, awp, awc = np.zeros(P, np.int32), np.zeros(P), np.zeros(P, np.int32)
    out = O.fast_render_forward(W, H, 0.2, 100.0, False, fm2, fcolors, fno, ftm, fim, pl, ranges, bucket_offset, t2,
                                amc, awp, awc)
    foc, foo, foe, fnc, max_contrib, b2t, sT, sacc, saux, flow = out
    c = _compose(std, trans_mat_t2=t2, flow_by_opacity=True)
    assert np.abs(flow - c['flow']).max() < 1e-7 * max(1.0, np.abs(c['flow']).max()) and np.abs(c['flow']).max() > 1e-2
    assert (c['opacity'] < 0.7).sum() > 100  # the two normalisations really differ from "no normalisation"
    assert np.abs(foo - c['opacity']).max() < 1e-9 and np.abs(foe[5] - c['distortion']).max() < 1e-9
    assert np.array_equal(awc, c['accum_weights_count']) and np.abs(awp - c['accum_weights_p']).max() < 1e-9
    assert np.array_equal(amc, c['accum_max_count']) and (amc != awc).any()
    assert not flow[foo == 0].any()
    # snapshots: 10 channels with flow; the first 8 are those of a run without flow, channels 8, 9 are the unnormalised
    # flow sums over the list entries before the bucket = (flow * opacity) of a forward over the truncated lists
    assert saux.shape[1] == 10 and (lens > 32).any()
    plain = O.fast_render_forward(W, H, 0.2, 100.0, False, fm2, fcolors, fno, ftm, fim, pl, ranges, bucket_offset)
    assert plain[8].shape[1] == 8 and np.array_equal(plain[8], saux[:, :8]) and np.array_equal(plain[6], sT)
    gx = (W + 15) // 16
    checked = 0
    for t in np.flatnonzero(lens > 32):
        b0 = 0 if t == 0 else int(bucket_offset[t - 1])
        ty, tx = divmod(int(t), gx)
        for k in range(1, int((lens[t] + 31) // 32)):
            cut = ranges.copy()
            cut[:, 1] = cut[:, 0]
            cut[t, 1] = cut[t, 0] + 32 * k
            o = O.fast_render_forward(W, H, 0.2, 100.0, False, fm2, fcolors, fno, ftm, fim, pl, cut, None, t2)
            raw = o[-1] * o[1][..., None]
            for ly in range(min(16, H - ty * 16)):
                for lx in range(min(16, W - tx * 16)):
                    rank = ly * 16 + lx
                    if sT[b0 + k, rank] == 0:  # this pixel had stopped blending before the bucket: nothing written
                        continue
                    assert abs(saux[b0 + k, 8, rank] - raw[ty * 16 + ly, tx * 16 + lx, 0]) < 1e-9
                    assert abs(saux[b0 + k, 9, rank] - raw[ty * 16 + ly, tx * 16 + lx, 1]) < 1e-9
                    checked += 1
    assert checked > 200


def test_fast_flow_backward(oracle_mod):
    """Per-pixel form: dL_dflow is taken as the gradient of the UNNORMALISED flow sum U = flow * opacity
    (gs_2d_fast_redner.cu:366, :494-510), so the check is central differences of sum_pix g . U(theta) from the forward,
    on surfels that never take the low-pass branch for the adjugate (the chain through the intersection is dropped
    there, :524-548) and on all surfels for the opacity.
    Per-splat form (:704-706, :765-782): its accumulator is (partial sum up to this entry) - (the NORMALISED final
    flow); since total - final = -final * T_final, that equals the per-pixel form plus an opacity-map gradient of
    -(final flow . g). The oracle restates the kernel literally (front-to-back partial sums); the identity is checked
    here."""
    from test_oracle_blend import _never_filtered
    O = oracle_mod
    s, std, (fm2, fcolors, ftm, fim, fno), ranges, pl, t2, rng = _flow_case(O, seed=4, scale_mul=40.0, P=30, W=32, H=32)
    W, H = s['W'], s['H']
    g_flow = np.ascontiguousarray(rng.normal(size=(H, W, 2)))
    z3, z1, z8 = np.zeros((3, H, W)), np.zeros((H, W)), np.zeros((8, H, W))

    def fwd(**over):
        t = dict(means2D=fm2, normal_opacity=fno, trans_mat=ftm, inverse_m=fim)
        t.update(over)
        return O.fast_render_forward(W, H, 0.2, 100.0, False, t['means2D'], fcolors, t['normal_opacity'],
                                     t['trans_mat'], t['inverse_m'], pl, ranges, None, t2)

    base = fwd()
    foo, foe, fnc, flow = base[1], base[2], base[3], base[-1]

    def loss(**over):
        o = fwd(**over)
        return (g_flow * (o[-1] * o[1][..., None])).sum()

    gc, gm, gt, gi, gn = O.fast_render_backward(0.2, 100.0, 0, fm2, fno, fcolors, ftm, fim, foo, foe, z3, z1, z8,
                                                ranges, pl, fnc, t2, flow, g_flow)
    assert not gc.any() and np.abs(gi).max() > 1e-3 and np.abs(gn[:, 3]).max() > 1e-3
    used = list(np.unique(pl))
    clean = [i for i in used if _never_filtered(std, i)]
    assert len(clean) >= 4
    eps, l0, checked = 1e-6, loss(), 0
    for name, grad, which in (('normal_opacity', gn, used), ('inverse_m', gi, clean), ('means2D', gm, used)):
        flat = grad.reshape(grad.shape[0], -1)
        src = dict(normal_opacity=fno, inverse_m=fim, means2D=fm2)[name]
        for i in which[:8]:
            for a in ([3] if name == 'normal_opacity' else range(flat.shape[1])):
                p, m = src.copy(), src.copy()
                p.reshape(p.shape[0], -1)[i, a] += eps
                m.reshape(m.shape[0], -1)[i, a] -= eps
                lp, lm = loss(**{name: p}), loss(**{name: m})
                if abs((lp - l0) - (l0 - lm)) > 1e-9 * max(1.0, abs(l0)):
                    continue
                fd = (lp - lm) / (2 * eps)
                assert abs(fd - flat[i, a]) < 1e-5 * max(1.0, abs(fd)), (name, i, a, fd, flat[i, a])
                checked += 1
    assert checked > 60

    # per-splat form = per-pixel flow terms + the other channels of the per-splat form with the opacity-map gradient
    # lowered by (final flow . g)
    g_img, g_opa = rng.normal(size=(3, H, W)), rng.normal(size=(H, W))
    g_ext = np.zeros((8, H, W))
    g_ext[[0, 1, 2, 3, 4, 6, 7]] = rng.normal(size=(7, H, W))
    lit = O.fast_render_backward(0.2, 100.0, 1, fm2, fno, fcolors, ftm, fim, foo, foe, g_img, g_opa, g_ext, ranges, pl,
                                 fnc, t2, flow, g_flow)
    rest = O.fast_render_backward(0.2, 100.0, 1, fm2, fno, fcolors, ftm, fim, foo, foe, g_img,
                                  np.ascontiguousarray(g_opa - (flow * g_flow).sum(-1)), g_ext, ranges, pl, fnc)
    only_flow = (gc, gm, gt, gi, gn)
    for a, b, c_ in zip(lit, rest, only_flow):
        assert np.abs(a - (b + c_)).max() < 1e-9 * max(1.0, np.abs(a).max())
    assert np.abs(lit[4][:, 3] - rest[4][:, 3] - 0).max() > 1e-3  # the flow terms are not negligible
