"""GPU parity of the 3D-Gaussian (EWA) path against the oracle, through the operators: preprocess forward (bit-exact
geometry) / backward, rasterise forward / backward with 0..4 extra channels and the accumulators, and the autograd entry
point `gaussian_render.render` end to end. Tolerances as for the surfel path: images 1e-4 abs, gradients 1e-3 of the
largest entry; contraction is off in the geometry, on in the blend kernels."""
import numpy as np
import pytest
import torch

import oracle as O
from util import abs_err, npy, rel_err

pytestmark = pytest.mark.gpu


def _scene(P, W, H, seed, device):
    from fast_sp_gs_amd import scenes
    scene, _ = scenes.config0(P=P, size=max(W, H), seed=seed)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]))
    g = torch.Generator().manual_seed(seed + 100)
    scales = torch.cat([scene.scales * 3, scene.scales[:, :1] * (0.5 + 3.5 * torch.rand(P, 1, generator=g))], 1).contiguous()
    scene.means3D[::9, 2] += 9.0  # some behind the camera
    tan_fov = (W / 2 / float(cam.Tv2s[0, 0]), H / 2 / float(cam.Tv2s[1, 1]))
    return scene, scales, cam, tan_fov


@pytest.mark.parametrize("name,deg,P,W,H", [("deg3", 3, 5001, 200, 120), ("deg0", 0, 3000, 97, 65),
                                            ("colors", -1, 2000, 64, 64), ("deg4", 4, 1500, 80, 48)])
def test_gs3d_preprocess(name, deg, P, W, H, device):
    from fast_sp_gs_amd._C import get_C_function
    scene, scales, cam, tan_fov = _scene(P, W, H, 21, device)
    g = torch.Generator().manual_seed(5)
    n_rows = {3: 16, 0: 1, 4: 25}.get(deg, 0)
    shs = torch.rand(P, 3, generator=g) if deg < 0 else (torch.randn(P, n_rows, 3, generator=g) * 0.3)
    culling = torch.rand(P, generator=g) < 0.1
    d = lambda t: None if t is None else t.to(device).contiguous()
    print(f"[gs3d preprocess {name}] P={P} {W}x{H}", flush=True)
    out = get_C_function('gs_preprocess_forward')(
        W, H, deg, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, None, None, None, d(culling))
    torch.cuda.synchronize()
    m2, dep, col, rad, tt, c3, co = [npy(t) for t in out]
    ref = O.gs3d_preprocess_forward(W, H, deg, False, npy(scene.means3D), npy(scales), npy(scene.rotations),
                                    npy(scene.opacities), npy(shs), None, npy(cam.Tw2v), npy(cam.Tv2c),
                                    npy(cam.campos), tan_fov, culling=npy(culling))
    r_m2, r_dep, r_col, r_rad, r_tt, r_c3, r_co = ref
    assert 0 < (rad > 0).sum() < P
    assert np.array_equal(rad, r_rad) and np.array_equal(tt, r_tt)
    assert np.array_equal(m2, r_m2) and np.array_equal(dep, r_dep) and np.array_equal(co, r_co)
    assert np.array_equal(c3, r_c3)
    assert abs_err(col, r_col) < 2e-6

    gm2, gcol, gco = torch.randn(P, 2, generator=g), torch.randn(P, 3, generator=g), torch.randn(P, 4, generator=g)
    nan = lambda *shape: torch.full(shape, float('nan'), device=device)
    g3, gs, gq, gop, gcov = nan(P, 3), nan(P, 3), nan(P, 4), nan(P, 1), nan(P, 6)
    gsh = None if deg < 0 else nan(*shs.shape)
    gm2_d = d(gm2)
    get_C_function('gs_preprocess_backward')(
        W, H, deg, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, out[5], None, out[3], out[2], gm2_d, None, d(gcol), d(gco),
        g3, gs, gq, gop, gsh, None, gcov)
    torch.cuda.synchronize()
    r3, rs, rq, rop, rsh, _, rcov, rm2 = O.gs3d_preprocess_backward(
        W, H, deg, False, npy(scene.means3D), npy(scales), npy(scene.rotations), npy(shs), None, npy(cam.Tw2v),
        npy(cam.Tv2c), npy(cam.campos), tan_fov, rad, col, c3, npy(gm2), npy(gcol), npy(gco))
    vis = rad > 0
    pairs = dict(means3D=(g3, r3), scales=(gs, rs), rot=(gq, rq), opac=(gop, rop), cov3D=(gcov, rcov))
    if gsh is not None:
        pairs['shs'] = (gsh, rsh)
    for k, (a, b) in pairs.items():
        a = npy(a)
        assert np.isfinite(a).all(), f"{k}: rows left unwritten"
        assert rel_err(a, b) < 1e-5, (k, rel_err(a, b))
        assert not a[~vis].any(), k
    assert np.array_equal(npy(gm2_d)[vis], rm2[vis]) and np.array_equal(npy(gm2_d)[~vis], npy(gm2)[~vis])


def _binned(P, W, H, seed, device):
    from fast_sp_gs_amd._C import get_C_function
    scene, scales, cam, tan_fov = _scene(P, W, H, seed, device)
    d = lambda t: None if t is None else t.to(device).contiguous()
    out = get_C_function('gs_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, None, None, None, None)
    m2, dep, col, rad, tt, c3, co = out
    ranges, pl, offsets = get_C_function('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True)
    _binned.offsets, _binned.radii = offsets, rad  # for the backward's ordered-sum path
    return m2, col, co, ranges, pl


@pytest.mark.parametrize("P,W,H,E", [(4000, 160, 96, 0), (4000, 131, 77, 2), (20000, 128, 128, 4), (3, 40, 40, 1),
                                     (300_000, 800, 800, 0)])
def test_gs3d_rasterize(P, W, H, E, device):
    from fast_sp_gs_amd._C import get_C_function
    m2, col, co, ranges, pl = _binned(P, W, H, 31 + E, device)
    g = torch.Generator().manual_seed(9)
    ex = torch.randn(P, E, generator=g).to(device) if E else None
    acc_max = torch.zeros(P, dtype=torch.int32, device=device)
    acc_w, acc_n = torch.zeros(P, device=device), torch.zeros(P, dtype=torch.int32, device=device)
    print(f"[gs3d rasterize] P={P} {W}x{H} E={E} R={pl.numel()}", flush=True)
    oc, oo, oe, nc = get_C_function('gaussian_rasterize_forward')(W, H, m2, co, col, ex, pl, ranges, acc_max, acc_w,
                                                                  acc_n)
    torch.cuda.synchronize()
    n = lambda t: None if t is None else npy(t)
    r_max, r_w, r_n = np.zeros(P, np.int32), np.zeros(P, np.float32), np.zeros(P, np.int32)
    r_oc, r_oo, r_oe, r_nc = O.gs3d_render_forward(W, H, n(m2), n(co), n(col), n(ex), n(pl), n(ranges), r_max, r_w, r_n)
    assert abs_err(n(oc), r_oc) < 1e-4 and abs_err(n(oo), r_oo) < 1e-4
    if E:
        assert abs_err(n(oe), r_oe) < 1e-4 * max(1.0, float(np.abs(r_oe).max()))
    flips = int((n(nc) != r_nc).sum())
    assert flips <= max(2, int(1e-4 * W * H)), flips  # pairs within rounding of the 1/255 or 1e-4 thresholds
    assert abs(float(acc_w.sum()) - float(r_w.sum())) < 1e-3 * max(1.0, float(r_w.sum()))
    assert abs(int(acc_n.sum()) - int(r_n.sum())) <= 4 and abs(int(acc_max.sum()) - int(r_max.sum())) <= 2
    # the plain variant (no accumulators) gives the same image
    oc2, oo2, _, nc2 = get_C_function('gaussian_rasterize_forward')(W, H, m2, co, col, ex, pl, ranges)
    assert torch.equal(oc, oc2) and torch.equal(oo, oo2) and torch.equal(nc, nc2)

    gi, go = torch.randn(3, H, W, generator=g).to(device), torch.randn(H, W, generator=g).to(device)
    ge = torch.randn(E, H, W, generator=g).to(device) if E else None
    g_col, g_ex, g_m2, g_co = get_C_function('gaussian_rasterize_backward')(m2, co, col, ex, oo, gi, go, ge, ranges,
                                                                            pl, nc)
    torch.cuda.synchronize()
    # the oracle backward from the GPU's own forward state, so threshold flips of the forward do not enter
    r_col, r_ex, r_m2, r_co = O.gs3d_render_backward(W, H, n(m2), n(co), n(col), n(ex), n(oo), n(nc), n(gi), n(ge),
                                                     n(go), n(pl), n(ranges))
    assert rel_err(n(g_col), r_col) < 1e-3 and rel_err(n(g_m2), r_m2) < 1e-3 and rel_err(n(g_co), r_co) < 1e-3
    if E:
        assert rel_err(n(g_ex), r_ex) < 1e-3
    else:
        assert g_ex is None
    # the same sums through per-(Gaussian, tile) records added in a fixed order: equal to the atomic sums up to the
    # order of the additions, identical from run to run, and every row assigned (the outputs are not zero-filled)
    bwd = lambda: get_C_function('gaussian_rasterize_backward')(m2, co, col, ex, oo, gi, go, ge, ranges, pl, nc,
                                                                _binned.offsets, _binned.radii)
    first, second = bwd(), bwd()
    torch.cuda.synchronize()
    for a, b, c in zip(first, second, (g_col, g_ex, g_m2, g_co)):
        if c is None:
            assert a is None
            continue
        assert torch.equal(a, b) and bool(torch.isfinite(a).all())
        assert float((a - c).abs().max()) <= 2e-5 * max(float(c.abs().max()), 1e-30)
        assert not a[_binned.radii <= 0].any()


@pytest.mark.parametrize("K", [1, 4, 7, 16])
def test_gs3d_topk_weights(K, device):
    from fast_sp_gs_amd._C import get_C_function
    P, W, H = 6000, 150, 90
    m2, col, co, ranges, pl = _binned(P, W, H, 41, device)
    print(f"[gs3d topk] K={K} P={P} {W}x{H} R={pl.numel()}", flush=True)
    ti, tw = get_C_function('gaussian_topk_weights')(K, W, H, P, pl.numel(), m2, co, ranges, pl)
    torch.cuda.synchronize()
    r_ti, r_tw = O.gs3d_topk_weights(K, W, H, npy(m2), npy(co), npy(ranges), npy(pl))
    assert abs_err(npy(tw), r_tw) < 1e-5
    # the same Gaussians in the same slots, except where two weights are equal to rounding or a pair sits on a threshold
    differ = (npy(ti) != r_ti).any(-1)
    assert int(differ.sum()) <= max(2, int(2e-3 * W * H)), int(differ.sum())
    assert (np.diff(npy(tw), axis=-1) <= 0).all() and ((npy(ti) == -1) == (npy(tw) == 0)).all()
    with pytest.raises(RuntimeError):
        get_C_function('gaussian_topk_weights')(17, W, H, P, pl.numel(), m2, co, ranges, pl)


def test_gs3d_render_autograd_and_empty(device):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.renderer import gaussian_render as GR
    P, W, H = 3000, 112, 80
    scene, scales, cam, tan_fov = _scene(P, W, H, 41, device)
    d = lambda t: t.to(device).contiguous()
    params = [d(t).requires_grad_(True) for t in (scene.means3D, scales, scene.rotations, scene.opacities, scene.shs)]
    feat = d(torch.randn(P, 2, generator=torch.Generator().manual_seed(2))).requires_grad_(True)
    focals = torch.tensor([float(cam.Tv2s[0, 0]), float(cam.Tv2s[1, 1])], device=device)
    out = GR.render(d(cam.Tw2v), d(cam.Tv2c), (W, H), params[0], params[3], scales=params[1], rotations=params[2],
                    campos=d(cam.campos), focals=focals, sh_features=params[4], sh_degree=3, feat=feat)
    assert set(out) >= {'images', 'opacity', 'viewspace_points', 'visibility_filter', 'radii', 'buffer', 'feat'}
    g = torch.Generator().manual_seed(3)
    gi, go, gf = (torch.randn(*out[k].shape, generator=g).to(device) for k in ('images', 'opacity', 'feat'))
    ((out['images'] * gi).sum() + (out['opacity'] * go).sum() + (out['feat'] * gf).sum()).backward()
    torch.cuda.synchronize()
    # the same chain on the oracle
    n = lambda t: npy(t.detach())
    m2, dep, col, rad, tt, c3, co = O.gs3d_preprocess_forward(W, H, 3, False, n(params[0]), n(params[1]), n(params[2]),
                                                              n(params[3]), n(params[4]), None, npy(cam.Tw2v),
                                                              npy(cam.Tv2c), npy(cam.campos), tan_fov)
    ranges, pl = O.prepare(W, H, m2, dep, rad, tt)
    oc, oo, oe, nc = O.gs3d_render_forward(W, H, m2, co, col, n(feat), pl, ranges)
    assert abs_err(n(out['images']), oc) < 1e-4 and abs_err(n(out['feat']), oe) < 1e-4 * max(1, np.abs(oe).max())
    assert np.array_equal(n(out['radii']), rad)
    g_col, g_ex, g_m2, g_co = O.gs3d_render_backward(W, H, m2, co, col, n(feat), oo, nc, npy(gi), npy(gf), npy(go), pl,
                                                     ranges)
    r3, rs, rq, rop, rsh, _, _, rm2 = O.gs3d_preprocess_backward(W, H, 3, False, n(params[0]), n(params[1]),
                                                                 n(params[2]), n(params[4]), None, npy(cam.Tw2v),
                                                                 npy(cam.Tv2c), npy(cam.campos), tan_fov, rad, col, c3,
                                                                 g_m2, g_col, g_co)
    for name, p_, r in zip(('means3D', 'scales', 'rotations', 'opacities', 'shs'), params, (r3, rs, rq, rop, rsh)):
        assert rel_err(n(p_.grad), r) < 1e-3, (name, rel_err(n(p_.grad), r))
    assert rel_err(n(feat.grad), g_ex) < 1e-3
    assert rel_err(n(out['viewspace_points'].grad), rm2) < 1e-3  # what densification reads
    # the same pass with the blend backward's sums taken in a fixed order (module switch): same gradients up to the
    # order of the additions, and identical when repeated
    atomic = [p_.grad.clone() for p_ in params] + [feat.grad.clone()]
    runs = []
    GR.DETERMINISTIC_SUMS = True
    try:
        for _ in range(2):
            for p_ in params + [feat]:
                p_.grad = None
            o2 = GR.render(d(cam.Tw2v), d(cam.Tv2c), (W, H), params[0], params[3], scales=params[1], rotations=params[2],
                           campos=d(cam.campos), focals=focals, sh_features=params[4], sh_degree=3, feat=feat)
            ((o2['images'] * gi).sum() + (o2['opacity'] * go).sum() + (o2['feat'] * gf).sum()).backward()
            runs.append([p_.grad.clone() for p_ in params] + [feat.grad.clone()])
    finally:
        GR.DETERMINISTIC_SUMS = False
    for a, b, c in zip(runs[0], runs[1], atomic):
        assert torch.equal(a, b) and float((a - c).abs().max()) <= 2e-5 * float(c.abs().max())
    # empty scene
    z = lambda *s: torch.zeros(s, device=device)
    out = GR.render(d(cam.Tw2v), d(cam.Tv2c), (W, H), z(0, 3), z(0, 1), scales=z(0, 3), rotations=z(0, 4),
                    campos=d(cam.campos), focals=focals, sh_features=z(0, 16, 3), sh_degree=3)
    assert out['images'].shape == (3, H, W) and not out['images'].any() and not out['opacity'].any()


@pytest.mark.parametrize("P,W,H,E", [(6000, 150, 90, 16), (4000, 131, 77, 5), (20000, 128, 128, 37), (3, 40, 40, 1)])
def test_gs3d_rasterize_extra(P, W, H, E, device):
    """gaussian_rasterize_extra_forward / backward: any number of channels on the weights of a finished forward pass;
    the oracle runs from the GPU's own n_contrib / opacity, so threshold flips of the main pass do not enter."""
    from fast_sp_gs_amd._C import get_C_function
    m2, col, co, ranges, pl = _binned(P, W, H, 51 + E, device)
    g = torch.Generator().manual_seed(10)
    ex = torch.randn(P, E, generator=g).to(device)
    print(f"[gs3d extra] P={P} {W}x{H} E={E} R={pl.numel()}", flush=True)
    oc, oo, _, nc = get_C_function('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges)
    out = get_C_function('gaussian_rasterize_extra_forward')(W, H, ex, m2, co, ranges, pl, nc)
    torch.cuda.synchronize()
    n = npy
    r_out = O.gs3d_extra_forward(W, H, n(ex), n(m2), n(co), n(ranges), n(pl), n(nc))
    assert out.shape == (H, W, E) and abs_err(n(out), r_out) < 1e-4 * max(1.0, float(np.abs(r_out).max()))
    # a shortened n_contrib cuts every pixel's traversal at that list position
    cut = (nc // 2).contiguous()
    out_cut = get_C_function('gaussian_rasterize_extra_forward')(W, H, ex, m2, co, ranges, pl, cut)
    r_cut = O.gs3d_extra_forward(W, H, n(ex), n(m2), n(co), n(ranges), n(pl), n(cut))
    assert abs_err(n(out_cut), r_cut) < 1e-4 * max(1.0, float(np.abs(r_cut).max()))

    go = torch.randn(H, W, E, generator=g).to(device)
    bwd = get_C_function('gaussian_rasterize_extra_backward')
    ge, gm, gc = torch.zeros_like(ex), torch.zeros_like(m2), torch.zeros_like(co)
    bwd(W, H, ex, oo, go, m2, co, ranges, pl, nc, ge, gm, gc)
    torch.cuda.synchronize()
    r_ge, r_gm, r_gc = O.gs3d_extra_backward(W, H, n(ex), n(oo), n(go), n(m2), n(co), n(ranges), n(pl), n(nc))
    assert rel_err(n(ge), r_ge) < 1e-3 and rel_err(n(gm), r_gm) < 1e-3 and rel_err(n(gc), r_gc) < 1e-3
    # optional outputs: only what is given is touched, and it is added to
    ge2 = torch.ones_like(ex)
    bwd(W, H, ex, oo, go, m2, co, ranges, pl, nc, ge2, None, None)
    assert rel_err(n(ge2) - 1.0, r_ge) < 1e-3
    gm2, gc2 = torch.zeros_like(m2), torch.zeros_like(co)
    get_C_function('gaussian_rasterize_extra_backward_v2')(W, H, ex, oo, go, m2, co, ranges, pl, nc,
                                                           torch.zeros_like(ex), gm2, gc2)
    assert rel_err(n(gm2), r_gm) < 1e-3 and rel_err(n(gc2), r_gc) < 1e-3
    bwd(W, H, ex, oo, go, m2, co, ranges, pl, nc, None, None, None)
    with pytest.raises(RuntimeError):
        get_C_function('gaussian_rasterize_extra_backward_v2')(W, H, ex, oo, go, m2, co, ranges, pl, nc, ge, None, gc)
    with pytest.raises(RuntimeError):
        get_C_function('gaussian_rasterize_extra_forward')(W, H, ex[None], m2, co, ranges, pl, nc)


def test_gs3d_render_extra_autograd(device):
    """`render(..., wide=[P,E > 4])` and `render_extra(buffer, ...)`: the autograd wiring of the further feature tables,
    against the oracle chain; with detach=True the geometry gets no gradient from them."""
    from fast_sp_gs_amd.renderer import gaussian_render as GR
    P, W, H, E = 3000, 112, 80, 12
    scene, scales, cam, tan_fov = _scene(P, W, H, 43, device)
    d = lambda t: t.to(device).contiguous()
    params = [d(t).requires_grad_(True) for t in (scene.means3D, scales, scene.rotations, scene.opacities, scene.shs)]
    gen = torch.Generator().manual_seed(5)
    wide = d(torch.randn(P, E, generator=gen)).requires_grad_(True)
    focals = torch.tensor([float(cam.Tv2s[0, 0]), float(cam.Tv2s[1, 1])], device=device)
    out = GR.render(d(cam.Tw2v), d(cam.Tv2c), (W, H), params[0], params[3], scales=params[1], rotations=params[2],
                    campos=d(cam.campos), focals=focals, sh_features=params[4], sh_degree=3, wide=wide)
    assert out['wide'].shape == (H, W, E)
    gw = torch.randn(H, W, E, generator=gen).to(device)
    (out['wide'] * gw).sum().backward()
    torch.cuda.synchronize()
    n = lambda t: npy(t.detach())
    m2, dep, col, rad, tt, c3, co = O.gs3d_preprocess_forward(W, H, 3, False, n(params[0]), n(params[1]), n(params[2]),
                                                              n(params[3]), n(params[4]), None, npy(cam.Tw2v),
                                                              npy(cam.Tv2c), npy(cam.campos), tan_fov)
    ranges, pl = O.prepare(W, H, m2, dep, rad, tt)
    oc, oo, _, nc = O.gs3d_render_forward(W, H, m2, co, col, None, pl, ranges)
    r_out = O.gs3d_extra_forward(W, H, n(wide), m2, co, ranges, pl, nc)
    assert abs_err(n(out['wide']), r_out) < 1e-4 * max(1.0, float(np.abs(r_out).max()))
    r_ge, r_gm, r_gc = O.gs3d_extra_backward(W, H, n(wide), oo, npy(gw), m2, co, ranges, pl, nc)
    z3 = np.zeros((P, 3), np.float32)
    r3, rs, rq, rop, rsh, _, _, rm2 = O.gs3d_preprocess_backward(W, H, 3, False, n(params[0]), n(params[1]),
                                                                 n(params[2]), n(params[4]), None, npy(cam.Tw2v),
                                                                 npy(cam.Tv2c), npy(cam.campos), tan_fov, rad, col, c3,
                                                                 r_gm, z3, r_gc)
    assert rel_err(n(wide.grad), r_ge) < 1e-3
    for name, p_, r in zip(('means3D', 'scales', 'rotations', 'opacities'), params, (r3, rs, rq, rop)):
        assert rel_err(n(p_.grad), r) < 1e-3, (name, rel_err(n(p_.grad), r))
    # render_extra on the buffer, detached from the geometry
    for p_ in params:
        p_.grad = None
    wide.grad = None
    out2 = GR.render(d(cam.Tw2v), d(cam.Tv2c), (W, H), params[0], params[3], scales=params[1], rotations=params[2],
                     campos=d(cam.campos), focals=focals, sh_features=params[4], sh_degree=3)
    a, b = GR.render_extra(out2['buffer'], wide, wide[:, :3] * 2.0, detach=True)
    assert torch.equal(a, out['wide']) and b.shape == (H, W, 3)
    assert abs_err(n(b), 2.0 * r_out[..., :3]) < 2e-4 * max(1.0, float(np.abs(r_out).max()))
    ((a * gw).sum() + b.sum()).backward()
    assert all(p_.grad is None or not p_.grad.any() for p_ in params[:4])
    assert rel_err(n(wide.grad)[:, 3:], r_ge[:, 3:]) < 1e-3 and wide.grad[:, :3].ne(0).any()


def test_covariance_operators(device):
    """gs_compute_cov3D_* / gs_compute_cov2D_* against the oracle (geometry evaluated with contraction off: forward
    values bit for bit, gradients to 1e-5 of the largest entry), and the autograd wrappers end to end."""
    from fast_sp_gs_amd._C import get_C_function as f
    from fast_sp_gs_amd.renderer.gaussian_render import compute_cov2D, compute_cov3D
    g = torch.Generator().manual_seed(4)
    N = 70001
    q = torch.randn(N, 4, generator=g)
    s = torch.rand(N, 3, generator=g) * 0.3 + 0.01
    gc = torch.randn(N, 6, generator=g)
    print(f"[gs3d covariance operators] N={N}", flush=True)
    d = lambda t: t.to(device).contiguous()
    cov3D = f('gs_compute_cov3D_forward')(d(q), d(s))
    want = O.gs3d_compute_cov3D(npy(q), npy(s))
    assert np.array_equal(npy(cov3D), want)
    dq, ds = f('gs_compute_cov3D_backward')(d(q), d(s), d(gc))
    wq, ws = O.gs3d_compute_cov3D_backward(npy(q), npy(s), npy(gc))
    assert rel_err(npy(dq), wq) < 1e-5 and rel_err(npy(ds), ws) < 1e-5

    Tw2v = torch.eye(4)
    Tw2v[:3, :3] = torch.tensor([[0.92, 0.0, 0.39], [0.1, 0.99, -0.05], [-0.39, 0.05, 0.92]])
    Tw2v[:3, 3] = torch.tensor([0.2, -0.1, 4.0])
    means = torch.randn(N, 3, generator=g) * torch.tensor([2.0, 2.0, 0.5])
    fx, fy, tx, ty = 500.0, 480.0, 0.4, 0.35
    g2 = torch.randn(N, 3, generator=g)
    cov2D = f('gs_compute_cov2D_forward')(cov3D, d(means), d(Tw2v), fx, fy, tx, ty)
    want2 = O.gs3d_compute_cov2D(want, npy(means), npy(Tw2v), fx, fy, tx, ty)
    assert np.array_equal(npy(cov2D), want2)
    g_cov3D, g_mean = f('gs_compute_cov2D_backward')(cov3D, d(means), d(Tw2v), fx, fy, tx, ty, d(g2))
    w3, wm = O.gs3d_compute_cov2D_backward(want, npy(means), npy(Tw2v), fx, fy, tx, ty, npy(g2))
    assert rel_err(npy(g_cov3D), w3) < 1e-5 and rel_err(npy(g_mean), wm) < 1e-5
    with pytest.raises(RuntimeError):  # a view-matrix gradient buffer of the wrong size
        f('gs_compute_cov2D_backward')(cov3D, d(means), d(Tw2v), fx, fy, tx, ty, d(g2), torch.zeros(3, 3, device=device))

    # autograd wrappers: scaling / rotation / means receive the chained gradients
    sa, qa, ma = d(s).requires_grad_(True), d(q).requires_grad_(True), d(means).requires_grad_(True)
    out = compute_cov2D(ma, compute_cov3D(sa, qa), d(Tw2v), fx, fy, tx, ty)
    out.backward(d(g2))
    c3g, wm2 = O.gs3d_compute_cov2D_backward(want, npy(means), npy(Tw2v), fx, fy, tx, ty, npy(g2))
    wq2, ws2 = O.gs3d_compute_cov3D_backward(npy(q), npy(s), c3g)
    assert rel_err(npy(ma.grad), wm2) < 1e-5 and rel_err(npy(qa.grad), wq2) < 1e-4 and rel_err(npy(sa.grad), ws2) < 1e-4


def test_gs3d_precomputed_covariances_and_camera_gradients(device):
    """gs_preprocess_forward / _backward with cov3D_precomp and cov2D_precomp (gaussian_preprocess.cu:76-92, :293-301),
    and the gradients of the view matrix and the camera position (:271, :318-355), against the oracle; the autograd
    entry `preprocess` hands the gradients to the right inputs."""
    from fast_sp_gs_amd._C import get_C_function
    from fast_sp_gs_amd.renderer.gaussian_render import compute_cov2D, compute_cov3D, preprocess
    P, W, H = 4000, 160, 96
    scene, scales, cam, tan_fov = _scene(P, W, H, 23, device)
    d = lambda t: None if t is None else t.to(device).contiguous()
    fwd = get_C_function('gs_preprocess_forward')
    bwd = get_C_function('gs_preprocess_backward')
    base_args = (W, H, 3, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs),
                 None, d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov)
    base = fwd(*base_args, None, None, None, None)
    fx, fy = 0.5 * W / tan_fov[0], 0.5 * H / tan_fov[1]
    cov3 = get_C_function('gs_compute_cov3D_forward')(d(scene.rotations), d(scales))
    cov2 = get_C_function('gs_compute_cov2D_forward')(cov3, d(scene.means3D), d(cam.Tw2v), fx, fy, *tan_fov)
    o3 = fwd(*base_args, cov3, None, None, None)
    o2 = fwd(*base_args, None, cov2, None, None)
    torch.cuda.synchronize()
    assert o3[5].data_ptr() == cov3.data_ptr()  # the pre-computed tensor is handed back
    n = lambda t: None if t is None else npy(t)
    host = (W, H, 3, False, n(scene.means3D), n(scales), n(scene.rotations), n(scene.opacities), n(scene.shs), None,
            n(cam.Tw2v), n(cam.Tv2c), n(cam.campos), tan_fov)
    r3 = O.gs3d_preprocess_forward(*host, cov3D_precomp=n(cov3))
    r2 = O.gs3d_preprocess_forward(*host, cov2D_precomp=n(cov2))
    for got, ref, name in ((o3, r3, 'cov3D'), (o2, r2, 'cov2D')):
        for k in (0, 1, 3, 4, 6):
            assert np.array_equal(n(got[k]), ref[k]), (name, k)
        assert abs_err(n(got[2]), ref[2]) < 2e-6
        assert np.array_equal(n(got[3]), n(base[3]))  # same radii as from scales + rotations
    assert not n(o2[5]).any()  # no 3D covariance is formed from a 2D one

    # backward: the three covariance sources, camera gradients on the ordinary one
    g = torch.Generator().manual_seed(7)
    gm2, gcol, gco = torch.randn(P, 2, generator=g), torch.randn(P, 3, generator=g), torch.randn(P, 4, generator=g)
    nan = lambda *shape: torch.full(shape, float('nan'), device=device)
    rad, col = base[3], base[2]
    bargs = (W, H, 3, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
             d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov)
    rargs = (W, H, 3, False, n(scene.means3D), n(scales), n(scene.rotations), n(scene.shs), None, n(cam.Tw2v),
             n(cam.Tv2c), n(cam.campos), tan_fov, n(rad), n(col))
    vis = n(rad) > 0
    # (a) cov2D given: [P,3] gradient
    g3, gop, gsh, gcov = nan(P, 3), nan(P, 1), nan(P, 16, 3), nan(P, 3)
    bwd(*bargs, None, cov2, rad, col, d(gm2), None, d(gcol), d(gco), g3, None, None, gop, gsh, None, gcov)
    ref = O.gs3d_preprocess_backward(*rargs, n(base[5]), n(gm2), n(gcol), n(gco), cov2D=n(cov2))
    torch.cuda.synchronize()
    for a, b, name in ((g3, ref[0], 'means3D'), (gcov, ref[6], 'cov2D'), (gsh, ref[4], 'shs')):
        assert np.isfinite(n(a)).all() and rel_err(n(a), b) < 1e-5 and not n(a)[~vis].any(), name
    with pytest.raises(RuntimeError):
        bwd(*bargs, None, cov2, rad, col, d(gm2), None, d(gcol), d(gco), g3, nan(P, 3), None, gop, gsh, None, gcov)
    # (b) cov3D given: [P,6] gradient, no scale / rotation outputs
    g3b, gcov6 = nan(P, 3), nan(P, 6)
    bwd(*bargs, cov3, None, rad, col, d(gm2), None, d(gcol), d(gco), g3b, None, None, gop, gsh, None, gcov6)
    ref = O.gs3d_preprocess_backward(*rargs, n(cov3), n(gm2), n(gcol), n(gco), precomputed=True)
    torch.cuda.synchronize()
    assert rel_err(n(g3b), ref[0]) < 1e-5 and rel_err(n(gcov6), ref[6]) < 1e-5
    # (c) camera gradients: added to the caller's buffers (start at 1 to show it)
    g_vm, g_cam = torch.ones(4, 4, device=device), torch.ones(3, device=device)
    g3c, gs, gq = nan(P, 3), nan(P, 3), nan(P, 4)
    bwd(*bargs, base[5], None, rad, col, d(gm2), None, d(gcol), d(gco), g3c, gs, gq, gop, gsh, None, None, g_vm, g_cam)
    ref = O.gs3d_preprocess_backward(*rargs, n(base[5]), n(gm2), n(gcol), n(gco), camera=True)
    torch.cuda.synchronize()
    r_vm, r_cam = ref[-2].astype(np.float64), ref[-1].astype(np.float64)
    # sums over ~3000 points in float32, in a different order on each side
    assert rel_err(n(g_vm) - 1.0, r_vm) < 1e-3 and np.all(n(g_vm)[3] == 1.0)
    assert rel_err(n(g_cam) - 1.0, r_cam) < 1e-3 and np.abs(r_cam).max() > 0
    assert rel_err(n(g3c), ref[0]) < 1e-5 and rel_err(n(gs), ref[1]) < 1e-5 and rel_err(n(gq), ref[2]) < 1e-5

    # the stand-alone cov2D backward with the view-matrix gradient
    g2 = torch.randn(P, 3, generator=g).to(device)
    gvm = torch.zeros(4, 4, device=device)
    gc3, gmean = get_C_function('gs_compute_cov2D_backward')(cov3, d(scene.means3D), d(cam.Tw2v), fx, fy, *tan_fov, g2,
                                                             gvm)
    torch.cuda.synchronize()
    r_gvm = np.zeros((4, 4), np.float32)
    r_gc3, r_gmean = O.gs3d_compute_cov2D_backward(n(cov3), n(scene.means3D), n(cam.Tw2v), fx, fy, *tan_fov, n(g2), r_gvm)
    assert rel_err(n(gc3), r_gc3) < 1e-5 and rel_err(n(gmean), r_gmean) < 1e-5 and rel_err(n(gvm), r_gvm) < 1e-3

    # autograd: the view matrix and the camera position as leaves; pre-computed covariances as leaves
    Tw2v = d(cam.Tw2v).requires_grad_()
    campos = d(cam.campos).requires_grad_()
    means = d(scene.means3D).requires_grad_()
    tan_t = torch.tensor(tan_fov)
    out = preprocess(means, d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None, Tw2v, d(cam.Tv2c),
                     campos, tan_t, W, H, 3, False)
    ((out[0] * d(gm2)).sum() + (out[2] * d(gcol)).sum() + (out[5] * d(gco)).sum()).backward()
    assert rel_err(n(Tw2v.grad), r_vm) < 1e-3 and rel_err(n(campos.grad), r_cam) < 1e-3
    assert rel_err(n(means.grad), ref[0]) < 1e-5
    c2 = cov2.clone().requires_grad_()
    out = preprocess(d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
                     d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_t, W, H, 3, False, None, c2)
    (out[5] * d(gco)).sum().backward()
    assert rel_err(n(c2.grad), n(gcov)) < 1e-6
    # cov3D built by the differentiable operator: scales / rotations get their gradient through it
    sc, rot = d(scales).requires_grad_(), d(scene.rotations).requires_grad_()
    out = preprocess(d(scene.means3D), sc, rot, d(scene.opacities), d(scene.shs), None, d(cam.Tw2v), d(cam.Tv2c),
                     d(cam.campos), tan_t, W, H, 3, False, compute_cov3D(sc, rot))
    ((out[0] * d(gm2)).sum() + (out[2] * d(gcol)).sum() + (out[5] * d(gco)).sum()).backward()
    assert rel_err(n(sc.grad), n(gs)) < 1e-5 and rel_err(n(rot.grad), n(gq)) < 1e-5
    assert compute_cov2D is not None


@pytest.mark.parametrize("P,W,H,E,mul", [(6000, 128, 96, 0, 2.5), (6000, 131, 77, 2, 2.5), (3, 40, 40, 1, 1.0)])
def test_gs3d_bucket_snapshots_and_fast_backward(P, W, H, E, mul, device):
    """gaussian_rasterize_forward with per_tile_bucket_offset (snapshots before every 32nd list entry) and
    gaussian_rasterize_fast_backward against the oracle's bucket-by-bucket restatement of the reference's per-Gaussian
    kernel (gaussian_render.cu:540-694); `GS_render_fast` end to end equals `GS_render`."""
    from fast_sp_gs_amd._C import get_C_function
    from fast_sp_gs_amd.renderer.gaussian_render import GS_render, GS_render_fast
    scene, scales, cam, tan_fov = _scene(P, W, H, 41 + E, device)
    d = lambda t: None if t is None else t.to(device).contiguous()
    out = get_C_function('gs_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scales * mul), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, None, None, None, None)
    m2, dep, col, rad, tt, c3, co = out
    ranges, pl = get_C_function('GS_prepare')(W, H, m2, dep, rad, tt, False)
    g = torch.Generator().manual_seed(9)
    ex = torch.randn(P, E, generator=g).to(device) if E else None
    lens = ranges[:, 1] - ranges[:, 0]
    offset = torch.cumsum((lens + 31) // 32, 0).contiguous()
    print(f"[gs3d snapshots] P={P} {W}x{H} E={E} R={pl.numel()} longest list {int(lens.max())}", flush=True)
    res = get_C_function('gaussian_rasterize_forward')(W, H, m2, co, col, ex, pl, ranges, None, None, None, offset)
    oc, oo, oe, nc, max_c, b2t, sT, sar = res
    plain = get_C_function('gaussian_rasterize_forward')(W, H, m2, co, col, ex, pl, ranges)
    torch.cuda.synchronize()
    assert torch.equal(oc, plain[0]) and torch.equal(nc, plain[3])
    n = lambda t: None if t is None else npy(t)
    n64 = lambda t: None if t is None else f64(npy(t))
    from util import f64
    ref = O.gs3d_render_forward(W, H, n64(m2), n64(co), n64(col), n64(ex), n(pl), n(ranges), bucket_offset=n(offset))
    r_oc, r_oo, r_oe, r_nc, r_max, r_b2t, r_sT, r_sar = ref
    flip = n(nc) != r_nc
    assert flip.sum() <= max(2, int(1e-5 * W * H))
    assert np.array_equal(n(b2t), r_b2t) and (n(max_c).reshape(-1) != r_max).sum() <= flip.sum()
    wrote = r_sT > 0
    tol = lambda a, b: np.abs(a.astype(np.float64) - b) > 1e-4 + 1e-3 * np.abs(b)
    bad = int((tol(n(sT), r_sT) & wrote).sum()) + sum(int((tol(n(sar)[:, c], r_sar[:, c]) & wrote).sum())
                                                      for c in range(3 + E))
    assert bad <= 32 * (4 + E) * int(flip.sum()) and (P < 10 or (lens > 40).any())

    gi, go = torch.randn(3, H, W, generator=g).to(device), torch.randn(H, W, generator=g).to(device)
    ge = torch.randn(E, H, W, generator=g).to(device) if E else None
    got = get_C_function('gaussian_rasterize_fast_backward')(m2, co, col, ex, oc, oe, oo, gi, go, ge, ranges, pl, nc,
                                                             max_c, offset, b2t, sT, sar)
    torch.cuda.synchronize()
    # the oracle's per-Gaussian form from the GPU's own forward outputs and snapshots
    want = O.gs3d_render_fast_backward(W, H, n64(m2), n64(co), n64(col), n64(ex), n64(oc), n64(oe), n64(oo), n(nc),
                                       n(max_c).reshape(-1), n(offset), n(b2t), n64(sT), n64(sar), n64(gi), n64(ge),
                                       n64(go), n(pl), n(ranges))
    for a, b, name in zip(got, want, ('colors', 'extras', 'means2D', 'conic_opacity')):
        assert (a is None) == (b is None), name
        if a is not None:
            assert rel_err(n(a), b) < 1e-3, (name, rel_err(n(a), b))
    # the reference's decomposition itself (one lane per list entry, pixels passed from lane to lane, started from the
    # snapshots): against the same oracle, with atomic sums and with ordered records (which must not depend on what
    # the workspace held, and must leave no row of the outputs unwritten)
    _, _, offsets = get_C_function('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True)
    fb = get_C_function('gaussian_rasterize_fast_backward')
    per_g = fb(m2, co, col, ex, oc, oe, oo, gi, go, ge, ranges, pl, nc, max_c, offset, b2t, sT, sar, per_gaussian=True)
    # the operator takes its record workspace from torch's caching allocator: leave a poisoned block of that size there
    from fast_sp_gs_amd import lib as L
    poison = torch.full((L.load().fsgs_gaussian_rasterize_backward_workspace_bytes(pl.numel()) // 4,), float('nan'),
                        device=device)
    del poison
    per_g_ordered = fb(m2, co, col, ex, oc, oe, oo, gi, go, ge, ranges, pl, nc, max_c, offset, b2t, sT, sar, offsets,
                       rad, per_gaussian=True)
    torch.cuda.synchronize()
    for a, o, b, name in zip(per_g, per_g_ordered, want, ('colors', 'extras', 'means2D', 'conic_opacity')):
        assert (a is None) == (b is None) == (o is None), name
        if a is not None:
            assert rel_err(n(a), b) < 1e-3, (name, rel_err(n(a), b))
            assert np.isfinite(n(o)).all() and rel_err(n(o), b) < 1e-3, (name, rel_err(n(o), b))
    # end to end: the bucketed pair gives GS_render's gradients
    leaves = [t.clone().requires_grad_() for t in (m2, col, co)]
    leaves2 = [t.clone().requires_grad_() for t in (m2, col, co)]
    a = GS_render_fast(W, H, leaves[0], leaves[1], leaves[2], ranges, pl, ex)
    b = GS_render(W, H, leaves2[0], leaves2[1], leaves2[2], ranges, pl, ex)
    ((a[0] * gi).sum() + (a[1] * go).sum()).backward()
    ((b[0] * gi).sum() + (b[1] * go).sum()).backward()
    for x, y in zip(leaves, leaves2):
        assert rel_err(n(x.grad), n(y.grad)) < 1e-4
