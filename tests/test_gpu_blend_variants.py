"""GPU parity of every variant of the standard blend against the CPU oracle (gs_2d_redner.cu:141-150, 180-197, 230-233,
326-332, 480-510): optical flow through a second set of transform matrices (forward, and backward with the per-surfel
sums taken in a fixed order and with atomics), the accum_max_count / accum_weights_p / accum_weights_count side
outputs element by element, the image-only variant forward and backward, and the blend's own dL/dmeans2D.

The checker is the oracle evaluated in float64 on the GPU's own float32 inputs, i.e. the exact value of the reference's
formulas: images and maps within 1e-4 abs (+1e-3 rel for unnormalised maps such as depth or flow in pixels),
gradients within 1e-3 rel (max|d| / max|ref|), integer outputs exact. A (pixel, surfel) pair whose alpha sits within
float32 rounding of a threshold (1/255, T < 1e-4) can fall on the other side in float32; such pixels are counted
(n_contrib differs) and at most max(2, 1e-5 HW) of them are allowed. (The oracle run in float32 WITHOUT fused
multiply-adds is the less accurate of the two float32 evaluations: on grazing surfels it misses the float64 value by
up to 2e-3 rel where the kernels, which use fused multiply-adds, stay within 1e-5.)
"""
import numpy as np
import pytest
import torch

from util import abs_err, f64, npy, rel_err

pytestmark = pytest.mark.gpu

CASES = {"c0_10k_256": (10_000, 256, 256), "partial_tiles_511x127": (4_000, 511, 127)}


def _stage(name, device):
    """Preprocess + binning on the GPU -> device tensors the blend operators take, and numpy copies for the oracle."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    P, W, H = CASES[name]
    scene, cam = scenes.config0(P=P, size=max(W, H), seed=0)
    if (W, H) != (cam.W, cam.H):
        cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    sc, cm = scene.to(device), cam.to(device)
    m2, colors, tm, no, depths, radii, tt = f('gs_2d_preprocess_forward')(
        W, H, 3, False, sc.means3D, sc.scales, sc.rotations, sc.opacities, sc.shs, None, cm.Tw2v, cm.Tv2c, cm.campos,
        None, None, None)
    ranges, point_list, offsets = f('GS_prepare')(W, H, m2, depths, radii, tt, False, return_offsets=True)
    # second time step: the same surfels with shifted centres and slightly different tangent scales
    g = torch.Generator().manual_seed(17)
    means_t2 = (scene.means3D + 0.03 * torch.randn(P, 3, generator=g)).to(device)
    scales_t2 = (scene.scales * torch.exp(0.05 * torch.randn(P, 2, generator=g))).to(device)
    Tw2c = (cm.Tv2c @ cm.Tw2v).contiguous()
    t2, _ = f('gs_2d_compute_transmat_forward')(W, H, means_t2, scales_t2, sc.rotations, cm.Tw2v, Tw2c)
    same, _ = f('gs_2d_compute_transmat_forward')(W, H, sc.means3D, sc.scales, sc.rotations, cm.Tw2v, Tw2c)
    vis = radii > 0
    assert rel_err(npy(same[vis]), npy(tm[vis])) < 1e-5  # the stand-alone operator gives the preprocess' matrices
    d = dict(W=W, H=H, P=P, near=cam.near, far=cam.far, means2D=m2, colors=colors, trans_mat=tm, normal_opacity=no,
             radii=radii, ranges=ranges, point_list=point_list, offsets=offsets, t2=t2)
    g2 = torch.Generator().manual_seed(5)
    d['grad_image'] = torch.randn(3, H, W, generator=g2).to(device)
    d['grad_extras'] = torch.cat([torch.randn(6, H, W, generator=g2), torch.zeros(3, H, W)]).to(device)
    d['grad_opacity'] = torch.randn(H, W, generator=g2).to(device)
    d['grad_flow'] = torch.randn(H, W, 2, generator=g2).to(device)
    return d


def _n(d, *keys):
    """numpy copies for the oracle: float tensors as float64 (same values), integer tensors unchanged."""
    return [f64(npy(d[k])) for k in keys]


def _flip_pixels(gpu_nc, ref_nc):
    return (gpu_nc != ref_nc).any(0)


def _allowed(d):
    return max(2, int(1e-5 * d['H'] * d['W']))


@pytest.mark.parametrize("name", list(CASES))
def test_flow_forward_and_backward(name, device, oracle_mod):
    """trans_mat_t2 -> out_flow (normalised by the sum of weights) and the gradients of all four per-surfel inputs with
    dL/dflow, once with the ordered per-instance sums (point_offsets given) and once with atomics (None)."""
    from fast_sp_gs_amd._C import get_C_function as f
    O = oracle_mod
    d = _stage(name, device)
    W, H = d['W'], d['H']
    oc, oo, oe, of, nc = f('GS_2D_render_forward')(W, H, d['means2D'], d['colors'], d['normal_opacity'],
                                                   d['trans_mat'], d['point_list'], d['ranges'], d['near'], d['far'],
                                                   False, d['t2'], None, None, None)
    torch.cuda.synchronize()
    m2, colors, no, tm, pl, ranges, t2 = _n(d, 'means2D', 'colors', 'normal_opacity', 'trans_mat', 'point_list',
                                            'ranges', 't2')
    rc_, ro, re_, rf, rnc = O.render_forward(W, H, m2, colors, no, tm, pl, ranges, d['near'], d['far'], False, t2)
    flips = _flip_pixels(npy(nc), rnc)
    assert flips.sum() <= _allowed(d)
    assert of.shape == (H, W, 2) and np.abs(rf).max() > 0.5  # the second time step really moves the surfels
    bad = (np.abs(npy(of).astype(np.float64) - rf) > 1e-4 + 1e-3 * np.abs(rf)).any(-1)
    print(f"[{name}] flow abs err {abs_err(npy(of), rf):.3e} (max |flow| {np.abs(rf).max():.2f}), "
          f"{int(bad.sum())} pixels out of tolerance, {int(flips.sum())} threshold-flip pixels")
    assert not (bad & ~flips).any()
    assert not ((np.abs(npy(oc) - rc_) > 1e-4).any(0) & ~flips).any()

    # backward on the GPU's own forward outputs, all gradient inputs non-zero
    gi, go, ge, gf = d['grad_image'], d['grad_opacity'], d['grad_extras'], d['grad_flow']
    n64 = lambda t: f64(npy(t))
    ref = O.render_backward(m2, no, colors, tm, t2, n64(oo), n64(oe), n64(of), n64(gi), n64(go), n64(ge), n64(gf),
                            ranges, pl, npy(nc), d['near'], d['far'])
    for ordered in (True, False):
        out = f('GS_2D_render_backward')(d['means2D'], d['normal_opacity'], d['colors'], d['trans_mat'], d['t2'], oo,
                                         oe, of, gi, go, ge, gf, d['ranges'], d['point_list'], nc, d['near'], d['far'],
                                         d['offsets'] if ordered else None, d['radii'] if ordered else None)
        torch.cuda.synchronize()
        errs = {k: rel_err(npy(a), b) for k, a, b in zip(('colors', 'means2D', 'trans', 'normal_opacity'), out, ref)}
        print(f"[{name}] flow backward ({'ordered' if ordered else 'atomic'}) rel errs {errs}")
        for k, v in errs.items():
            assert v < 1e-3, (k, ordered)
    # the flow gradient really contributes: without it the matrices' gradient is different
    ref0 = O.render_backward(m2, no, colors, tm, None, n64(oo), n64(oe), None, n64(gi), n64(go), n64(ge), None, ranges,
                             pl, npy(nc), d['near'], d['far'])
    assert rel_err(ref0[2], ref[2]) > 1e-2


@pytest.mark.parametrize("with_flow", [False, True])
@pytest.mark.parametrize("name", list(CASES))
def test_accum_side_outputs(name, with_flow, device, oracle_mod):
    """accum_max_count (credited to the running arg-max of the weights, whose flag is never reset), accum_weights_p and
    accum_weights_count, element by element; the kernels add to the caller's buffers."""
    from fast_sp_gs_amd._C import get_C_function as f
    O = oracle_mod
    d = _stage(name, device)
    W, H, P = d['W'], d['H'], d['P']
    amc = torch.zeros(P, dtype=torch.int32, device=device)
    awp = torch.full((P,), 0.5, device=device)  # a non-zero start shows that the kernel accumulates
    awc = torch.zeros(P, dtype=torch.int32, device=device)
    t2 = d['t2'] if with_flow else None
    oc, oo, oe, of, nc = f('GS_2D_render_forward')(W, H, d['means2D'], d['colors'], d['normal_opacity'],
                                                   d['trans_mat'], d['point_list'], d['ranges'], d['near'], d['far'],
                                                   False, t2, amc, awp, awc)
    torch.cuda.synchronize()
    m2, colors, no, tm, pl, ranges = _n(d, 'means2D', 'colors', 'normal_opacity', 'trans_mat', 'point_list', 'ranges')
    r_amc, r_awp, r_awc = np.zeros(P, np.int32), np.full(P, 0.5, np.float64), np.zeros(P, np.int32)
    rc_, ro, re_, rf, rnc = O.render_forward(W, H, m2, colors, no, tm, pl, ranges, d['near'], d['far'], False,
                                             None if t2 is None else f64(npy(t2)), r_amc, r_awp, r_awc)
    flips = _flip_pixels(npy(nc), rnc)
    n_flip = int(flips.sum())
    assert n_flip <= _allowed(d)
    g_amc, g_awp, g_awc = npy(amc), npy(awp), npy(awc)
    assert r_awc.sum() > 10 * P / 4 and (r_amc != r_awc).any()
    # a pixel whose list is cut one entry earlier or later on one side moves the counters of the surfels in that pixel's
    # tile by one; everything else is exact
    diff_c, diff_m = np.abs(g_awc - r_awc), np.abs(g_amc - r_amc)
    print(f"[{name}] accum: count mismatches {int((diff_c > 0).sum())}, max-count mismatches {int((diff_m > 0).sum())}, "
          f"weights abs err {abs_err(g_awp, r_awp):.3e}, threshold-flip pixels {n_flip}")
    if n_flip == 0:
        assert not diff_c.any() and not diff_m.any()
    else:
        assert diff_c.sum() <= 4 * n_flip and diff_m.sum() <= 8 * n_flip
    assert g_amc.sum() == g_awc.sum()  # one arg-max credit per contributing pair
    assert (np.abs(g_awp - r_awp) <= 1e-4 + 1e-5 * np.abs(r_awp) + 1e-2 * n_flip).all()  # sums over up to 1e3 pixels
    assert not ((np.abs(npy(oc) - rc_) > 1e-4).any(0) & ~flips).any()
    # second call: the buffers accumulate (counts double exactly)
    f('GS_2D_render_forward')(W, H, d['means2D'], d['colors'], d['normal_opacity'], d['trans_mat'], d['point_list'],
                              d['ranges'], d['near'], d['far'], False, t2, amc, None, awc)
    torch.cuda.synchronize()
    assert np.array_equal(npy(amc), 2 * g_amc) and np.array_equal(npy(awc), 2 * g_awc)
    # only the max counter, through the image-only variant: untouched (the arg-max lives in the auxiliary branch)
    amc2 = torch.zeros(P, dtype=torch.int32, device=device)
    f('GS_2D_render_forward')(W, H, d['means2D'], d['colors'], d['normal_opacity'], d['trans_mat'], d['point_list'],
                              d['ranges'], d['near'], d['far'], True, None, amc2, None, None)
    torch.cuda.synchronize()
    assert not npy(amc2).any()


@pytest.mark.parametrize("name", list(CASES))
def test_only_image_and_means2D_gradient(name, device, oracle_mod):
    """only_image: no auxiliary maps, n_contrib[1] all zero, and a backward from the image and opacity gradients alone.
    Also the blend's own dL/dmeans2D (the low-pass-filter branch), compared directly, with and without auxiliary
    gradients, in both summation modes."""
    from fast_sp_gs_amd._C import get_C_function as f
    O = oracle_mod
    d = _stage(name, device)
    W, H = d['W'], d['H']
    m2, colors, no, tm, pl, ranges = _n(d, 'means2D', 'colors', 'normal_opacity', 'trans_mat', 'point_list', 'ranges')
    gi, go, ge = d['grad_image'], d['grad_opacity'], d['grad_extras']
    for only_image in (True, False):
        oc, oo, oe, of, nc = f('GS_2D_render_forward')(W, H, d['means2D'], d['colors'], d['normal_opacity'],
                                                       d['trans_mat'], d['point_list'], d['ranges'], d['near'],
                                                       d['far'], only_image, None, None, None, None)
        torch.cuda.synchronize()
        rc_, ro, re_, _, rnc = O.render_forward(W, H, m2, colors, no, tm, pl, ranges, d['near'], d['far'], only_image)
        flips = _flip_pixels(npy(nc)[:1], rnc[:1])
        assert flips.sum() <= _allowed(d)
        assert not ((np.abs(npy(oc) - rc_) > 1e-4).any(0) & ~flips).any()
        assert not ((np.abs(npy(oo) - ro) > 1e-4) & ~flips).any()
        if only_image:
            assert oe is None and of is None and re_ is None
            assert not npy(nc)[1].any() and not rnc[1].any()
        n64 = lambda t: f64(npy(t))
        ref = O.render_backward(m2, no, colors, tm, None, n64(oo), None if only_image else n64(oe), None, n64(gi),
                                n64(go), None if only_image else n64(ge), None, ranges, pl, npy(nc), d['near'],
                                d['far'])
        assert np.abs(ref[1]).max() > 0  # some pairs take the low-pass branch, so means2D has a gradient of its own
        for ordered in (True, False):
            out = f('GS_2D_render_backward')(d['means2D'], d['normal_opacity'], d['colors'], d['trans_mat'], None, oo,
                                             oe, None, gi, go, None if only_image else ge, None, d['ranges'],
                                             d['point_list'], nc, d['near'], d['far'],
                                             d['offsets'] if ordered else None, d['radii'] if ordered else None)
            torch.cuda.synchronize()
            errs = {k: rel_err(npy(a), b)
                    for k, a, b in zip(('colors', 'means2D', 'trans', 'normal_opacity'), out, ref)}
            print(f"[{name}] only_image={only_image} {'ordered' if ordered else 'atomic'} backward rel errs {errs}")
            for k, v in errs.items():
                assert v < 1e-3, (k, only_image, ordered)
