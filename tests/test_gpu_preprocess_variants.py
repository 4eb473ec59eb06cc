"""GPU parity of the standard preprocess forward/backward against the oracle over its input variants: SH degree 0..4
(degree <= 3 stages SH rows through LDS, degree 4 takes the direct path), split `shs[P,1,3] + sh_rest[P,M,3]` layout
with more rows than the active degree needs, pre-computed colours (sh_degree < 0), culling mask, caller-provided
means2D, pre-computed transform. Geometry is bit-exact; colours and SH gradients agree to rounding (FMA contraction).
Backward outputs are allocated NaN-filled to show that every row is written by the kernel.
"""
import numpy as np
import pytest
import torch

from util import abs_err, npy, rel_err

pytestmark = pytest.mark.gpu

VARIANTS = [
    # name, sh_degree, n_rows (full layout) or None, rest_rows (split layout) or None
    ("deg3_full16", 3, 16, None),
    ("deg2_full16", 2, 16, None),
    ("deg0_full1", 0, 1, None),
    ("deg3_split15", 3, None, 15),
    ("deg1_split24", 1, None, 24),
    ("deg4_full25", 4, 25, None),
    ("deg4_split24", 4, None, 24),
    ("colors", -1, None, None),
]


def _scene(P, W, H, seed):
    from fast_sp_gs_amd import scenes
    scene, _ = scenes.config0(P=P, size=max(W, H), seed=seed)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.2, 0.1, 4.0]))
    scene.means3D[::7, 2] += 9.0  # every 7th surfel behind the camera: rows that must come back as zeros
    return scene, cam


@pytest.mark.parametrize("name,deg,n_rows,rest_rows", VARIANTS)
def test_preprocess_variants(name, deg, n_rows, rest_rows, device, oracle_mod):
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    P, W, H = 3001, 200, 120  # P is not a multiple of the block size
    scene, cam = _scene(P, W, H, seed=11)
    g = torch.Generator().manual_seed(3)
    if deg < 0:
        shs, rest = torch.rand(P, 3, generator=g), None
    elif rest_rows is None:
        shs, rest = torch.randn(P, n_rows, 3, generator=g) * 0.3, None
    else:
        shs, rest = torch.randn(P, 1, 3, generator=g) * 0.3, torch.randn(P, rest_rows, 3, generator=g) * 0.1
    culling = torch.rand(P, generator=g) < 0.1
    means2D_in = torch.full((P, 2), -7.0)
    print(f"[preprocess {name}] P={P} {W}x{H} deg={deg}", flush=True)

    d = lambda t: None if t is None else t.to(device).contiguous()
    out = get_C_function('gs_2d_preprocess_forward')(
        W, H, deg, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(shs), d(rest),
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), None, d(means2D_in), d(culling))
    torch.cuda.synchronize()
    # the packed per-surfel record written by the same kernel == the one packed afterwards from the outputs, on every
    # rendered surfel (radius field included; the last field is unused); rows of surfels that are not rendered are zeros
    with_rec = get_C_function('gs_2d_preprocess_forward')(
        W, H, deg, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(shs), d(rest),
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), None, d(means2D_in), d(culling), return_records=True)
    for a, b in zip(out, with_rec[:7]):
        assert torch.equal(a, b)
    packed = get_C_function('gs_2d_pack_records')(out[0], out[1], out[3], out[2], out[5], None)
    seen = out[5] > 0
    assert torch.equal(with_rec[7][seen][:, :19].view(torch.int32), packed[seen][:, :19].view(torch.int32))
    assert 0 < int(seen.sum()) < P and not with_rec[7][~seen].any()
    m2, colors, tm, no, dep, radii, tt = [npy(t) for t in out]
    s = dict(means3D=npy(scene.means3D), scales=npy(scene.scales), rotations=npy(scene.rotations),
             opacities=npy(scene.opacities), Tw2v=npy(cam.Tw2v), Tv2c=npy(cam.Tv2c), campos=npy(cam.campos))
    r_m2, r_colors, r_tm, r_no, r_dep, r_radii, r_tt = O.preprocess_forward(
        W, H, deg, s['means3D'], s['scales'], s['rotations'], s['opacities'], npy(shs), npy(rest), s['Tw2v'],
        s['Tv2c'], s['campos'], None, npy(means2D_in).copy(), npy(culling))
    assert np.array_equal(radii, r_radii) and np.array_equal(tt, r_tt)
    assert np.array_equal(m2, r_m2) and np.array_equal(tm, r_tm) and np.array_equal(dep, r_dep)
    assert np.array_equal(no, r_no)
    vis = radii > 0
    assert 0 < vis.sum() < P and (m2[~vis] == -7.0).all()  # caller's means2D kept where nothing was rendered
    assert abs_err(colors, r_colors) < 2e-6

    # backward with NaN-filled outputs
    gm2 = torch.randn(P, 2, generator=g)
    gt, gc, gno = torch.randn(P, 3, 3, generator=g), torch.randn(P, 3, generator=g), torch.randn(P, 4, generator=g)
    nan = lambda *shape: torch.full(shape, float('nan'), device=device)
    g3, gs, gr, gop = nan(P, 3), nan(P, 2), nan(P, 4), nan(P, 1)
    gsh = None if deg < 0 else nan(*shs.shape)
    grest = None if rest is None else nan(*rest.shape)
    gm2_d = d(gm2)
    get_C_function('gs_2d_preprocess_backward')(
        W, H, deg, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(shs), d(rest),
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), out[2], out[5], out[1], out[3], gm2_d, d(gt), None, d(gc), d(gno),
        g3, gs, gr, gop, gsh, grest)
    torch.cuda.synchronize()
    r3, rs, rr, rop, rsh, rrest, rm2 = O.preprocess_backward(
        W, H, deg, s['means3D'], s['scales'], s['rotations'], npy(shs), npy(rest), s['Tw2v'], s['Tv2c'], s['campos'],
        tm, radii, colors, npy(gm2), npy(gt), npy(gc), npy(gno))
    pairs = dict(means3D=(g3, r3), scales=(gs, rs), rot=(gr, rr), opac=(gop, rop), mean2D=(gm2_d, rm2))
    if gsh is not None:
        pairs['shs'] = (gsh, rsh)
    if grest is not None:
        pairs['sh_rest'] = (grest, rrest)
    for k, (a, b) in pairs.items():
        a = npy(a)
        assert np.isfinite(a).all(), f"{k}: rows left unwritten"
        assert rel_err(a, b) < 1e-5, (k, rel_err(a, b))
        if k != 'mean2D':
            assert not a[~vis].any(), f"{k}: non-zero gradient for a surfel that was not rendered"
    # grad_scales / grad_rotations are optional in the reference (gs_2d_preprocess.cu:436, :447-448): the other outputs
    # are what they are with them
    g3b, gopb, gm2_b = nan(P, 3), nan(P, 1), d(gm2)
    get_C_function('gs_2d_preprocess_backward')(
        W, H, deg, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(shs), d(rest),
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), out[2], out[5], out[1], out[3], gm2_b, d(gt), None, d(gc), d(gno),
        g3b, None, None, gopb, None if gsh is None else nan(*shs.shape), None if grest is None else nan(*rest.shape))
    torch.cuda.synchronize()
    assert torch.equal(g3b, g3) and torch.equal(gopb, gop) and torch.equal(gm2_b, gm2_d)


def test_precomputed_transform(device, oracle_mod):
    """trans_precomp replaces the per-surfel transform: normals are (0, 0, +-1) and trans_mat is the input itself."""
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    P, W, H = 500, 96, 64
    scene, cam = _scene(P, W, H, seed=5)
    d = lambda t: t.to(device).contiguous()
    base = get_C_function('gs_2d_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), None, None, None)
    pre = base[2].clone()
    out = get_C_function('gs_2d_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), pre, None, None)
    torch.cuda.synchronize()
    ref = O.preprocess_forward(W, H, 3, npy(scene.means3D), npy(scene.scales), npy(scene.rotations),
                               npy(scene.opacities), npy(scene.shs), None, npy(cam.Tw2v), npy(cam.Tv2c),
                               npy(cam.campos), npy(pre), None, None)
    assert out[2].data_ptr() == pre.data_ptr()
    for a, b in zip((out[0], out[3], out[4], out[5], out[6]), (ref[0], ref[3], ref[4], ref[5], ref[6])):
        assert np.array_equal(npy(a), b)
    assert abs_err(npy(out[1]), ref[1]) < 2e-6
