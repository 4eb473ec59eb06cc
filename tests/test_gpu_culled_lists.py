"""The culled binning of the standard path (GS_prepare(..., cull=True), what `_GS_2D_Render` uses and what the benchmark reports beside its headline):
(surfel, tile) instances that no pixel of their tile can blend are left out of the tile lists. The reference's lists hold
every tile of a surfel's rectangle, so the lists differ by construction; what must not change is everything computed
from them. Checked here: every tile's culled list is the full list with entries removed (order kept), the forward's
images and maps are identical bit for bit, the gradients agree to the rounding of a different grouping of the same
additions, the keep masks written by the preprocess kernel equal those of the stand-alone kernel, the ordered-sum
workspace needs no clearing with culled lists either, and switching the culling off for debugging gives back the full
lists."""
import numpy as np
import pytest
import torch

from util import npy, rel_err

pytestmark = pytest.mark.gpu

CASES = {
    "c0_10k_256": (10_000, 256, 256, 1.0),
    "partial_tiles_511x127": (4_000, 511, 127, 1.0),
    "big_surfels_96x80": (300, 96, 80, 10.0),  # rectangles above 32 tiles are kept whole
    "dense_6k_96": (6_000, 96, 96, 12.0),
    "c2_300k_800": (300_000, 800, 800, 1.0),
}


def _make(name, device):
    from fast_sp_gs_amd import scenes
    P, W, H, scale_mul = CASES[name]
    if name.startswith("c2_"):
        scene, cam = scenes.config2(P=P, size=W, seed=0)
    else:
        scene, _ = scenes.config0(P=P, size=max(W, H), seed=0)
        scene.scales = scene.scales * scale_mul
        cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]))
    g = torch.Generator().manual_seed(7)
    gi = torch.randn(3, H, W, generator=g).to(device)
    ge = torch.cat([torch.randn(6, H, W, generator=g), torch.zeros(3, H, W)]).to(device)
    go = torch.randn(H, W, generator=g).to(device)
    return scene.to(device), cam.to(device), gi, ge, go


@pytest.mark.parametrize("ordered", [True, False])
@pytest.mark.parametrize("name", list(CASES))
def test_culled_lists_change_no_result(name, ordered, device):
    from fast_sp_gs_amd.renderer import render_step
    scene, cam, gi, ge, go = _make(name, device)
    full = render_step(scene, cam, gi, ge, go, ordered_sums=ordered)
    cull = render_step(scene, cam, gi, ge, go, ordered_sums=ordered, cull=True)
    torch.cuda.synchronize()
    ra, rb = npy(full['ranges']), npy(cull['ranges'])
    la, lb = ra[:, 1] - ra[:, 0], rb[:, 1] - rb[:, 0]
    print(f"[culled {name} ordered={ordered}] instances {int(la.sum())} -> {int(lb.sum())}, longest list "
          f"{int(la.max())} -> {int(lb.max())}", flush=True)
    assert (lb <= la).all() and (name.startswith("big_") or lb.sum() < la.sum())
    if scene.P <= 10_000:  # tile by tile: the culled list is the full list with entries taken out
        pa, pb = npy(full['point_list']), npy(cull['point_list'])
        for t in range(ra.shape[0]):
            a, b = pa[ra[t, 0]:ra[t, 1]], pb[rb[t, 0]:rb[t, 1]]
            assert np.array_equal(a[np.isin(a, b)], b), t
    for k in ('image', 'opacity', 'extras', 'means2D', 'radii', 'tiles_touched'):
        assert torch.equal(full[k], cull[k]), k
    for k in ('g_colors', 'g_means2D', 'g_trans', 'g_normal_opacity', 'g_means3D', 'g_scales', 'g_rot', 'g_opac',
              'g_shs'):
        assert bool(torch.isfinite(cull[k]).all()), k
        assert rel_err(npy(cull[k]), npy(full[k])) < (1e-5 if ordered else 1e-4), k


@pytest.mark.parametrize("name", ["partial_tiles_511x127", "big_surfels_96x80", "dense_6k_96"])
def test_keep_masks_of_the_preprocess_equal_the_stand_alone_kernel(name, device):
    from fast_sp_gs_amd import lib as L
    from fast_sp_gs_amd._C import get_C_function as f
    lib = L.load()
    scene, cam, *_ = _make(name, device)
    *_, radii, tt, records, masks = f('gs_2d_preprocess_forward')(
        cam.W, cam.H, 3, False, scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs, None,
        cam.Tw2v, cam.Tv2c, cam.campos, None, None, None, return_records=True, return_masks=True)
    alone = torch.full_like(masks, 12345)
    L.check(lib.fsgs_gs_2d_cull_masks(scene.P, cam.W, cam.H, L.ptr(records), L.ptr(radii), L.ptr(alone),
                                      L.current_stream()), 'cull_masks')
    torch.cuda.synchronize()
    assert torch.equal(masks, alone)
    m, area = npy(masks).view(np.uint32), npy(tt)
    small = (area > 0) & (area <= 32)
    # no bit beyond the rectangle, some tile dropped somewhere, large rectangles and hidden surfels keep every bit
    assert ((m[small] >> area[small].astype(np.uint32)) == 0).all()
    assert (m[~small] == 0xffffffff).all()
    popcount = np.array([bin(int(v)).count('1') for v in m[small]])
    assert (popcount < area[small]).any() or name.startswith("big_")


def test_culling_switched_off_gives_the_full_lists(device):
    from fast_sp_gs_amd import lib as L
    from fast_sp_gs_amd.renderer import render_step
    lib = L.load()
    scene, cam, gi, ge, go = _make("c0_10k_256", device)
    full = render_step(scene, cam, gi, ge, go)
    lib.fsgs_debug_set_culling(0)
    try:
        off = render_step(scene, cam, gi, ge, go, cull=True)
        torch.cuda.synchronize()
    finally:
        lib.fsgs_debug_set_culling(1)
    assert torch.equal(full['ranges'], off['ranges']) and torch.equal(full['point_list'], off['point_list'])
    for k in ('image', 'opacity', 'extras'):
        assert torch.equal(full[k], off[k]), k


@pytest.mark.parametrize("variant", ["aux", "image_only"])
def test_culled_backward_workspace_needs_no_clearing(variant, device):
    """fsgs_gs_2d_render_backward_culled through the C ABI with a poisoned workspace: the positions of a surfel's span that
    the binning left out are never written, and the record sum must not read them."""
    from fast_sp_gs_amd import lib as L, scenes
    from fast_sp_gs_amd._C import get_C_function as f
    lib = L.load()
    W, H, P = 320, 208, 6000
    g = torch.Generator().manual_seed(3)
    scene = scenes._surfels(g, P, 'cube', -3.2, 0.4, 3.0, 1.0)
    scene.means3D[:, 0] = scene.means3D[:, 0] * 0.6 - 0.5
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    sc, cm = scene.to(device), cam.to(device)
    m2, colors, tm, no, depths, radii, tt, records, masks = f('gs_2d_preprocess_forward')(
        W, H, 3, False, sc.means3D, sc.scales, sc.rotations, sc.opacities, sc.shs, None, cm.Tw2v, cm.Tv2c, cm.campos,
        None, None, None, return_records=True, return_masks=True)
    ranges, point_list, offsets = f('GS_prepare')(W, H, m2, depths, radii, tt, False, return_offsets=True,
                                                  records=records, cull=True, keep_masks=masks)[:3]
    kept, total = int((ranges[:, 1] - ranges[:, 0]).sum()), int(point_list.numel())
    print(f"[culled contract {variant}] {kept} of {total} instances kept")
    assert 0 < kept < total
    only_image = variant == "image_only"
    oc, oo, oe, of, nc = f('GS_2D_render_forward')(W, H, m2, colors, no, tm, point_list, ranges, cam.near, cam.far,
                                                   only_image, None, None, None, None, records)
    g2 = torch.Generator().manual_seed(9)
    gi = torch.randn(3, H, W, generator=g2).to(device)
    ge = torch.cat([torch.randn(6, H, W, generator=g2), torch.zeros(3, H, W)]).to(device)
    go = torch.randn(H, W, generator=g2).to(device)
    aux = not only_image
    nbytes = lib.fsgs_gs_2d_render_backward_workspace_bytes(total)

    def run(fill, ordered=True):
        ws = torch.empty(nbytes // 4, device=device)
        ws.fill_(fill)
        out = [torch.full((P, n), float('nan'), device=device) if ordered else torch.zeros(P, n, device=device)
               for n in (3, 2, 9, 4)]
        rc = lib.fsgs_gs_2d_render_backward_culled(
            P, W, H, float(cam.near), float(cam.far), L.ptr(m2), L.ptr(no), L.ptr(colors), L.ptr(tm), None, L.ptr(oo),
            L.ptr(oe) if aux else None, None, L.ptr(gi), L.ptr(go), L.ptr(ge) if aux else None, None, L.ptr(ranges),
            L.ptr(point_list), L.ptr(nc), L.ptr(out[0]), L.ptr(out[1]), L.ptr(out[2]), L.ptr(out[3]), total,
            L.ptr(offsets) if ordered else None, L.ptr(radii) if ordered else None, L.ptr(ws) if ordered else None,
            nbytes if ordered else 0, L.ptr(records), L.ptr(masks), L.current_stream())
        L.check(rc, 'fsgs_gs_2d_render_backward_culled')
        torch.cuda.synchronize()
        return [npy(o) for o in out]

    zeroed = run(0.0)
    for fill in (float('nan'), 3.0e30):
        poisoned = run(fill)
        for a, b in zip(poisoned, zeroed):
            assert np.isfinite(a).all(), fill
            assert np.array_equal(a, b), fill
    atomic = run(0.0, ordered=False)
    for name, a, b in zip(('colors', 'means2D', 'trans', 'normal_opacity'), zeroed, atomic):
        if np.abs(b).max() > 0:
            assert rel_err(a, b) < 1e-3, name


# ---- 3D Gaussians: the same culling with the conic's alpha >= 1/255 ellipse ---------------------------------------------
def _gs3d_stages(device, P, W, H, scale_mul, seed=3):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    scene, _ = scenes.config0(P=P, size=max(W, H), seed=seed)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]))
    g = torch.Generator().manual_seed(seed + 100)
    scales = torch.cat([scene.scales * scale_mul,
                        scene.scales[:, :1] * scale_mul * (0.3 + 3.0 * torch.rand(P, 1, generator=g))], 1).contiguous()
    tan_fov = (W / 2 / float(cam.Tv2s[0, 0]), H / 2 / float(cam.Tv2s[1, 1]))
    d = lambda t: t.to(device).contiguous()
    m2, dep, col, rad, tt, c3, co = f('gs_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, None, None, None, None)
    gi = torch.randn(3, H, W, generator=g).to(device)
    go = torch.randn(H, W, generator=g).to(device)
    return f, m2, dep, col, rad, tt, co, gi, go


@pytest.mark.parametrize("name,P,W,H,mul", [("small_4k_200x120", 4_000, 200, 120, 3.0),
                                            ("big_300_96x80", 300, 96, 80, 30.0),
                                            ("c2_300k_800", 300_000, 800, 800, 1.0)])
@pytest.mark.parametrize("sums", ["atomic", "ordered", "ordered_bucket"])
def test_gs3d_culled_lists_change_no_result(name, P, W, H, mul, sums, device):
    f, m2, dep, col, rad, tt, co, gi, go = _gs3d_stages(device, P, W, H, mul)
    masks = f('gs_cull_masks')(W, H, m2, co, rad)
    full = f('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True)
    cull = f('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True, cull=True, keep_masks=masks)
    ra, rb = npy(full[0]), npy(cull[0])
    la, lb = ra[:, 1] - ra[:, 0], rb[:, 1] - rb[:, 0]
    print(f"[gs3d culled {name} {sums}] instances {int(la.sum())} -> {int(lb.sum())}, longest list {int(la.max())} -> "
          f"{int(lb.max())}", flush=True)
    assert (lb <= la).all() and (name.startswith("big_") or lb.sum() < la.sum())
    assert torch.equal(full[2], cull[2])  # the scan is over the full rectangles either way
    if P <= 10_000:
        pa, pb = npy(full[1]), npy(cull[1])
        for t in range(ra.shape[0]):
            a, b = pa[ra[t, 0]:ra[t, 1]], pb[rb[t, 0]:rb[t, 1]]
            assert np.array_equal(a[np.isin(a, b)], b), t
    outs = []
    for (ranges, pl, offsets), keep in ((full[:3], None), (cull[:3], masks)):
        if sums == "ordered_bucket":
            boff = torch.cumsum((ranges[:, 1] - ranges[:, 0] + 31) // 32, 0).contiguous()
            oc, oo, _, nc, mc, b2t, sT, sar = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges, None,
                                                                              None, None, boff)
            # poison what the caching allocator is going to hand out as the record workspace
            junk = torch.full((int(pl.numel()) * 16 + 64,), float('nan'), device=device)
            del junk
            g = f('gaussian_rasterize_fast_backward')(m2, co, col, None, oc, None, oo, gi, go, None, ranges, pl, nc, mc,
                                                      boff, b2t, sT, sar, offsets, rad, per_gaussian=True, culled=keep)
        else:
            oc, oo, _, nc = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges)
            junk = torch.full((int(pl.numel()) * 16 + 64,), float('nan'), device=device)
            del junk
            g = f('gaussian_rasterize_backward')(m2, co, col, None, oo, gi, go, None, ranges, pl, nc,
                                                 offsets if sums == "ordered" else None,
                                                 rad if sums == "ordered" else None, culled=keep)
        outs.append((oc, oo, g))
    torch.cuda.synchronize()
    (oc_a, oo_a, g_a), (oc_b, oo_b, g_b) = outs
    assert torch.equal(oc_a, oc_b) and torch.equal(oo_a, oo_b)
    for k, (a, b) in zip(('g_colors', 'g_extras', 'g_means2D', 'g_conic_opacity'), zip(g_a, g_b)):
        if a is None:
            continue
        assert bool(torch.isfinite(b).all()), k
        assert rel_err(npy(b), npy(a)) < (1e-5 if sums != "atomic" else 1e-4), k


def test_gs3d_renderer_culls_by_default(device):
    """`RasterizeGaussians` (CULL_LISTS) against the same call on the reference's lists: images bit for bit, parameter
    gradients to rounding, for the atomic and the ordered sums."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.renderer import gaussian_render as GR
    P, W, H = 5_000, 160, 112
    scene, _ = scenes.config0(P=P, size=W, seed=5)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]))
    g = torch.Generator().manual_seed(9)
    scales = torch.cat([scene.scales * 3, scene.scales[:, :1] * (0.5 + 3.5 * torch.rand(P, 1, generator=g))], 1)
    gi = torch.randn(3, H, W, generator=g).to(device)
    d = lambda t: t.to(device).contiguous()
    focals = torch.tensor([float(cam.Tv2s[0, 0]), float(cam.Tv2s[1, 1])], device=device)
    results = {}
    try:
        for ordered in (False, True):
            for cull in (False, True):
                GR.CULL_LISTS, GR.DETERMINISTIC_SUMS = cull, ordered
                params = [d(t).requires_grad_(True) for t in (scene.means3D, scene.opacities, scales, scene.rotations,
                                                              scene.shs)]
                out = GR.render(d(cam.Tw2v), d(cam.Tv2c), (W, H), params[0], params[1], scales=params[2],
                                rotations=params[3], campos=d(cam.campos), focals=focals, sh_features=params[4],
                                sh_degree=3)
                (out['images'] * gi).sum().backward()
                results[(ordered, cull)] = (out['images'].detach(), [p.grad for p in params],
                                            int(out['buffer'].point_list.numel()),
                                            int((out['buffer'].tile_ranges[:, 1] - out['buffer'].tile_ranges[:, 0]).sum()))
    finally:
        GR.CULL_LISTS, GR.DETERMINISTIC_SUMS = True, False
    torch.cuda.synchronize()
    for ordered in (False, True):
        (im_a, g_a, _, n_a), (im_b, g_b, _, n_b) = results[(ordered, False)], results[(ordered, True)]
        assert n_b < n_a
        assert torch.equal(im_a, im_b)
        for a, b in zip(g_a, g_b):
            assert rel_err(npy(b), npy(a)) < 1e-4


def test_culled_paths_with_nothing_to_do(device):
    """A scene entirely behind the camera through the culled paths (R == 0: every mask is all-ones by convention and no
    kernel of the binning or the backward has anything to visit), surfels and 3D Gaussians."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    from fast_sp_gs_amd.renderer import render_step
    scene, cam = scenes.config0(P=64, size=64, seed=3)
    scene.means3D[:, 2] += 10.0
    for ordered in (True, False):
        out = render_step(scene.to(device), cam.to(device), torch.zeros(3, 64, 64, device=device), cull=True,
                          ordered_sums=ordered)
        torch.cuda.synchronize()
        assert out['point_list'].numel() == 0 and int(out['ranges'].abs().sum()) == 0
        assert float(out['image'].abs().sum()) == 0 and float(out['g_means3D'].abs().sum()) == 0
    W = H = 64
    tan_fov = (W / 2 / float(cam.Tv2s[0, 0]), H / 2 / float(cam.Tv2s[1, 1]))
    d = lambda t: t.to(device).contiguous()
    scales = torch.cat([scene.scales, scene.scales[:, :1]], 1)
    m2, dep, col, rad, tt, c3, co = f('gs_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, None, None, None, None)
    masks = f('gs_cull_masks')(W, H, m2, co, rad)
    ranges, pl, offsets = f('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True, cull=True,
                                          keep_masks=masks)[:3]
    oc, oo, _, nc = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges)
    z = torch.zeros(3, H, W, device=device)
    for ordered in (True, False):
        g = f('gaussian_rasterize_backward')(m2, co, col, None, oo, z, z[0], None, ranges, pl, nc,
                                             offsets if ordered else None, rad if ordered else None,
                                             culled=masks if ordered else None)
        torch.cuda.synchronize()
        assert pl.numel() == 0 and int((masks != -1).sum()) == 0
        assert all(float(t.abs().sum()) == 0 for t in g if t is not None)
    # no points at all
    e = lambda *s: torch.zeros(*s, device=device)
    masks0 = f('gs_cull_masks')(W, H, e(0, 2), e(0, 4), torch.zeros(0, dtype=torch.int32, device=device))
    assert masks0.numel() == 1
