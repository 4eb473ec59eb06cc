"""The ordered-sum path of fsgs_gs_2d_render_backward promises that its workspace needs no clearing: every (surfel, tile)
instance's record is written on every call -- by the tile's block at the flush of the batch that staged it, or by the
block's tail clear for the instances behind the tile's deepest contributor. Tests that take the workspace from torch's
caching allocator cannot see a record that is never written (the block still holds the previous call's values), so
this one calls the C ABI itself and poisons the workspace first: NaN, a huge constant, and zeros must give bit-identical,
finite outputs, for every instantiation of the kernel (auxiliary maps, auxiliary maps + flow, image only), with the
per-surfel inputs taken from the four tensors, from packed records that carry radius and offset, and from records
packed without them (radius and offset read -1, the kernel falls back to its radii / point_offsets arguments).
The scene is built so that every class of tile occurs, and the test asserts that it does: empty tiles, lists longer than
one staged batch (64), and tiles whose deepest contributor lies before the end of the list.
"""
import numpy as np
import pytest
import torch

from util import npy, rel_err

pytestmark = pytest.mark.gpu


def _scene(device):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    W, H, P = 320, 208, 6000
    g = torch.Generator().manual_seed(3)
    # opaque, fairly large surfels in the left two thirds of the view: pixels saturate long before their lists end, the
    # right-hand tiles stay empty
    scene = scenes._surfels(g, P, 'cube', -3.2, 0.4, 3.0, 1.0)
    scene.means3D[:, 0] = scene.means3D[:, 0] * 0.6 - 0.5
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    sc, cm = scene.to(device), cam.to(device)
    m2, colors, tm, no, depths, radii, tt = f('gs_2d_preprocess_forward')(
        W, H, 3, False, sc.means3D, sc.scales, sc.rotations, sc.opacities, sc.shs, None, cm.Tw2v, cm.Tv2c, cm.campos,
        None, None, None)
    ranges, point_list, offsets = f('GS_prepare')(W, H, m2, depths, radii, tt, False, return_offsets=True)
    Tw2c = (cm.Tv2c @ cm.Tw2v).contiguous()
    t2, _ = f('gs_2d_compute_transmat_forward')(W, H, (sc.means3D + 0.02).contiguous(), sc.scales, sc.rotations,
                                                cm.Tw2v, Tw2c)
    d = dict(W=W, H=H, P=P, near=cam.near, far=cam.far, means2D=m2, colors=colors, trans_mat=tm, normal_opacity=no,
             radii=radii, ranges=ranges, point_list=point_list, offsets=offsets, t2=t2)
    g2 = torch.Generator().manual_seed(9)
    d['gi'] = torch.randn(3, H, W, generator=g2).to(device)
    d['ge'] = torch.cat([torch.randn(6, H, W, generator=g2), torch.zeros(3, H, W)]).to(device)
    d['go'] = torch.randn(H, W, generator=g2).to(device)
    d['gf'] = torch.randn(H, W, 2, generator=g2).to(device)
    return d


def _tile_classes(d, nc):
    """(#empty tiles, #tiles longer than a staged batch, #tiles whose deepest contributor is not the list's last entry)."""
    W, H = d['W'], d['H']
    gx, gy = (W + 15) // 16, (H + 15) // 16
    ranges = npy(d['ranges'])
    length = ranges[:, 1] - ranges[:, 0]
    last = npy(nc)[0]
    pad = np.zeros((gy * 16, gx * 16), last.dtype)
    pad[:H, :W] = last
    deepest = pad.reshape(gy, 16, gx, 16).max(axis=(1, 3)).reshape(-1)
    return int((length == 0).sum()), int((length > 64).sum()), int(((deepest < length) & (length > 0)).sum())


@pytest.mark.parametrize("variant", ["aux", "aux_flow", "image_only"])
@pytest.mark.parametrize("source", ["tensors", "records_full", "records_bare"])
def test_backward_workspace_needs_no_clearing(variant, source, device):
    from fast_sp_gs_amd import lib as L
    from fast_sp_gs_amd._C import get_C_function as f
    lib = L.load()
    d = _scene(device)
    W, H, P = d['W'], d['H'], d['P']
    flow, only_image = variant == "aux_flow", variant == "image_only"
    oc, oo, oe, of, nc = f('GS_2D_render_forward')(W, H, d['means2D'], d['colors'], d['normal_opacity'],
                                                   d['trans_mat'], d['point_list'], d['ranges'], d['near'], d['far'],
                                                   only_image, d['t2'] if flow else None, None, None, None)
    empty, long_, cut = _tile_classes(d, nc)
    print(f"[{variant}/{source}] tiles: {empty} empty, {long_} longer than 64 entries, {cut} cut before their end")
    assert empty > 0 and long_ > 0 and cut > 0

    records = None
    if source != "tensors":
        records = torch.empty(P, 20, device=device)
        full = source == "records_full"
        L.check(lib.fsgs_gs_2d_pack_records(P, L.ptr(d['means2D']), L.ptr(d['colors']), L.ptr(d['normal_opacity']),
                                            L.ptr(d['trans_mat']), L.ptr(d['radii']) if full else None,
                                            L.ptr(d['offsets']) if full else None, L.ptr(records), L.current_stream()),
                'pack_records')
        if not full:
            tail = npy(records)[:, 18:20].copy().view(np.int32)
            assert (tail == -1).all()  # neither radius nor offset in the record

    R = int(d['point_list'].numel())
    nbytes = lib.fsgs_gs_2d_render_backward_workspace_bytes(R)
    aux = not only_image

    def run(fill, ordered=True):
        ws = torch.empty(nbytes // 4, device=device)
        ws.fill_(fill)
        out = [torch.full((P, n), float('nan'), device=device) if ordered else torch.zeros(P, n, device=device)
               for n in (3, 2, 9, 4)]
        rc = lib.fsgs_gs_2d_render_backward(
            P, W, H, float(d['near']), float(d['far']), L.ptr(d['means2D']), L.ptr(d['normal_opacity']),
            L.ptr(d['colors']), L.ptr(d['trans_mat']), L.ptr(d['t2']) if flow else None, L.ptr(oo),
            L.ptr(oe) if aux else None, L.ptr(of) if flow else None, L.ptr(d['gi']), L.ptr(d['go']),
            L.ptr(d['ge']) if aux else None, L.ptr(d['gf']) if flow else None, L.ptr(d['ranges']),
            L.ptr(d['point_list']), L.ptr(nc), L.ptr(out[0]), L.ptr(out[1]), L.ptr(out[2]), L.ptr(out[3]), R,
            L.ptr(d['offsets']) if ordered else None, L.ptr(d['radii']) if ordered else None,
            L.ptr(ws) if ordered else None, nbytes if ordered else 0, L.ptr(records), L.current_stream())
        L.check(rc, 'fsgs_gs_2d_render_backward')
        torch.cuda.synchronize()
        return [npy(o) for o in out]

    zeroed = run(0.0)
    for o in zeroed:
        assert np.isfinite(o).all()
    for fill in (float('nan'), 3.0e30):
        poisoned = run(fill)
        for a, b in zip(poisoned, zeroed):
            assert np.isfinite(a).all(), fill
            assert np.array_equal(a, b), fill  # bit for bit: no record keeps what the workspace held before
    atomic = run(0.0, ordered=False)
    for name, a, b in zip(('colors', 'means2D', 'trans', 'normal_opacity'), zeroed, atomic):
        if np.abs(b).max() > 0:
            assert rel_err(a, b) < 1e-3, name


@pytest.mark.parametrize("masks", ["test_repeated", "keep_masks"])
@pytest.mark.parametrize("kernel", ["tile", "per_splat"])
@pytest.mark.parametrize("variant", ["aux", "image_only"])
def test_fast_backward_workspace_needs_no_clearing(variant, kernel, masks, device):
    """The same promise on the fast path, whose key spans hold positions that belong to no tile's list (tiles of the
    rectangle that fail the corner test): the record sum repeats the binning's test and reads only the positions the
    blend wrote, so nothing is cleared there either. Both backward kernels (back to front per tile / the per-splat
    decomposition over 32-entry buckets), with and without the auxiliary maps, the sum repeating the test or reading its
    verdicts from the preprocess kernel's keep masks."""
    from fast_sp_gs_amd import lib as L, scenes
    from fast_sp_gs_amd._C import get_C_function as f
    lib = L.load()
    W, H, P = 320, 208, 6000
    g = torch.Generator().manual_seed(3)
    scene = scenes._surfels(g, P, 'cube', -3.2, 0.4, 3.0, 1.0)
    scene.means3D[:, 0] = scene.means3D[:, 0] * 0.6 - 0.5
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    sc, cm = scene.to(device), cam.to(device)
    (m2, colors, tm, im, no, depths, radii, ranges, point_list, keys, tt, offsets,
     keep) = f('gs_2d_fast_preprocess_forward')(
        W, H, 3, False, sc.means3D, sc.scales, sc.rotations, sc.opacities, sc.shs, None, cm.Tw2v, cm.Tv2c, cm.Tv2s,
        cm.campos, None, None, None, False, True, True, True)
    b_off = torch.cumsum((ranges[:, 1] - ranges[:, 0] + 31) // 32, 0).contiguous()
    image, oo, oe, _, nc, max_c, b2t, s_T, s_acc, s_aux = f('GS_2D_fast_render_forward')(
        W, H, cam.near, cam.far, False, m2, colors, no, tm, im, point_list, ranges, None, None, None, None, b_off)[:10]
    d = dict(W=W, H=H, ranges=ranges)
    empty, long_, cut = _tile_classes(d, nc)
    n_pad = int((point_list == -1).sum())
    print(f"[fast {variant}/{kernel}] tiles: {empty} empty, {long_} longer than 64 entries, {cut} cut before their "
          f"end; {n_pad} of {point_list.numel()} key positions are padding")
    assert empty > 0 and long_ > 0 and cut > 0 and n_pad > 0
    g2 = torch.Generator().manual_seed(9)
    gi = torch.randn(3, H, W, generator=g2).to(device)
    ge = torch.randn(8, H, W, generator=g2).to(device)
    go = torch.randn(H, W, generator=g2).to(device)
    aux = variant == "aux"
    R = int(point_list.numel())
    nbytes = lib.fsgs_gs_2d_fast_render_backward_workspace_bytes(R)
    B = int(b2t.numel())

    def run(fill, ordered=True):
        ws = torch.empty(nbytes // 4, device=device)
        ws.fill_(fill)
        out = [torch.full((P, n), float('nan'), device=device) if ordered else torch.zeros(P, n, device=device)
               for n in (3, 2, 9, 9, 4)]  # colours, means2D, transform, adjugate, normal + opacity
        tail = (R, L.ptr(offsets) if ordered else None, L.ptr(radii) if ordered else None,
                L.ptr(ws) if ordered else None, nbytes if ordered else 0,
                L.ptr(keep) if ordered and masks == "keep_masks" else None, L.current_stream())
        if kernel == "tile":
            rc = lib.fsgs_gs_2d_fast_render_backward(
                P, W, H, float(cam.near), float(cam.far), 1, L.ptr(m2), L.ptr(no), L.ptr(colors), L.ptr(tm), L.ptr(im),
                None, L.ptr(oo), L.ptr(oe) if aux else None, None, L.ptr(gi), L.ptr(go), L.ptr(ge) if aux else None,
                None, L.ptr(ranges), L.ptr(point_list), L.ptr(nc), L.ptr(out[0]), L.ptr(out[1]), L.ptr(out[2]),
                L.ptr(out[3]), L.ptr(out[4]), *tail)
        else:
            rc = lib.fsgs_gs_2d_fast_render_bucket_backward(
                P, W, H, float(cam.near), float(cam.far), B, L.ptr(m2), L.ptr(no), L.ptr(colors), L.ptr(tm), L.ptr(im),
                L.ptr(image), L.ptr(oo), L.ptr(oe) if aux else None, L.ptr(nc), L.ptr(max_c), L.ptr(b_off), L.ptr(b2t),
                L.ptr(s_T), L.ptr(s_acc), L.ptr(s_aux), L.ptr(gi), L.ptr(go), L.ptr(ge) if aux else None,
                L.ptr(ranges), L.ptr(point_list), L.ptr(out[0]), L.ptr(out[1]), L.ptr(out[2]), L.ptr(out[3]),
                L.ptr(out[4]), *tail)
        L.check(rc, 'fast backward')
        torch.cuda.synchronize()
        return [npy(o) for o in out]

    zeroed = run(0.0)
    for o in zeroed:
        assert np.isfinite(o).all()
    for fill in (float('nan'), 3.0e30):
        poisoned = run(fill)
        for a, b in zip(poisoned, zeroed):
            assert np.isfinite(a).all(), fill
            assert np.array_equal(a, b), fill
    atomic = run(0.0, ordered=False)
    for name, a, b in zip(('colors', 'means2D', 'trans', 'inv', 'normal_opacity'), zeroed, atomic):
        if np.abs(b).max() > 0:
            assert rel_err(a, b) < 1e-3, name
    assert np.abs(zeroed[0]).max() > 0 and np.abs(zeroed[3]).max() > 0


@pytest.mark.parametrize("lists", ["full", "culled"])
def test_gs3d_backward_workspace_needs_no_clearing(lists, device):
    """The same promise on the 3D-Gaussian path: every staged instance writes its record, a tile's block clears the
    records of its never-staged tail, and with culled lists fsgs_gaussian_rasterize_clear_culled zeroes exactly the
    records of the instances that are in no list. A workspace full of NaN or 3e30 gives the zeroed workspace's result
    bit for bit."""
    from fast_sp_gs_amd import lib as L, scenes
    from fast_sp_gs_amd._C import get_C_function as f
    lib = L.load()
    W, H, P = 320, 208, 6000
    scene, _ = scenes.config0(P=P, size=W, seed=3)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]))
    g = torch.Generator().manual_seed(103)
    scales = torch.cat([scene.scales * 3, scene.scales[:, :1] * (0.5 + 3.5 * torch.rand(P, 1, generator=g))], 1)
    scene.opacities[::3] = 0.999  # opaque Gaussians in front: tiles whose lists are cut before their end
    tan_fov = (W / 2 / float(cam.Tv2s[0, 0]), H / 2 / float(cam.Tv2s[1, 1]))
    d = lambda t: t.to(device).contiguous()
    m2, dep, col, rad, tt, c3, co = f('gs_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), tan_fov, None, None, None, None)
    masks = f('gs_cull_masks')(W, H, m2, co, rad)
    culled = lists == "culled"
    ranges, pl, offsets = f('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True, cull=culled,
                                          keep_masks=masks if culled else None)[:3]
    oc, oo, _, nc = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges)
    lens = npy(ranges[:, 1] - ranges[:, 0]).reshape((H + 15) // 16, (W + 15) // 16)
    deepest = torch.nn.functional.max_pool2d(nc[None, None].float(), 16, ceil_mode=True)[0, 0].cpu().numpy()
    empty, long_, cut = int((lens == 0).sum()), int((lens > 64).sum()), int(((deepest < lens) & (lens > 0)).sum())
    print(f"[gs3d {lists}] tiles: {empty} empty, {long_} longer than 64 entries, {cut} cut before their end; "
          f"{int(lens.sum())} of {pl.numel()} instances listed")
    assert empty > 0 and long_ > 0 and cut > 0
    gi = torch.randn(3, H, W, generator=g).to(device)
    go = torch.randn(H, W, generator=g).to(device)
    R = int(pl.numel())
    nbytes = lib.fsgs_gaussian_rasterize_backward_workspace_bytes(R)

    def run(fill, ordered=True):
        ws = torch.empty(nbytes // 4, device=device)
        ws.fill_(fill)
        out = [torch.full((P, n), float('nan'), device=device) if ordered else torch.zeros(P, n, device=device)
               for n in (2, 4, 3)]  # means2D, conic + opacity, colours
        if ordered and culled:
            L.check(lib.fsgs_gaussian_rasterize_clear_culled(P, R, L.ptr(offsets), L.ptr(masks), L.ptr(ws), nbytes,
                                                             L.current_stream()), 'clear_culled')
        rc = lib.fsgs_gaussian_rasterize_backward(
            P, W, H, 0, L.ptr(m2), L.ptr(co), L.ptr(col), None, L.ptr(oo), L.ptr(nc), L.ptr(gi), None, L.ptr(go),
            L.ptr(pl), L.ptr(ranges), L.ptr(out[0]), L.ptr(out[1]), L.ptr(out[2]), None, R,
            L.ptr(offsets) if ordered else None, L.ptr(rad) if ordered else None, L.ptr(ws) if ordered else None,
            nbytes if ordered else 0, L.current_stream())
        L.check(rc, 'fsgs_gaussian_rasterize_backward')
        torch.cuda.synchronize()
        return [npy(o) for o in out]

    zeroed = run(0.0)
    for o in zeroed:
        assert np.isfinite(o).all()
    for fill in (float('nan'), 3.0e30):
        poisoned = run(fill)
        for a, b in zip(poisoned, zeroed):
            assert np.isfinite(a).all(), fill
            assert np.array_equal(a, b), fill
    atomic = run(0.0, ordered=False)
    for name, a, b in zip(('means2D', 'conic_opacity', 'colors'), zeroed, atomic):
        assert np.abs(b).max() > 0 and rel_err(a, b) < 1e-3, name
