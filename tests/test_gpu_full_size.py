"""Full-size checks of the render path through size-independent properties, beside the stage-by-stage comparisons with
the oracle that test_gpu_render_parity.py and test_gpu_fast_parity.py also run at 300 000 / 3 000 000 surfels:
  * the per-quadrant culling of the blend kernels is exact: with it switched off (every staged surfel evaluated at every
    pixel, as the reference does) the forward outputs are identical bit for bit and the gradients agree to the rounding
    of the reordered atomic sums;
  * the tile lists without the instances that no pixel of their tile can blend (what _GS_2D_Render bins) give the
    same maps bit for bit and the same gradients to rounding as the reference's full lists;
  * binning invariants: sorted masked keys, ranges partition [0, R) in tile order, every entry carries its tile's id;
  * the blend weights accumulated per surfel sum to the opacity image;
  * the backward is linear in the upstream gradients, and its two ways of summing a surfel's gradient over tiles
    (per-instance records summed in order / device-scope atomics) agree;
  * K-NN at 3M x 2048, k = 8: distances ascending, equal to the distance recomputed from the returned index, no
    closer control point exists for a sample of queries (brute force with torch), and indices and distances bit for
    bit against the oracle's all-pairs search.
Sizes: 300 000 surfels at 800x800, 3 000 000 surfels at 1352x1014 (each of the four views), 400 000 surfels at
3840x2160.
The fast path and the 3D-Gaussian path get the same kind of checks at 300 000 / 800x800 (culling, ordered against atomic
sums, linearity, weight sums; for the fast path also its two backward algorithms against each other).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _culling(enabled):
    from fast_sp_gs_amd import lib
    lib.check(lib.load().fsgs_debug_set_culling(int(enabled)), 'debug_set_culling')


def _render(scene, cam, gi, ge, go, ordered_sums=True, packed=True, cull=False):
    from fast_sp_gs_amd.renderer import render_step
    out = render_step(scene, cam, gi, ge, go, ordered_sums=ordered_sums, packed=packed, cull=cull)
    torch.cuda.synchronize()
    return out


def _check_binning(out, W, H):
    T = ((W + 15) // 16) * ((H + 15) // 16)
    ranges, pl = out['ranges'], out['point_list']
    R = pl.numel()
    lens = ranges[:, 1] - ranges[:, 0]
    assert int(lens.min()) >= 0 and int(lens.sum()) == R
    nz = lens > 0
    starts, ends = ranges[nz, 0], ranges[nz, 1]
    assert int(starts[0]) == 0 and int(ends[-1]) == R and torch.equal(starts[1:], ends[:-1])
    assert T == ranges.shape[0]
    # within a tile, depth bits ascend; recompute the keys from the outputs
    tile_of = torch.repeat_interleave(torch.arange(T, device=pl.device), lens)
    depth_bits = out['depths'].view(torch.int32)[pl.long()].long()
    keys = (tile_of << 32) | depth_bits
    assert bool((keys[1:] >= keys[:-1]).all())
    # every listed surfel's rectangle contains its tile
    m2, rad = out['means2D'][pl.long()], out['radii'][pl.long()].float()
    gx = (W + 15) // 16
    tx, ty = (tile_of % gx).float(), (tile_of // gx).float()
    assert bool(((m2[:, 0] + rad + 16 > tx * 16) & (m2[:, 0] - rad < (tx + 1) * 16)).all())
    assert bool(((m2[:, 1] + rad + 16 > ty * 16) & (m2[:, 1] - rad < (ty + 1) * 16)).all())


@pytest.mark.parametrize("config", ["c2_300k_800", "c4_3m_1352x1014_view0", "c4_3m_1352x1014_view1",
                                    "c4_3m_1352x1014_view2", "c4_3m_1352x1014_view3", "uhd_400k_3840x2160"])
def test_render_path_properties(config, device):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function
    if config == "c2_300k_800":
        scene_h, cam_h = scenes.config2()
    elif config == "uhd_400k_3840x2160":  # pixel coordinates in the thousands stress the footprint-box arithmetic
        scene_h, _ = scenes.config2(P=400_000, size=64)
        cam_h = scenes.pinhole(3840, 2160, 40.0, torch.tensor([0.5, 0.3, 4.0]))
    else:
        scene_h, cams = scenes.config4()
        cam_h = cams[int(config[-1])]
    W, H = cam_h.W, cam_h.H
    g = torch.Generator().manual_seed(9)
    gi = torch.randn(3, H, W, generator=g).to(device)
    ge = torch.cat([torch.randn(6, H, W, generator=g), torch.zeros(3, H, W)]).to(device)
    go = torch.randn(H, W, generator=g).to(device)
    scene, cam = scene_h.to(device), cam_h.to(device)
    print(f"[full {config}] P={scene.P} {W}x{H}", flush=True)

    _culling(True)
    a = _render(scene, cam, gi, ge, go)
    print(f"[full {config}] R={a['point_list'].numel()} visible={int((a['radii'] > 0).sum())}", flush=True)
    _check_binning(a, W, H)
    try:
        _culling(False)
        b = _render(scene, cam, gi, ge, go)
    finally:
        _culling(True)
    for k in ('image', 'opacity', 'extras', 'n_contrib', 'point_list', 'ranges'):
        assert torch.equal(a[k], b[k]), f"{k} depends on the culling"
    for k in ('g_colors', 'g_trans', 'g_normal_opacity', 'g_means3D', 'g_scales', 'g_rot', 'g_opac', 'g_shs'):
        ref = b[k].abs().max().clamp_min(1e-30)
        assert float((a[k] - b[k]).abs().max() / ref) < 2e-5, k

    # per-surfel sums through per-instance records (default) == device-scope atomics
    # ... and gathering from the packed per-surfel records (default) == gathering from the four tensors
    d = _render(scene, cam, gi, ge, go, ordered_sums=False, packed=False)
    for k in ('image', 'opacity', 'extras', 'n_contrib'):
        assert torch.equal(a[k], d[k]), f"{k} depends on the packed records"
    for k in ('g_colors', 'g_trans', 'g_normal_opacity', 'g_means2D', 'g_means3D', 'g_scales', 'g_rot', 'g_opac', 'g_shs'):
        ref = a[k].abs().max().clamp_min(1e-30)
        assert float((a[k] - d[k]).abs().max() / ref) < 2e-5, k

    # lists without the instances that no pixel of their tile can blend (what _GS_2D_Render uses)
    # == the reference's full lists: maps bit for bit, gradients to the rounding of a different grouping of the sums
    e = _render(scene, cam, gi, ge, go, cull=True)
    n_full, n_cull = int((a['ranges'][:, 1] - a['ranges'][:, 0]).sum()), int((e['ranges'][:, 1] - e['ranges'][:, 0]).sum())
    print(f"[full {config}] instances in the tile lists {n_full} -> {n_cull}", flush=True)
    assert n_cull < n_full
    for k in ('image', 'opacity', 'extras'):
        assert torch.equal(a[k], e[k]), f"{k} depends on the culled lists"
    for k in ('g_colors', 'g_trans', 'g_normal_opacity', 'g_means2D', 'g_means3D', 'g_scales', 'g_rot', 'g_opac', 'g_shs'):
        ref = a[k].abs().max().clamp_min(1e-30)
        assert float((a[k] - e[k]).abs().max() / ref) < 2e-5, k
    del e

    # accumulated blend weights == opacity image (both are the sum of alpha * T over blended pairs)
    acc = torch.zeros(scene.P, device=device)
    get_C_function('GS_2D_render_forward')(W, H, a['means2D'], a['colors'], a['normal_opacity'], a['trans_mat'],
                                           a['point_list'], a['ranges'], cam.near, cam.far, False, None, None, acc, None)
    torch.cuda.synchronize()
    tot_w, tot_o = float(acc.double().sum()), float(a['opacity'].double().sum())
    assert abs(tot_w - tot_o) < 1e-4 * tot_o

    # linearity of the backward in the upstream gradients
    c = _render(scene, cam, 2.0 * gi, 2.0 * ge, 2.0 * go)
    for k in ('g_colors', 'g_trans', 'g_normal_opacity', 'g_means3D', 'g_shs'):
        ref = a[k].abs().max().clamp_min(1e-30)
        assert float((c[k] - 2.0 * a[k]).abs().max() / ref) < 2e-5, k


def test_knn_3m_by_2048_k8(device):
    from fast_sp_gs_amd._C import get_C_function
    g = torch.Generator().manual_seed(4)
    N, M, K = 3_000_000, 2048, 8
    x = torch.randn(N, 3, generator=g).to(device)
    y = torch.randn(M, 3, generator=g).to(device)
    print(f"[full knn] {N} x {M}, k={K}", flush=True)
    d2, idx = get_C_function('knn_topk')(x, y, K)
    torch.cuda.synchronize()
    assert idx.dtype == torch.int64 and int(idx.min()) >= 0 and int(idx.max()) < M
    assert bool((d2[:, 1:] >= d2[:, :-1]).all())
    re = ((x[:, None, :] - y[idx]) ** 2).sum(-1)
    assert float((re - d2).abs().max()) < 1e-5 * float(d2.max())
    assert bool((idx.sort(dim=1).values[:, 1:] != idx.sort(dim=1).values[:, :-1]).all())  # k distinct neighbours
    sample = torch.randint(0, N, (4096,), generator=g).to(device)
    full = torch.cdist(x[sample], y) ** 2
    kth = full.topk(K, dim=1, largest=False).values
    assert float((kth - d2[sample]).abs().max()) < 1e-4 * float(kth.max())
    # all 3M queries against the oracle's all-pairs search (6.1e9 distances): indices and distances bit for bit
    import oracle as O
    rd, ri = np.zeros((N, K), np.float32), np.zeros((N, K), np.int64)
    O.call("knn_topk_f32", N, M, 3, K, x.cpu().numpy(), y.cpu().numpy(), rd, ri)
    assert np.array_equal(idx.cpu().numpy(), ri) and np.array_equal(d2.cpu().numpy(), rd)


@pytest.mark.parametrize("per_splat", [False, True])
def test_fast_path_properties_at_300k_800(per_splat, device):
    """The fast path at the benchmark size: culling off == on (forward bit for bit, gradients to the rounding of
    reordered sums), ordered per-instance sums == atomics, the backward linear in the upstream gradients, and the two
    backward algorithms (per pixel / per 32-entry bucket from the forward's snapshots) agreeing with each other."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.renderer import fast_render_step
    scene_h, cam_h = scenes.config2()
    W, H = cam_h.W, cam_h.H
    g = torch.Generator().manual_seed(13)
    gi, ge, go = torch.randn(3, H, W, generator=g).to(device), torch.randn(8, H, W, generator=g).to(device), \
        torch.randn(H, W, generator=g).to(device)
    scene, cam = scene_h.to(device), cam_h.to(device)
    print(f"[full fast per_splat={per_splat}] P={scene.P} {W}x{H}", flush=True)
    grads = ('g_colors', 'g_means2D_blend', 'g_trans', 'g_inv', 'g_normal_opacity', 'g_means3D', 'g_scales',
             'g_rotations', 'g_opacities', 'g_shs')

    def close(x, y, tol, what):
        for k in grads:
            ref = x[k].abs().max().clamp_min(1e-30)
            assert float((x[k] - y[k]).abs().max() / ref) < tol, (what, k)

    a = fast_render_step(scene, cam, gi, ge, go, per_splat=per_splat)
    torch.cuda.synchronize()
    print(f"[full fast] R={a['point_list'].numel()}", flush=True)
    assert all(bool(torch.isfinite(a[k]).all()) for k in grads)
    try:
        _culling(False)
        b = fast_render_step(scene, cam, gi, ge, go, per_splat=per_splat)
        torch.cuda.synchronize()
    finally:
        _culling(True)
    for k in ('image', 'opacity', 'extras', 'n_contrib', 'point_list', 'ranges'):
        assert torch.equal(a[k], b[k]), f"{k} depends on the culling"
    close(a, b, 2e-5, 'culling')
    # the ordered sum with the corner test repeated instead of read from the preprocess kernel's keep masks: the same
    # records in the same order, bit for bit
    m = fast_render_step(scene, cam, gi, ge, go, per_splat=per_splat, reuse_masks=False)
    for k in grads:
        assert torch.equal(a[k], m[k]), ('keep masks', k)
    del m
    # (the atomics add in arrival order; the fast preprocess backward amplifies that rounding in dL/dscales)
    close(a, fast_render_step(scene, cam, gi, ge, go, per_splat=per_splat, ordered_sums=False), 1e-4, 'atomic sums')
    c = fast_render_step(scene, cam, 2.0 * gi, 2.0 * ge, 2.0 * go, per_splat=per_splat)
    for k in grads:
        ref = a[k].abs().max().clamp_min(1e-30)
        assert float((c[k] - 2.0 * a[k]).abs().max() / ref) < 2e-5, ('linearity', k)
    if per_splat:
        # The bucketed backward restarts from the forward's snapshots: same gradients up to their rounding, for the
        # upstream channels both algorithms define alike (the per-pixel one differentiates the distortion map, channel 5,
        # the bucketed one takes channels 6 and 7, the two depth moments, as plain linear outputs).
        ge_c = ge.clone()
        ge_c[5:] = 0
        close(fast_render_step(scene, cam, gi, ge_c, go, per_splat=True),
              fast_render_step(scene, cam, gi, ge_c, go, per_splat=False), 2e-4, 'per-pixel backward')


def test_gs3d_path_properties_at_300k_800(device):
    """The 3D-Gaussian path at the benchmark size (the benchmark's centres with a third scale): culling off == on,
    culled tile lists == the reference's lists, ordered per-instance sums == atomics, blend weights summing to the opacity image, linearity of the backward."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    scene_h, cam_h = scenes.config2()
    scene, cam = scene_h.to(device), cam_h.to(device)
    W, H = cam.W, cam.H
    g = torch.Generator().manual_seed(11)
    scales = torch.cat([scene_h.scales, scene_h.scales[:, :1] * (0.5 + torch.rand(scene.P, 1, generator=g))],
                       1).to(device).contiguous()
    gi, go = torch.randn(3, H, W, generator=g).to(device), torch.randn(H, W, generator=g).to(device)
    tan_fov = (W / 2 / float(cam.Tv2s[0, 0]), H / 2 / float(cam.Tv2s[1, 1]))
    print(f"[full gs3d] P={scene.P} {W}x{H}", flush=True)

    def step(gi, go, ordered, cull=False):
        m2, dep, col, rad, tt, c3, co = f('gs_preprocess_forward')(
            W, H, 3, False, scene.means3D, scales, scene.rotations, scene.opacities, scene.shs, None, cam.Tw2v,
            cam.Tv2c, cam.campos, tan_fov, None, None, None, None)
        keep = f('gs_cull_masks')(W, H, m2, co, rad) if cull else None
        ranges, pl, offsets = f('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True, cull=cull,
                                              keep_masks=keep)[:3]
        oc, oo, _, nc = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges)
        g_col, _, g_m2, g_co = f('gaussian_rasterize_backward')(m2, co, col, None, oo, gi, go, None, ranges, pl, nc,
                                                                offsets if ordered else None, rad if ordered else None,
                                                                culled=keep if ordered else None)
        g3, gs, gq = torch.empty_like(scene.means3D), torch.empty_like(scales), torch.empty_like(scene.rotations)
        gop, gsh = torch.empty_like(scene.opacities), torch.empty_like(scene.shs)
        f('gs_preprocess_backward')(W, H, 3, False, scene.means3D, scales, scene.rotations, scene.opacities, scene.shs,
                                    None, cam.Tw2v, cam.Tv2c, cam.campos, tan_fov, c3, None, rad, col, g_m2.clone(), None,
                                    g_col, g_co, g3, gs, gq, gop, gsh, None, None)
        torch.cuda.synchronize()
        return dict(image=oc, opacity=oo, n_contrib=nc, point_list=pl, ranges=ranges, m2=m2, co=co, col=col,
                    g_col=g_col, g_m2=g_m2, g_co=g_co, g3=g3, gs=gs, gq=gq, gop=gop, gsh=gsh)

    grads = ('g_col', 'g_m2', 'g_co', 'g3', 'gs', 'gq', 'gop', 'gsh')

    def close(x, y, tol, what, scale=1.0):
        for k in grads:
            ref = x[k].abs().max().clamp_min(1e-30)
            assert float((y[k] - scale * x[k]).abs().max() / ref) < tol, (what, k)

    a = step(gi, go, True)
    print(f"[full gs3d] R={a['point_list'].numel()}", flush=True)
    assert all(bool(torch.isfinite(a[k]).all()) for k in grads)
    try:
        _culling(False)
        b = step(gi, go, True)
    finally:
        _culling(True)
    for k in ('image', 'opacity', 'n_contrib', 'point_list', 'ranges'):
        assert torch.equal(a[k], b[k]), f"{k} depends on the culling"
    close(a, b, 2e-5, 'culling')
    close(a, step(gi, go, False), 1e-4, 'atomic sums')
    close(a, step(2.0 * gi, 2.0 * go, True), 2e-5, 'linearity', 2.0)
    # lists without the instances that no pixel of their tile can blend (what RasterizeGaussians bins)
    for ordered in (True, False):
        e = step(gi, go, ordered, cull=True)
        n_full, n_cull = int((a['ranges'][:, 1] - a['ranges'][:, 0]).sum()), int((e['ranges'][:, 1] - e['ranges'][:, 0]).sum())
        print(f"[full gs3d] instances in the tile lists {n_full} -> {n_cull}", flush=True)
        assert n_cull < n_full
        for k in ('image', 'opacity'):
            assert torch.equal(a[k], e[k]), f"{k} depends on the culled lists"
        close(a, e, 2e-5 if ordered else 1e-4, 'culled lists')
    acc = torch.zeros(scene.P, device=device)
    f('gaussian_rasterize_forward')(W, H, a['m2'], a['co'], a['col'], None, a['point_list'], a['ranges'], None, acc, None)
    torch.cuda.synchronize()
    tot_w, tot_o = float(acc.double().sum()), float(a['opacity'].double().sum())
    assert abs(tot_w - tot_o) < 1e-4 * tot_o
