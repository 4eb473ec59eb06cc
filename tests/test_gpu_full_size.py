"""Full-size checks of the render path through size-independent properties (the oracle takes minutes at these sizes):
  * the per-quadrant culling of the blend kernels is exact: with it switched off (every staged surfel evaluated at every
    pixel, as the reference does) the forward outputs are identical bit for bit and the gradients agree to the rounding
    of the reordered atomic sums;
  * binning invariants: sorted masked keys, ranges partition [0, R) in tile order, every entry carries its tile's id;
  * the blend weights accumulated per surfel sum to the opacity image;
  * the backward is linear in the upstream gradients, and its two ways of summing a surfel's gradient over tiles
    (per-instance records summed in order / device-scope atomics) agree;
  * K-NN at 3M x 2048, k = 8: distances ascending, equal to the distance recomputed from the returned index, and no
    closer control point exists for a sample of queries (brute force with torch).
Sizes: 300 000 surfels at 800x800, 3 000 000 surfels at 1352x1014 (one view), 400 000 surfels at 3840x2160.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _culling(enabled):
    from fast_sp_gs_amd import lib
    lib.check(lib.load().fsgs_debug_set_culling(int(enabled)), 'debug_set_culling')


def _render(scene, cam, gi, ge, go, ordered_sums=True, packed=True):
    from fast_sp_gs_amd.renderer import render_step
    out = render_step(scene, cam, gi, ge, go, ordered_sums=ordered_sums, packed=packed)
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


@pytest.mark.parametrize("config", ["c2_300k_800", "c4_3m_1352x1014", "uhd_400k_3840x2160"])
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
        cam_h = cams[1]
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
