"""GPU parity of the "fast" surfel path (intrinsics transform + adjugate -> fused corner-test binning -> blend
forward/backward in both channel sets -> preprocess backward) against the CPU oracle, stage by stage, on the same seeded
inputs. Every stage is fed the GPU's own upstream outputs so integer results are compared on identical float inputs.

Tolerances: images 1e-4 abs, gradients 1e-3 rel (max|d|/max|ref|), bit-exact geometry / keys / ranges / point lists
(including the -1 padding entries). Float results of the blend are compared with the oracle evaluated in float64 on
the GPU's float32 inputs; at most max(2, 1e-5 * H * W) pixels may sit on the other side of the 1/255 or T < 1e-4
thresholds (their n_contrib differs) and every other pixel must hold the tolerance (see test_gpu_render_parity.py).
"""
import numpy as np
import pytest
import torch

from util import abs_err, check_blend_forward, check_blend_gradients, f64, npy, rel_err

pytestmark = pytest.mark.gpu

CASES = {
    "c0_10k_256": (10_000, 256, 256, 1.0),
    "partial_tiles_511x127": (4_000, 511, 127, 1.0),
    "big_surfels_96x80": (300, 96, 80, 10.0),  # rectangles of more than 32 tiles: wave-cooperative emission
    "dense_6k_96": (6_000, 96, 96, 12.0),  # tile lists longer than one 256-entry batch, many 32-entry buckets
    "tiny_3_surfels": (3, 40, 24, 1.0),
    "c2_300k_800": (300_000, 800, 800, 1.0),  # the benchmark's scene at full size
}


def _make(name):
    from fast_sp_gs_amd import scenes
    P, W, H, scale_mul = CASES[name]
    if name.startswith("c2_"):
        scene, cam = scenes.config2(P=P, size=W, seed=0)
    else:
        scene, _ = scenes.config0(P=P, size=max(W, H), seed=0)
        scene.scales = scene.scales * scale_mul
        cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.3, -0.2, 4.0]))  # off-axis: x/y translation in the view matrix
    g = torch.Generator().manual_seed(7)
    gi = torch.randn(3, H, W, generator=g)
    ge = torch.randn(8, H, W, generator=g)
    go = torch.randn(H, W, generator=g)
    return scene, cam, gi, ge, go


@pytest.mark.parametrize("per_splat", [False, True])
@pytest.mark.parametrize("name", list(CASES))
def test_fast_path_stage_by_stage(name, per_splat, device, oracle_mod):
    from fast_sp_gs_amd.renderer import fast_render_step
    O = oracle_mod
    scene, cam, gi, ge, go = _make(name)
    W, H = cam.W, cam.H
    print(f"[fast {name} per_splat={per_splat}] P={scene.P} {W}x{H}", flush=True)
    out = fast_render_step(scene.to(device), cam.to(device), gi.to(device), ge.to(device), go.to(device),
                           per_splat=per_splat)
    torch.cuda.synchronize()
    g = {k: npy(v) for k, v in out.items()}
    s = dict(means3D=npy(scene.means3D), scales=npy(scene.scales), rotations=npy(scene.rotations),
             opacities=npy(scene.opacities), shs=npy(scene.shs), Tw2v=npy(cam.Tw2v), Tv2s=npy(cam.Tv2s),
             campos=npy(cam.campos))

    # --- preprocess forward: geometry and adjugate bit-exact, colours to rounding
    m2, colors, tm, im, no, dep, radii, tt = O.fast_preprocess_forward(
        W, H, 3, s['means3D'], s['scales'], s['rotations'], s['opacities'], s['shs'], None, s['Tw2v'], s['Tv2s'],
        s['campos'])
    for k, ref in (('radii', radii), ('tiles_touched', tt), ('means2D', m2), ('trans_mat', tm), ('inverse_m', im),
                   ('depths', dep), ('normal_opacity', no)):
        assert np.array_equal(g[k], ref), k
    assert abs_err(g['colors'], colors) < 2e-6

    # --- fused binning on the GPU's own preprocess outputs: bit-exact, padding included
    ranges, pl, keys = O.fast_prepare(W, H, g['means2D'], g['inverse_m'], g['depths'], s['opacities'], g['radii'],
                                      g['tiles_touched'], return_keys=True)
    assert g['point_list'].shape == pl.shape
    assert np.array_equal(g['ranges'], ranges)
    assert np.array_equal(g['point_list'], pl)
    assert np.array_equal(g['keys'], keys)
    n_pad = int((pl == -1).sum())
    print(f"[fast {name}] R={pl.size} of which padding {n_pad}", flush=True)

    # --- blend forward on the GPU's own inputs, against the oracle in float64 on those float32 values
    offset = g.get('bucket_offset')
    d64 = {k: f64(g[k]) for k in ('means2D', 'colors', 'normal_opacity', 'trans_mat', 'inverse_m', 'opacity', 'extras')}
    ref_f = O.fast_render_forward(W, H, cam.near, cam.far, False, d64['means2D'], d64['colors'], d64['normal_opacity'],
                                  d64['trans_mat'], d64['inverse_m'], g['point_list'], g['ranges'], offset)
    oc, oo, oe, nc = ref_f[:4]
    def forward32():
        f32 = lambda k: g[k].astype(np.float32)
        r = O.fast_render_forward(W, H, cam.near, cam.far, False, f32('means2D'), f32('colors'), f32('normal_opacity'),
                                  f32('trans_mat'), f32('inverse_m'), g['point_list'], g['ranges'], offset)
        return r[0], r[1], r[2], r[3]

    flip = check_blend_forward(f"fast {name}", (g['image'], g['opacity'], g['extras'][:8], g['n_contrib']),
                               (oc, oo, oe[:8], nc), forward32, max(2, int(1e-5 * H * W)))

    if per_splat:
        # snapshots: compared where the oracle wrote them (a written transmittance is always >= 1e-4 > 0)
        max_c, b2t, sT, sacc, saux = ref_f[4:9]
        assert np.array_equal(g['bucket_to_tile'], b2t)
        assert (g['max_contrib'].reshape(-1) != max_c).sum() <= flip.sum()
        wrote = sT > 0
        assert wrote.any() or pl.size == n_pad
        tol = lambda a, b: np.abs(a.astype(np.float64) - b) > 1e-4 + 1e-3 * np.abs(b)
        bad = int((tol(g['sampled_T'], sT) & wrote).sum())
        for c in range(3):
            bad += int((tol(g['sampled_acc'][:, c], sacc[:, c]) & wrote).sum())
        for c in (0, 1, 2, 3, 5, 6, 7):
            bad += int((tol(g['sampled_aux'][:, c], saux[:, c]) & wrote).sum())
        print(f"[fast {name}] snapshot entries {int(wrote.sum())}, out of tolerance {bad}", flush=True)
        assert bad <= 32 * 11 * int(flip.sum())  # a flipped pixel moves its later snapshots

    # --- blend backward on the GPU's own forward outputs
    gc, gm, gt, ginv, gn = O.fast_render_backward(
        cam.near, cam.far, int(per_splat), d64['means2D'], d64['normal_opacity'], d64['colors'], d64['trans_mat'],
        d64['inverse_m'], d64['opacity'], d64['extras'], f64(npy(gi)), f64(npy(go)), f64(npy(ge)), g['ranges'],
        g['point_list'], g['n_contrib'])
    def backward32():
        f32 = lambda a: np.asarray(a, np.float32)
        r = O.fast_render_backward(
            cam.near, cam.far, int(per_splat), f32(d64['means2D']), f32(d64['normal_opacity']), f32(d64['colors']),
            f32(d64['trans_mat']), f32(d64['inverse_m']), f32(d64['opacity']), f32(d64['extras']), npy(gi), npy(go),
            npy(ge), g['ranges'], g['point_list'], g['n_contrib'])
        return dict(colors=r[0], means2D=r[1], trans=r[2], inv=r[3], normal_opacity=r[4])

    check_blend_gradients(f"fast {name} blend backward",
                          dict(colors=g['g_colors'], trans=g['g_trans'], inv=g['g_inv'],
                               normal_opacity=g['g_normal_opacity'], means2D=g['g_means2D_blend']),
                          dict(colors=gc, trans=gt, inv=ginv, normal_opacity=gn, means2D=gm), backward32)
    assert np.abs(g['g_trans'][:, :2]).max() == 0  # only the depth row of the transform receives gradient here

    # --- preprocess backward on the GPU's own blend gradients
    g3, gs, gr, gop, gsh, _, gm2_after = O.fast_preprocess_backward(
        W, H, 3, s['means3D'], s['scales'], s['rotations'], s['shs'], None, s['Tw2v'], s['Tv2s'], s['campos'],
        g['trans_mat'], g['radii'], g['colors'], g['g_means2D_blend'], g['g_trans'], g['g_inv'], g['g_colors'],
        g['g_normal_opacity'])
    errs = dict(means3D=rel_err(g['g_means3D'], g3), scales=rel_err(g['g_scales'], gs),
                rot=rel_err(g['g_rotations'], gr), opac=rel_err(g['g_opacities'], gop), shs=rel_err(g['g_shs'], gsh),
                mean2D_proxy=rel_err(g['g_means2D_proxy'], gm2_after))
    print(f"[fast {name}] preprocess backward rel errs {errs}", flush=True)
    for k, v in errs.items():
        assert v < 1e-5, k


def test_fast_transmat_ops(device, oracle_mod):
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    scene, cam, *_ = _make("tiny_3_surfels")
    from fast_sp_gs_amd import scenes
    scene, _ = scenes.config0(P=5000, size=64, seed=4)
    sd, cd = scene.to(device), cam.to(device)
    tm, nrm = get_C_function('gs_2d_fast_compute_transmat_forward')(sd.means3D, sd.scales, sd.rotations, cd.Tw2v,
                                                                    cd.Tv2s)
    P = scene.P
    rtm, rn = np.zeros((P, 3, 3), np.float32), np.zeros((P, 3), np.float32)
    a = [npy(scene.means3D), npy(scene.scales), npy(scene.rotations), npy(cam.Tw2v), npy(cam.Tv2s)]
    assert O.call("gs_2d_fast_compute_transmat_forward_f32", P, *a, rtm, rn) == 0
    assert np.array_equal(npy(tm), rtm) and np.array_equal(npy(nrm), rn)
    g = torch.Generator().manual_seed(1)
    gM, gN = torch.randn(P, 3, 3, generator=g), torch.randn(P, 3, generator=g)
    outs = get_C_function('gs_2d_fast_compute_trans_mat_backward')(sd.means3D, sd.scales, sd.rotations, cd.Tw2v,
                                                                   cd.Tv2s, gM.to(device), gN.to(device))
    ref = [np.zeros((P, 3), np.float32), np.zeros((P, 2), np.float32), np.zeros((P, 4), np.float32)]
    assert O.call("gs_2d_fast_compute_transmat_backward_f32", P, *a, npy(gM), npy(gN), *ref) == 0
    for o, r in zip(outs, ref):
        assert np.array_equal(npy(o), r)


def test_fast_autograd_wrapper_and_accum(device):
    """GS_2D_fast_render (autograd) reproduces the raw-operator step, and the accumulated blend weights sum to the
    opacity image (both are the sum of alpha * T over all blended pairs)."""
    from fast_sp_gs_amd.renderer import GS_2D_fast_render, fast_render_step
    scene, cam, gi, ge, go = _make("c0_10k_256")
    sd, cd = scene.to(device), cam.to(device)
    leaves = [t.clone().requires_grad_(True) for t in (sd.means3D, sd.scales, sd.rotations, sd.opacities, sd.shs)]
    acc_p = torch.zeros(scene.P, device=device)
    acc_n = torch.zeros(scene.P, dtype=torch.int32, device=device)
    acc_m = torch.zeros(scene.P, dtype=torch.int32, device=device)
    out = GS_2D_fast_render(leaves[0], leaves[1], leaves[2], leaves[3], (cam.W, cam.H), cd.Tw2v, cd.Tv2c, cd.Tv2s,
                            campos=cd.campos, near=cam.near, far=cam.far, sh_degree=3, sh_features=leaves[4],
                            accum_max_count=acc_m, accum_weights_p=acc_p, accum_weights_count=acc_n)
    (out['images'] * gi.to(device)).sum().backward()
    raw = fast_render_step(sd, cd, gi.to(device), None, None)
    torch.cuda.synchronize()
    assert abs_err(npy(out['images']), npy(raw['image'])) < 1e-6
    for leaf, k in zip(leaves, ('g_means3D', 'g_scales', 'g_rotations', 'g_opacities', 'g_shs')):
        assert rel_err(npy(leaf.grad), npy(raw[k])) < 1e-4, k  # atomics reorder float sums between the two runs
    assert rel_err(npy(out['viewspace_points'].grad), npy(raw['g_means2D_proxy'])) < 1e-4
    tot_w, tot_o = float(acc_p.double().sum()), float(out['opacity'].detach().double().sum())
    assert abs(tot_w - tot_o) < 1e-4 * tot_o
    assert int(acc_n.sum()) > 0 and int(acc_m.sum()) > 0
    assert int(acc_n.sum()) >= int((raw['n_contrib'][0] > 0).sum())


@pytest.mark.parametrize("per_splat", [False, True])
@pytest.mark.parametrize("name", ["partial_tiles_511x127", "dense_6k_96"])
def test_fast_ordered_sums_match_the_atomic_sums(name, per_splat, device):
    """The blend backward's per-surfel sums through per-(surfel, tile) records added in a fixed order (what
    fast_render_step does by default, and what the stage-by-stage test holds to the oracle) against the reference's way,
    device-scope atomics into zero-filled outputs: equal up to the order of the additions, identical from run to run,
    every row assigned (the record path's outputs are not zero-filled), rows 0 and 1 of dL/dtrans_mat zeros."""
    from fast_sp_gs_amd.renderer import fast_render_step
    scene, cam, gi, ge, go = _make(name)
    args = (scene.to(device), cam.to(device), gi.to(device), ge.to(device), go.to(device))
    a = fast_render_step(*args, per_splat=per_splat)
    b = fast_render_step(*args, per_splat=per_splat)
    c = fast_render_step(*args, per_splat=per_splat, ordered_sums=False)
    torch.cuda.synchronize()
    hidden = a['radii'] <= 0
    assert int(hidden.sum()) < scene.P and (name != 'partial_tiles_511x127' or int(hidden.sum()) > 0)
    for k in ('g_colors', 'g_means2D_blend', 'g_trans', 'g_inv', 'g_normal_opacity', 'g_means3D', 'g_scales',
              'g_rotations', 'g_opacities', 'g_shs'):
        assert torch.equal(a[k], b[k]) and bool(torch.isfinite(a[k]).all()), k
        ref = float(c[k].abs().max())
        assert ref > 0 and float((a[k] - c[k]).abs().max()) <= 5e-5 * ref, k  # the atomics add in any order
        if k in ('g_colors', 'g_means2D_blend', 'g_trans', 'g_inv', 'g_normal_opacity'):
            assert not a[k][hidden].any(), k
    assert not a['g_trans'][:, :2].any() and a['g_trans'][:, 2].any()


@pytest.mark.parametrize("ordered", [True, False])
@pytest.mark.parametrize("name", ["partial_tiles_511x127", "dense_6k_96", "big_surfels_96x80"])
def test_fast_image_only_backward(name, ordered, device):
    """Without gradients of the auxiliary maps the backward runs its image-only instantiation (no depth terms, the
    projected-centre pairs' means2D sums on their own path). Its results against the full instantiation fed zeros for
    those gradients, which the stage-by-stage test holds to the oracle: the same sums up to rounding."""
    from fast_sp_gs_amd.renderer import fast_render_step
    scene, cam, gi, _, _ = _make(name)
    sc, cm, gi = scene.to(device), cam.to(device), gi.to(device)
    lean = fast_render_step(sc, cm, gi, ordered_sums=ordered)
    full = fast_render_step(sc, cm, gi, torch.zeros(8, cam.H, cam.W, device=device),
                            torch.zeros(cam.H, cam.W, device=device), ordered_sums=ordered)
    torch.cuda.synchronize()
    assert float(full['g_means2D_blend'].abs().max()) > 0  # some pair is met by its projected centre
    for k in ('g_colors', 'g_means2D_blend', 'g_inv', 'g_normal_opacity', 'g_means3D', 'g_scales', 'g_rotations',
              'g_opacities', 'g_shs'):
        ref = float(full[k].abs().max())
        err = float((lean[k] - full[k]).abs().max())
        print(f"[fast image-only {name} ordered={ordered}] {k}: max {ref:.3e} diff {err:.3e}", flush=True)
        assert bool(torch.isfinite(lean[k]).all()) and err <= 2e-5 * max(ref, 1e-30), k
    assert not lean['g_trans'].any()  # the third row only carries depth gradients


@pytest.mark.parametrize("ordered", [True, False])
@pytest.mark.parametrize("name", ["c0_10k_256", "partial_tiles_511x127", "big_surfels_96x80", "dense_6k_96",
                                  "tiny_3_surfels", "c2_300k_800"])
def test_fast_per_splat_kernel(name, ordered, device):
    """The reference's per-splat decomposition (one lane per list entry, pixels handed from lane to lane, restart from
    the forward's snapshots) against the back-to-front kernel with the same channel set, which the stage-by-stage test
    holds to the oracle: the same derivative summed in another order (front to back instead of back to front)."""
    from fast_sp_gs_amd.renderer import fast_render_step
    scene, cam, gi, ge, go = _make(name)
    args = (scene.to(device), cam.to(device), gi.to(device), ge.to(device), go.to(device))
    tile = fast_render_step(*args, per_splat=True, ordered_sums=ordered)
    splat = fast_render_step(*args, per_splat=True, ordered_sums=ordered, per_splat_kernel=True)
    torch.cuda.synchronize()
    errs = {}
    for k in ('g_colors', 'g_means2D_blend', 'g_trans', 'g_inv', 'g_normal_opacity', 'g_means3D', 'g_scales',
              'g_rotations', 'g_opacities', 'g_shs'):
        assert bool(torch.isfinite(splat[k]).all()), k
        errs[k] = rel_err(npy(splat[k]), npy(tile[k]))
    print(f"[fast per-splat kernel {name} ordered={ordered}] rel errs {errs}", flush=True)
    assert name.startswith('tiny') or (float(tile['g_inv'].abs().max()) > 0 and float(tile['g_trans'].abs().max()) > 0)
    for k, v in errs.items():
        assert v < 1e-3, k
    if ordered:  # fixed order of the additions: identical from run to run
        again = fast_render_step(*args, per_splat=True, per_splat_kernel=True)
        for k in ('g_colors', 'g_means2D_blend', 'g_trans', 'g_inv', 'g_normal_opacity'):
            assert torch.equal(again[k], splat[k]), k


@pytest.mark.parametrize("layout", ["full", "split", "wide"])
def test_fast_preprocess_backward_assigns_every_row(layout, device):
    """gs_2d_fast_preprocess_backward writes every row of its geometry gradients and of a fully active SH gradient
    (zeros for surfels that were not rendered): outputs poisoned with NaN come out equal to outputs that started from
    zeros. With unused higher coefficients ("wide") or a split DC / rest layout the wrapper still starts from zeros."""
    from fast_sp_gs_amd._C import get_C_function as f
    from fast_sp_gs_amd.renderer import fast_render_step
    from fast_sp_gs_amd.renderer.gs_2d_fast_render import _grad_buffers
    scene, cam, gi, ge, go = _make("partial_tiles_511x127")
    sc, cm = scene.to(device), cam.to(device)
    out = fast_render_step(sc, cm, gi.to(device), ge.to(device), go.to(device))
    hidden = out['radii'] <= 0
    assert 0 < int(hidden.sum()) < scene.P
    shs, rest, degree = sc.shs, None, 3
    if layout == "split":
        shs, rest = sc.shs[:, :1].contiguous(), sc.shs[:, 1:].contiguous()
    elif layout == "wide":
        degree = 2
    W, H = cam.W, cam.H

    def run(poison):
        bufs = list(_grad_buffers(sc.means3D, sc.scales, sc.rotations, sc.opacities, shs, rest, degree, True, True))
        expect_assigned = [True, True, True, True, layout == "full", False]
        for b, assigned in zip(bufs, expect_assigned):
            if b is None:
                continue
            if poison and assigned:
                b.fill_(float('nan'))
            elif not assigned:
                assert not b.any()  # the wrapper's own zeros
        gm2 = out['g_means2D_blend'].clone()
        f('gs_2d_fast_preprocess_backward')(
            W, H, degree, False, sc.means3D, sc.scales, sc.rotations, sc.opacities, shs, rest, cm.Tw2v, cm.Tv2s,
            cm.campos, out['trans_mat'], out['radii'], out['colors'], out['normal_opacity'], gm2, out['g_trans'],
            out['g_inv'], None, out['g_colors'], out['g_normal_opacity'], *bufs)
        return bufs

    a, b = run(False), run(True)
    torch.cuda.synchronize()
    for x, y in zip(a, b):
        if x is None:
            continue
        assert bool(torch.isfinite(y).all())
        assert torch.equal(x, y)
        assert not y[hidden].any()


@pytest.mark.parametrize("name", ["partial_tiles_511x127", "tiny_3_surfels"])
def test_fast_forward_writes_every_pixel(name, device):
    """The forward's outputs are allocated uninitialised: every pixel of every map is written by the tile's block, empty
    tiles and partial tiles included. The allocator's free blocks are poisoned with NaN / a large count first; the
    second call must reproduce the first bit for bit and hold no NaN."""
    from fast_sp_gs_amd.renderer import fast_render_step
    scene, cam, gi, ge, go = _make(name)
    args = (scene.to(device), cam.to(device), gi.to(device), ge.to(device), go.to(device))
    first = fast_render_step(*args, per_splat=True)
    keep = {k: first[k].clone() for k in ('image', 'opacity', 'extras', 'n_contrib')}
    del first
    H, W = cam.H, cam.W
    poison = [torch.full((3, H, W), float('nan'), device=device), torch.full((H, W), float('nan'), device=device),
              torch.full((8, H, W), float('nan'), device=device),
              torch.full((2, H, W), 1 << 30, dtype=torch.int32, device=device)]
    torch.cuda.synchronize()
    del poison
    again = fast_render_step(*args, per_splat=True)
    torch.cuda.synchronize()
    for k, v in keep.items():
        assert bool(torch.isfinite(again[k].float()).all()), k
        assert torch.equal(again[k], v), k
    assert int(again['n_contrib'].max()) < 1 << 30


@pytest.mark.parametrize("name", ["c0_10k_256", "partial_tiles_511x127", "big_surfels_96x80", "dense_6k_96"])
def test_fast_binning_per_tile_equals_device_wide_sort(name, device):
    """fsgs_gs_2d_fast_prepare_fill builds the lists per tile when its workspace has room for the per-tile counters and
    by the reference's device-wide sort of the padded key array otherwise: ranges, lists (padding tail included) and
    sorted keys are the same bit for bit (the stage-by-stage test holds the per-tile result to the oracle). The per-tile
    scheme with the corner test's verdicts read from the preprocess kernel's keep masks (what the operator does) and
    with the test repeated in both walks (no masks) give the same as well."""
    from fast_sp_gs_amd import lib as L
    from fast_sp_gs_amd._C import get_C_function as f
    lib = L.load()
    scene, cam, *_ = _make(name)
    sc, cm = scene.to(device), cam.to(device)
    W, H, P = cam.W, cam.H, scene.P
    (m2, colors, tm, im, no, depths, radii, ranges, point_list, keys, tt, offsets,
     masks) = f('gs_2d_fast_preprocess_forward')(
        W, H, 3, False, sc.means3D, sc.scales, sc.rotations, sc.opacities, sc.shs, None, cm.Tw2v, cm.Tv2c, cm.Tv2s,
        cm.campos, None, None, None, False, True, True, True)
    R = int(point_list.numel())
    small, large = lib.fsgs_gs_prepare_fill_workspace_bytes(R), lib.fsgs_gs_2d_fast_prepare_fill_workspace_bytes(P, W, H, R)
    assert large > small
    small_rects = (tt > 0) & (tt <= 32)
    assert int(small_rects.sum()) > 0 and int((masks[small_rects] != -1).sum()) > 0  # some tile of some rectangle fails
    results = []
    for nbytes, use_masks in ((small, False), (large, False), (large, True)):
        ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=device)
        rng = torch.full_like(ranges, -7)
        pl = torch.full((R,), -9, dtype=torch.int32, device=device)
        ks = torch.full((R,), -11, dtype=torch.int64, device=device)
        L.check(lib.fsgs_gs_2d_fast_prepare_fill(P, W, H, L.ptr(m2), L.ptr(im), L.ptr(depths), L.ptr(sc.opacities),
                                                 L.ptr(radii), L.ptr(offsets), R, L.ptr(rng), L.ptr(pl), L.ptr(ks),
                                                 L.ptr(ws), nbytes, L.ptr(masks) if use_masks else None,
                                                 L.current_stream()), 'fast_prepare_fill')
        torch.cuda.synchronize()
        results.append((rng, pl, ks))
    for other in (1, 2):
        for a, b, what in zip(results[0], results[other], ('ranges', 'point_list', 'keys')):
            assert torch.equal(a, b), (what, other)
    assert torch.equal(results[1][0], ranges) and torch.equal(results[1][1], point_list)
    assert int((point_list == -1).sum()) > 0


def test_fast_empty_scene(device):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.renderer import fast_render_step
    scene, cam = scenes.config0(P=64, size=64, seed=3)
    scene.means3D[:, 2] += 10.0
    out = fast_render_step(scene.to(device), cam.to(device), torch.zeros(3, 64, 64, device=device), per_splat=True)
    torch.cuda.synchronize()
    assert out['point_list'].numel() == 0 and out['bucket_to_tile'].numel() == 0
    assert int(out['radii'].abs().sum()) == 0 and int(out['ranges'].abs().sum()) == 0
    assert float(out['image'].abs().sum()) == 0 and float(out['g_means3D'].abs().sum()) == 0


@pytest.mark.parametrize("name", ["c0_10k_256", "partial_tiles_511x127", "dense_6k_96"])
def test_fast_flow_and_accum(name, device, oracle_mod):
    """Optical flow on the fast path (gs_2d_fast_redner.cu:141-150, 247-263, 494-510, 637-697, 765-782): out_flow divided
    by the final opacity, the 10-channel snapshots, both backward forms with dL/dflow, and the accum_* side outputs of
    the fast forward element by element."""
    from fast_sp_gs_amd._C import get_C_function as f
    from fast_sp_gs_amd.renderer import fast_render_step
    O = oracle_mod
    scene, cam, gi, ge, go = _make(name)
    W, H, P = cam.W, cam.H, scene.P
    sc, cm = scene.to(device), cam.to(device)
    out = fast_render_step(sc, cm, gi.to(device), ge.to(device), go.to(device), per_splat=True)
    gen = torch.Generator().manual_seed(23)
    means_t2 = (scene.means3D + 0.03 * torch.randn(P, 3, generator=gen)).to(device)
    t2, _ = f('gs_2d_fast_compute_transmat_forward')(means_t2, sc.scales, sc.rotations, cm.Tw2v, cm.Tv2s)
    gf = torch.randn(H, W, 2, generator=gen).to(device)
    amc = torch.zeros(P, dtype=torch.int32, device=device)
    awp = torch.zeros(P, device=device)
    awc = torch.zeros(P, dtype=torch.int32, device=device)
    args = (out['means2D'], out['colors'], out['normal_opacity'], out['trans_mat'], out['inverse_m'],
            out['point_list'], out['ranges'])
    offset = out['bucket_offset']
    res = f('GS_2D_fast_render_forward')(W, H, cam.near, cam.far, False, *args, t2, amc, awp, awc, offset)
    oc, oo, oe, of, nc, max_c, b2t, sT, sacc, saux = res
    torch.cuda.synchronize()
    assert of.shape == (H, W, 2) and saux.shape[1] == 10
    d64 = [f64(npy(t)) for t in args]
    r_amc, r_awp, r_awc = np.zeros(P, np.int32), np.zeros(P), np.zeros(P, np.int32)
    ref = O.fast_render_forward(W, H, cam.near, cam.far, False, *d64, npy(offset), f64(npy(t2)), r_amc, r_awp, r_awc)
    rc_, ro, re_, rnc, r_max, r_b2t, r_sT, r_sacc, r_saux, rf = ref
    flip = (npy(nc) != rnc).any(0)
    keep = ~flip
    n_flip = int(flip.sum())
    assert n_flip <= max(2, int(1e-5 * H * W))
    bad = (np.abs(npy(of).astype(np.float64) - rf) > 1e-4 + 1e-3 * np.abs(rf)).any(-1)
    print(f"[fast flow {name}] flow abs err {abs_err(npy(of)[keep], rf[keep]):.3e} (max |flow| {np.abs(rf).max():.2f}), "
          f"threshold-flip pixels {n_flip}", flush=True)
    assert np.abs(rf).max() > 0.5 and not (bad & keep).any()
    assert abs_err(npy(oc)[:, keep], rc_[:, keep]) < 1e-4
    # side outputs: exact counts (away from flipped pixels), weights to 1e-4 + 1e-5 rel
    if n_flip == 0:
        assert np.array_equal(npy(amc), r_amc) and np.array_equal(npy(awc), r_awc)
    else:
        assert np.abs(npy(awc) - r_awc).sum() <= 4 * n_flip and np.abs(npy(amc) - r_amc).sum() <= 8 * n_flip
    assert r_awc.sum() > 0 and (r_amc != r_awc).any() and int(npy(amc).sum()) == int(npy(awc).sum())
    assert (np.abs(npy(awp) - r_awp) <= 1e-4 + 1e-5 * np.abs(r_awp) + 1e-2 * n_flip).all()
    # snapshots of the two flow channels
    wrote = r_sT > 0
    tol = lambda a, b: np.abs(a.astype(np.float64) - b) > 1e-4 + 1e-3 * np.abs(b)
    bad = sum(int((tol(npy(saux)[:, c], r_saux[:, c]) & wrote).sum()) for c in (0, 1, 2, 3, 5, 6, 7, 8, 9))
    assert bad <= 32 * 9 * n_flip
    lens = npy(out['ranges'])[:, 1] - npy(out['ranges'])[:, 0]
    if name == "dense_6k_96":  # lists longer than one bucket: the flow channels of later snapshots are non-zero
        assert (lens > 64).any() and np.abs(r_saux[:, 8:] * wrote[:, None]).max() > 0

    # backward, both forms, all upstream gradients non-zero
    n64 = lambda t: f64(npy(t))
    for per_splat in (False, True):
        snap = (offset, b2t, max_c, sT, sacc, saux) if per_splat else (None,) * 6
        got = f('GS_2D_fast_render_backward')(
            out['means2D'], out['normal_opacity'], out['colors'], out['trans_mat'], out['inverse_m'], t2, oc, oo, oe,
            of, gi.to(device), go.to(device), ge.to(device), gf, out['ranges'], out['point_list'], nc, cam.near,
            cam.far, *snap)
        torch.cuda.synchronize()
        want = O.fast_render_backward(cam.near, cam.far, int(per_splat), d64[0], d64[2], d64[1], d64[3], d64[4],
                                      n64(oo), n64(oe), n64(gi), n64(go), n64(ge), npy(out['ranges']),
                                      npy(out['point_list']), npy(nc), f64(npy(t2)), n64(of), n64(gf))
        errs = {k: rel_err(npy(a), b)
                for k, a, b in zip(('colors', 'means2D', 'trans', 'inv', 'normal_opacity'), got, want)}
        print(f"[fast flow {name}] backward per_splat={per_splat} rel errs {errs}", flush=True)
        for k, v in errs.items():
            assert v < 1e-3, (k, per_splat)
        plain = O.fast_render_backward(cam.near, cam.far, int(per_splat), d64[0], d64[2], d64[1], d64[3], d64[4],
                                       n64(oo), n64(oe), n64(gi), n64(go), n64(ge), npy(out['ranges']),
                                       npy(out['point_list']), npy(nc))
        assert rel_err(plain[3], want[3]) > 1e-2  # the flow gradient is a visible part of the total
