"""GPU parity of the "fast" surfel path (intrinsics transform + adjugate -> fused corner-test binning -> blend
forward/backward in both channel sets -> preprocess backward) against the CPU oracle, stage by stage, on the same seeded
inputs. Every stage is fed the GPU's own upstream outputs so integer results are compared on identical float inputs.

Tolerances: images 1e-4 abs, gradients 1e-3 rel (max|d|/max|ref|), bit-exact geometry / keys / ranges / point lists
(including the -1 padding entries). At most max(2, 1e-5 * H * W) pixels may sit on the other side of the 1/255 or
T < 1e-4 thresholds (see test_gpu_render_parity.py).
"""
import numpy as np
import pytest
import torch

from util import abs_err, npy, rel_err

pytestmark = pytest.mark.gpu

CASES = {
    "c0_10k_256": (10_000, 256, 256, 1.0),
    "partial_tiles_511x127": (4_000, 511, 127, 1.0),
    "big_surfels_96x80": (300, 96, 80, 10.0),  # rectangles of more than 32 tiles: wave-cooperative emission
    "dense_6k_96": (6_000, 96, 96, 12.0),  # tile lists longer than one 256-entry batch, many 32-entry buckets
    "tiny_3_surfels": (3, 40, 24, 1.0),
}


def _make(name):
    from fast_sp_gs_amd import scenes
    P, W, H, scale_mul = CASES[name]
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

    # --- blend forward on the GPU's own inputs
    offset = g.get('bucket_offset')
    ref_f = O.fast_render_forward(W, H, cam.near, cam.far, False, g['means2D'], g['colors'], g['normal_opacity'],
                                  g['trans_mat'], g['inverse_m'], g['point_list'], g['ranges'], offset)
    oc, oo, oe, nc = ref_f[:4]
    flips = max(int((np.abs(g['image'] - oc) > 1e-4).any(0).sum()), int((np.abs(g['opacity'] - oo) > 1e-4).sum()))
    allowed = max(2, int(1e-5 * H * W))
    print(f"[fast {name}] image abs err {abs_err(g['image'], oc):.3e}, opacity {abs_err(g['opacity'], oo):.3e}, "
          f"threshold-flip pixels {flips} (allowed {allowed})", flush=True)
    assert flips <= allowed
    if flips == 0:
        assert abs_err(g['image'], oc) < 1e-4 and abs_err(g['opacity'], oo) < 1e-4
    for ch in range(8):
        bad = np.abs(g['extras'][ch].astype(np.float64) - oe[ch]) > 1e-4 + 1e-3 * np.abs(oe[ch])
        assert bad.sum() <= allowed, f"extras channel {ch}: {int(bad.sum())} pixels out of tolerance"
    assert (g['n_contrib'] != nc).any(0).sum() <= allowed

    if per_splat:
        # snapshots: compared where the oracle wrote them (a written transmittance is always >= 1e-4 > 0)
        max_c, b2t, sT, sacc, saux = ref_f[4:]
        assert np.array_equal(g['bucket_to_tile'], b2t)
        assert (g['max_contrib'].reshape(-1) != max_c).sum() <= allowed
        wrote = sT > 0
        assert wrote.any() or pl.size == n_pad
        tol = lambda a, b: np.abs(a.astype(np.float64) - b) > 1e-4 + 1e-3 * np.abs(b)
        bad = int((tol(g['sampled_T'], sT) & wrote).sum())
        for c in range(3):
            bad += int((tol(g['sampled_acc'][:, c], sacc[:, c]) & wrote).sum())
        for c in (0, 1, 2, 3, 5, 6, 7):
            bad += int((tol(g['sampled_aux'][:, c], saux[:, c]) & wrote).sum())
        print(f"[fast {name}] snapshot entries {int(wrote.sum())}, out of tolerance {bad}", flush=True)
        assert bad <= 32 * allowed

    # --- blend backward on the GPU's own forward outputs
    gc, gm, gt, ginv, gn = O.fast_render_backward(
        cam.near, cam.far, int(per_splat), g['means2D'], g['normal_opacity'], g['colors'], g['trans_mat'],
        g['inverse_m'], g['opacity'], g['extras'], npy(gi), npy(go), npy(ge), g['ranges'], g['point_list'],
        g['n_contrib'])
    errs = dict(colors=rel_err(g['g_colors'], gc), trans=rel_err(g['g_trans'], gt), inv=rel_err(g['g_inv'], ginv),
                normal_opacity=rel_err(g['g_normal_opacity'], gn), means2D=rel_err(g['g_means2D_blend'], gm))
    print(f"[fast {name}] blend backward rel errs {errs}", flush=True)
    for k, v in errs.items():
        assert v < 1e-3, k
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
