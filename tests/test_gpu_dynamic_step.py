"""The assembled training step of the dynamic superpoint scene (fast_sp_gs_amd/dynamic_step.py; reference:
fast_2d_gs/network.py:576-647, 700-730, gaussian_splatting.py:295-321, sparse_gaussian_adam.py:18-46):
  * at the benchmark's shape (200 000 surfels, 512 control points, K = 4, 800 x 800) two iterations run, the loss is
    finite, rows the visibility mask excludes keep their parameters and Adam moments bit for bit, visible rows move;
  * at a reduced size every autograd edge between the network's outputs and the loss (K-NN distances, neighbour
    weights, rigid warp, deformed parameters, background composite, L1 + D-SSIM) is compared with the same computation
    written in torch operators around the same renderer, whose own gradients are checked against the oracle elsewhere.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from util import npy, rel_err

pytestmark = pytest.mark.gpu


def _state(device, P, M, size, seed, **kw):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.dynamic_step import DynamicStep
    scene, cam = scenes.config2(P=P, size=size, seed=seed)
    g = torch.Generator().manual_seed(seed)
    ctrl = (torch.rand(M, 3, generator=g) * 2 - 1).to(device)
    target = torch.rand(3, cam.H, cam.W, generator=g).to(device)
    torch.manual_seed(seed)
    return DynamicStep(scene.to(device), cam.to(device), ctrl, target, **kw), scene


def test_full_size_step_runs_and_respects_the_mask(device):
    state, scene = _state(device, 200_000, 512, 800, 2, K=4, temperature=0.01, net_lr=1e-4)
    # put a fifth of the surfels behind the camera so that the visibility mask excludes something
    with torch.no_grad():
        state.params[0][::5, 2] += 10.0
    before = [p.detach().clone() for p in state.params]
    net_before = [p.detach().clone() for p in state.net.parameters()]
    ctrl_before = state.ctrl.detach().clone()
    print("[dynamic step] 200000 surfels, 512 control points, K=4, 800x800, two iterations", flush=True)
    losses, masks = [], []
    for i in range(2):
        loss, visible = state.step(torch.full((1,), 0.25 + 0.5 * i, device=device))
        losses.append(float(loss)), masks.append(visible.clone())
    torch.cuda.synchronize()
    assert all(np.isfinite(l) and 0 < l < 2 for l in losses), losses
    never = ~(masks[0] | masks[1])
    ever = masks[0] | masks[1]
    assert int(never.sum()) >= 40_000 and int(ever.sum()) > 100_000
    for p, b in zip(state.params, before):
        assert torch.equal(p.detach()[never], b[never])
        st = state.opt.state[p]
        assert not st['exp_avg'][never].any() and not st['exp_avg_sq'][never].any()
        assert torch.isfinite(p).all()
        assert float(st['step']) == 2.0
    moved = (state.params[0].detach() != before[0]).any(-1)
    assert not (moved & never).any() and int(moved.sum()) > 0.9 * int(ever.sum())
    # the network and the control points received gradients and stepped
    assert any(not torch.equal(a.detach(), b) for a, b in zip(state.net.parameters(), net_before))
    assert not torch.equal(state.ctrl.detach(), ctrl_before)
    assert all(torch.isfinite(p).all() for p in state.net.parameters()) and torch.isfinite(state.ctrl).all()
    # accum_max_count travelled with every render (network.py:706): only surfels that were rendered hold counts
    amc = state.accum_max_count
    assert int(amc.sum()) > 0 and not amc[never].any() and int((amc > 0).sum()) > 1000


def _ssim_torch(img1, img2):
    """The reference's conv2d form (losses/ssim.py:49-67): 11-tap Gaussian window, sigma 1.5, zero padding."""
    x = torch.arange(11, dtype=torch.float32, device=img1.device) - 5
    g = torch.exp(-x * x / (2 * 1.5 ** 2))
    g = g / g.sum()
    w = (g[:, None] * g[None, :]).expand(3, 1, 11, 11).contiguous()
    conv = lambda t: F.conv2d(t, w, padding=5, groups=3)
    mu1, mu2 = conv(img1), conv(img2)
    s1, s2, s12 = conv(img1 * img1) - mu1 * mu1, conv(img2 * img2) - mu2 * mu2, conv(img1 * img2) - mu1 * mu2
    C1, C2 = 0.01 ** 2, 0.03 ** 2
    return ((2 * mu1 * mu2 + C1) * (2 * s12 + C2)) / ((mu1 * mu1 + mu2 * mu2 + C1) * (s1 + s2 + C2))


@pytest.mark.parametrize("warp_method,LBS_method", [('LBS', 'dist'), ('LBS_c', 'dist')])
def test_autograd_edges_against_torch_formulation(warp_method, LBS_method, device):
    from fast_sp_gs_amd.deform import deform_apply, knn_points, superpoint_deform
    from fast_sp_gs_amd.renderer import GS_2D_render
    from fast_sp_gs_amd.ssim import l1_dssim_loss
    state, scene = _state(device, 4000, 48, 160, 5, K=4, temperature=0.05, warp_method=warp_method,
                          LBS_method=LBS_method)
    cam = state.cam
    g = torch.Generator().manual_seed(9)
    M = state.ctrl.shape[0]
    # stand-ins for the network's four outputs, as leaves (the network's own backward has its test elsewhere)
    mk = lambda c, s: (s * torch.randn(M, c, generator=g)).to(device).requires_grad_()
    net_out = [mk(3, 0.05), mk(4, 0.1), mk(2, 0.02), mk(4, 0.2)]
    leaves = state.params + [state.ctrl] + net_out
    names = ['means3D', 'scales', 'rotations', 'opacities', 'shs', 'ctrl', 'sp_t', 'sp_r', 'sp_s', 'sp_rot']

    # product path; the gradients that arrive at the renderer's inputs and at its image are kept, so that the stages
    # around the renderer can be compared on identical upstream gradients (two renders of inputs that differ in the
    # last bit can differ by a (pixel, surfel) pair that crosses the 1/255 threshold)
    means3D, scales, rotations = state.params[:3]
    c_xyz, c_rot, c_scale, c_local = net_out
    d_xyz, d_rot, d_scale, w, idx = superpoint_deform(means3D.detach(), state.ctrl, c_xyz, c_rot, c_scale,
                                                      sp_rot=c_local, K=4, temperature=0.05,
                                                      warp_method=warp_method, LBS_method=LBS_method)
    xyz, sc, rot = deform_apply(means3D, d_xyz, scales, d_scale, rotations, d_rot)
    out = GS_2D_render(xyz, sc, rot, state.params[3], (cam.W, cam.H), cam.Tw2v, cam.Tv2c, campos=cam.campos,
                       near=cam.near, far=cam.far, sh_degree=3, sh_features=state.params[4],
                       background=state.background)
    image = out['images']
    loss = l1_dssim_loss(image, state.target, 0.2)
    g_image, g_xyz, g_sc, g_rot = torch.autograd.grad(loss, [image, xyz, sc, rot], retain_graph=True)
    got = torch.autograd.grad(loss, leaves, allow_unused=True)

    # --- loss edge: 0.8 L1 + 0.2 (1 - SSIM) in torch on the same image
    im2 = image.detach().clone().requires_grad_()
    loss2 = 0.8 * (im2 - state.target).abs().mean() + 0.2 * (1 - _ssim_torch(im2[None], state.target[None]).mean())
    assert abs(float(loss2) - float(loss)) < 1e-6
    err = rel_err(npy(g_image), npy(torch.autograd.grad(loss2, im2)[0]))
    print(f"[dynamic step edges {warp_method}] dL/dimage: rel err {err:.2e}", flush=True)
    assert err < 1e-4

    # --- torch formulation of everything in front of the renderer (network.py:498-517, 545-573, 630-645)
    pts = means3D.detach()
    diff = pts[:, None, :] - state.ctrl[idx]
    nn_dist = (diff * diff).sum(-1)
    wt = torch.softmax(-nn_dist / 0.05, dim=-1)
    assert float((wt.detach() - w).abs().max()) < 1e-5
    q = c_local + torch.tensor([0, 0, 0, 1.0], device=device)
    q = q / q.norm(dim=-1, keepdim=True)
    qx, qy, qz, qs = q.unbind(-1)
    R = torch.stack([1 - 2 * (qy * qy + qz * qz), 2 * (qx * qy - qz * qs), 2 * (qy * qs + qx * qz),
                     2 * (qx * qy + qz * qs), 1 - 2 * (qx * qx + qz * qz), 2 * (qy * qz - qx * qs),
                     2 * (qx * qz - qy * qs), 2 * (qx * qs + qy * qz), 1 - 2 * (qx * qx + qy * qy)], -1).view(M, 3, 3)
    tt = c_xyz
    if warp_method == 'LBS_c':
        tt = c_xyz + state.ctrl - torch.einsum('mab,mb->ma', R, state.ctrl)
    moved = torch.einsum('nkab,nb->nka', R[idx], pts) + tt[idx]
    e_xyz = (wt[..., None] * moved).sum(1) - pts
    e_rot = (wt[..., None] * c_rot[idx]).sum(1)
    e_scale = (wt[..., None] * c_scale[idx]).sum(1)
    xyz2, sc2, rot2 = means3D + e_xyz, scales + e_scale, F.normalize(rotations + e_rot, dim=-1)
    assert float((xyz2 - xyz).detach().abs().max()) < 1e-5 and float((rot2 - rot).detach().abs().max()) < 1e-5
    deform_leaves = [means3D, scales, rotations, state.ctrl] + net_out
    deform_names = ['means3D', 'scales', 'rotations', 'ctrl', 'sp_t', 'sp_r', 'sp_s', 'sp_rot']
    want = torch.autograd.grad([xyz2, sc2, rot2], deform_leaves, grad_outputs=[g_xyz, g_sc, g_rot], allow_unused=True)
    got_by_name = dict(zip(names, got))
    for name, b in zip(deform_names, want):
        a = got_by_name[name]
        assert a is not None and b is not None, name
        err = rel_err(npy(a), npy(b))
        print(f"[dynamic step edges {warp_method}] {name}: rel err {err:.2e} (max |grad| {float(b.abs().max()):.2e})",
              flush=True)
        assert float(b.abs().max()) > 0, name
        assert err < 1e-4, (name, err)
    # the leaves that reach the loss through the renderer alone
    for name in ('opacities', 'shs'):
        assert got_by_name[name] is not None and float(got_by_name[name].abs().max()) > 0
