"""GPU parity of the fused render epilogue (normals to world space, nan_to_num, surf_depth, depth_to_normal * opacity,
background composite) and its backward: against the oracle through the operators, and through `GS_2D_render` against
the reference's own torch formulation of the same lines (the path `GS_2D_render` keeps for cameras that require
gradients). Tolerances: outputs 1e-4 abs (unit normals, depths of a few units), gradients 1e-3 of the largest entry."""
import numpy as np
import pytest
import torch

from util import abs_err, npy, rel_err

pytestmark = pytest.mark.gpu


def _inputs(W, H, seed, device):
    from fast_sp_gs_amd import scenes
    g = torch.Generator().manual_seed(seed)
    cam = scenes.pinhole(W, H, 45.0, torch.tensor([0.6, -0.3, 3.8]))
    extras = torch.randn(9, H, W, generator=g)
    # a smooth depth surface + noise: neighbouring world points differ by ~1e-2, like a rendered depth map
    yy, xx = torch.meshgrid(torch.linspace(-1, 1, H), torch.linspace(-1, 1, W), indexing='ij')
    extras[0] = 3.5 + 0.3 * xx + 0.2 * yy * yy + 0.01 * torch.rand(H, W, generator=g)
    extras[4] = 3.4 + 0.25 * xx * yy + 0.01 * torch.rand(H, W, generator=g)
    if H > 8 and W > 8:
        extras[0, 3, 4], extras[4, 5, 6], extras[4, 7, 2] = float('nan'), float('inf'), float('nan')
    else:
        extras[0, 0, 0] = float('nan')
    opacity = torch.rand(H, W, generator=g)
    images = torch.rand(3, H, W, generator=g)
    bg = torch.tensor([0.1, 0.6, 0.9])
    grads = [torch.randn(c, H, W, generator=g) for c in (3, 1, 1, 3, 1, 3)]
    d = lambda t: t.to(device).contiguous()
    return cam, extras, opacity, images, bg, grads, d


@pytest.mark.parametrize("W,H,ratio,composite", [(96, 64, 1.0, True), (131, 77, 0.3, True), (40, 33, 0.0, False),
                                                 (2, 2, 0.5, True), (800, 800, 1.0, True)])
def test_epilogue_against_oracle(W, H, ratio, composite, device, oracle_mod):
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    cam, extras, opacity, images, bg, grads, d = _inputs(W, H, 50 + W, device)
    print(f"[epilogue] {W}x{H} ratio={ratio} composite={composite}", flush=True)
    out = get_C_function('gs_2d_epilogue_forward')(W, H, ratio, d(cam.Tw2v), d(cam.Tv2c), d(extras), d(opacity),
                                                   d(images) if composite else None, d(bg) if composite else None)
    torch.cuda.synchronize()
    z = lambda *s: np.zeros(s, np.float32)
    ref = [z(3, H, W), z(1, H, W), z(1, H, W), z(3, H, W), z(3, H, W) if composite else None]
    O.call("gs_2d_epilogue_forward_f32", W, H, ratio, npy(cam.Tw2v), npy(cam.Tv2c), npy(extras), npy(opacity),
           npy(images) if composite else None, npy(bg) if composite else None, *ref)
    names = ('normals', 'depths', 'surf_depth', 'surf_normal', 'composited')
    for name, a, b in zip(names, out, ref):
        assert (a is None) == (b is None), name
        if a is not None:
            assert np.isfinite(npy(a)).all() and abs_err(npy(a), b) < 1e-4, (name, abs_err(npy(a), b))
    g_n, g_d, g_sd, g_sn, g_dist, g_c = grads
    got = get_C_function('gs_2d_epilogue_backward')(W, H, ratio, d(cam.Tw2v), d(cam.Tv2c), d(extras), d(opacity),
                                                    d(bg) if composite else None, d(g_n), d(g_d), d(g_sd), d(g_sn),
                                                    d(g_dist), d(g_c) if composite else None)
    torch.cuda.synchronize()
    r_extras, r_opa = z(9, H, W), z(H, W) if composite else None
    O.call("gs_2d_epilogue_backward_f32", W, H, ratio, npy(cam.Tw2v), npy(cam.Tv2c), npy(extras), npy(opacity),
           npy(bg) if composite else None, npy(g_n), npy(g_d), npy(g_sd), npy(g_sn), npy(g_dist),
           npy(g_c) if composite else None, r_extras, r_opa)
    assert np.isfinite(npy(got[0])).all()
    for ch in range(9):  # per channel: the depth channels carry gradients ~1e3 larger than the others
        assert rel_err(npy(got[0])[ch], r_extras[ch]) < 1e-3, (ch, rel_err(npy(got[0])[ch], r_extras[ch]))
    assert (got[1] is None) == (not composite)
    if composite:
        assert rel_err(npy(got[1]), r_opa) < 1e-5
    # absent upstream gradients are zeros
    none = get_C_function('gs_2d_epilogue_backward')(W, H, ratio, d(cam.Tw2v), d(cam.Tv2c), d(extras), d(opacity),
                                                     None, None, None, None, None, None, None)
    assert not npy(none[0]).any() and none[1] is None


def test_render_epilogue_autograd_matches_torch_path(device):
    """GS_2D_render end to end: the fused epilogue (default) and the reference's torch ops (taken when the camera
    requires gradients) give the same output dict and the same parameter gradients."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.renderer import GS_2D_render
    scene_h, cam_h = scenes.config0(P=4000, size=160, seed=3)
    scene, cam = scene_h.to(device), cam_h.to(device)
    bg = torch.tensor([0.3, 0.7, 0.2], device=device)
    g = torch.Generator().manual_seed(8)
    keys = ('images', 'depths', 'normals', 'opacity', 'distortion', 'surf_depth', 'surf_normal')
    weights = {k: None for k in keys}
    results = []
    for camera_grad in (False, True):
        params = [getattr(scene, k).clone().requires_grad_(True) for k in
                  ('means3D', 'scales', 'rotations', 'opacities', 'shs')]
        Tw2v = cam.Tw2v.clone().requires_grad_(camera_grad)
        out = GS_2D_render(params[0], params[1], params[2], params[3], (cam.W, cam.H), Tw2v, cam.Tv2c,
                           campos=cam.campos, near=cam.near, far=cam.far, sh_degree=3, sh_features=params[4],
                           depth_ratio=0.4, background=bg)
        loss = 0
        for k in keys:
            if weights[k] is None:
                weights[k] = torch.randn(out[k].shape, generator=g).to(device)
            loss = loss + (out[k] * weights[k]).sum()
        loss.backward()
        results.append(({k: out[k].detach() for k in keys}, [p.grad for p in params]))
    (o_fused, g_fused), (o_torch, g_torch) = results
    for k in keys:
        assert float((o_fused[k] - o_torch[k]).abs().max()) < 1e-4, k
    for name, a, b in zip(('means3D', 'scales', 'rotations', 'opacities', 'shs'), g_fused, g_torch):
        assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max()), name
