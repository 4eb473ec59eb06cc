"""Pins the oracle's stand-alone operators (oracle/ops.cpp) against library routines and closed forms:
cdist top-1 and its tie rules, K-NN, LBS, masked Adam vs torch.optim.Adam, the frequency encoder vs torch.sin/cos,
the deformation MLP vs a torch.nn.functional.linear chain."""
import numpy as np
import pytest
import torch


def test_cdist_top_matches_torch_and_tie_rules(oracle_mod):
    O = oracle_mod
    rng = np.random.default_rng(0)
    B, N, M, D = 2, 300, 40, 5
    x = np.ascontiguousarray(rng.normal(size=(B, N, D)).astype(np.float32))
    y = np.ascontiguousarray(rng.normal(size=(B, M, D)).astype(np.float32))
    for largest in (0, 1):
        dist, idx = np.zeros((B, N), np.float32), np.zeros((B, N), np.int64)
        assert O.call("cdist_top_forward_f32", B, N, M, D, largest, x, y, dist, idx) == 0
        full = torch.cdist(torch.from_numpy(x).double(), torch.from_numpy(y).double())
        ref_v, ref_i = (full.max(-1) if largest else full.min(-1))
        assert np.array_equal(idx, ref_i.numpy()) and np.abs(dist - ref_v.numpy()).max() < 1e-5
    # ties: smallest keeps the LAST equal minimum, largest keeps the FIRST equal maximum (cdist_top.cu:24)
    x1 = np.zeros((1, 1, 2), np.float32)
    y1 = np.ascontiguousarray(np.array([[[1, 0], [0, 1], [-1, 0], [3, 0], [0, 3]]], np.float32))
    dist, idx = np.zeros((1, 1), np.float32), np.zeros((1, 1), np.int64)
    O.call("cdist_top_forward_f32", 1, 1, 5, 2, 0, x1, y1, dist, idx)
    assert idx[0, 0] == 2 and dist[0, 0] == 1
    O.call("cdist_top_forward_f32", 1, 1, 5, 2, 1, x1, y1, dist, idx)
    assert idx[0, 0] == 3 and dist[0, 0] == 3


def test_cdist_top_backward_matches_autograd(oracle_mod):
    O = oracle_mod
    rng = np.random.default_rng(1)
    B, N, M, D = 2, 50, 20, 3
    x = torch.from_numpy(rng.normal(size=(B, N, D))).requires_grad_()
    y = torch.from_numpy(rng.normal(size=(B, M, D))).requires_grad_()
    gd = torch.from_numpy(rng.normal(size=(B, N)))
    v, i = torch.cdist(x, y).min(-1)
    (v * gd).sum().backward()
    g1, g2 = np.zeros((B, N, D)), np.zeros((B, M, D))
    assert O.call("cdist_top_backward_f64", B, N, M, D, x.detach().numpy(), y.detach().numpy(), v.detach().numpy(),
                  np.ascontiguousarray(i.numpy()), gd.numpy(), g1, g2) == 0
    assert np.abs(g1 - x.grad.numpy()).max() < 1e-12 and np.abs(g2 - y.grad.numpy()).max() < 1e-12


def test_knn_matches_sorting(oracle_mod):
    O = oracle_mod
    rng = np.random.default_rng(2)
    N, M, D, K = 400, 64, 3, 4
    x = np.ascontiguousarray(rng.uniform(-1, 1, size=(N, D)).astype(np.float32))
    y = np.ascontiguousarray(rng.uniform(-1, 1, size=(M, D)).astype(np.float32))
    y[10] = y[3]  # an exact duplicate: the lower index must come first
    d2, idx = np.zeros((N, K), np.float32), np.zeros((N, K), np.int64)
    assert O.call("knn_topk_f32", N, M, D, K, x, y, d2, idx) == 0
    diff = x[:, None, :] - y[None]
    full = ((diff[..., 0] * diff[..., 0] + diff[..., 1] * diff[..., 1]) + diff[..., 2] * diff[..., 2]).astype(np.float32)
    order = np.argsort(full, axis=1, kind="stable")[:, :K]
    assert np.array_equal(idx, order)
    assert np.array_equal(d2, np.take_along_axis(full, order, 1))
    assert (np.diff(d2, axis=1) >= 0).all()
    # K larger than M: padded with -1
    d2, idx = np.zeros((2, 5), np.float32), np.zeros((2, 5), np.int64)
    O.call("knn_topk_f32", 2, 3, D, 5, x[:2].copy(), y[:3].copy(), d2, idx)
    assert (idx[:, 3:] == -1).all() and (d2[:, 3:] == -1).all()


def _lbs(O, points, ctrl, sp_t, sp_r, sp_s, d2, idx, temperature, centred):
    N, K = d2.shape
    S = sp_s.shape[1]
    w, dx, dr, ds = np.zeros((N, K)), np.zeros((N, 3)), np.zeros((N, 4)), np.zeros((N, S))
    assert O.call("lbs_blend_f64", N, ctrl.shape[0], K, int(centred), float(temperature), points, ctrl, sp_t, sp_r,
                  sp_s, S, d2, idx, w, dx, dr, ds) == 0
    return w, dx, dr, ds


def test_lbs_closed_forms(oracle_mod):
    O = oracle_mod
    rng = np.random.default_rng(3)
    N, M, K = 50, 8, 4
    pts, ctrl = rng.normal(size=(N, 3)), rng.normal(size=(M, 3))
    idx = np.ascontiguousarray(np.stack([rng.permutation(M)[:K] for _ in range(N)]).astype(np.int64))
    d2 = np.ascontiguousarray(np.sort(rng.uniform(0, 0.05, size=(N, K)), 1))
    zero3, zero4, s0 = np.zeros((M, 3)), np.zeros((M, 4)), np.zeros((M, 2))
    # identity transforms (residual rotation 0 -> q = (0,0,0,1), t = 0) move nothing; weights are a softmax
    w, dx, dr, ds = _lbs(O, pts, ctrl, zero3, zero4, s0, d2, idx, 0.01, False)
    assert np.abs(dx).max() < 1e-14 and np.abs(dr).max() == 0
    assert np.allclose(w, torch.softmax(torch.from_numpy(-d2 / 0.01), -1).numpy(), atol=1e-14)
    # one control point everywhere with weight 1: a rigid motion p -> R p + t
    ang, axis = 0.7, np.array([0.0, 0.6, 0.8])
    q = np.concatenate([axis * np.sin(ang / 2), [np.cos(ang / 2)]])
    from scipy.spatial.transform import Rotation
    Rm = Rotation.from_quat(q).as_matrix()
    t = np.array([0.1, -0.2, 0.3])
    sp_r = np.tile(2.5 * q - np.array([0, 0, 0, 1.0]), (M, 1))  # normalize(r + (0,0,0,1)) == q
    sp_t = np.tile(t, (M, 1))
    w, dx, dr, ds = _lbs(O, pts, ctrl, sp_t, sp_r, s0 + 0.5, d2, idx, 0.01, False)
    assert np.abs(dx - (pts @ Rm.T + t - pts)).max() < 1e-12
    assert np.allclose(dr, sp_r[0]) and np.allclose(ds, 0.5)
    # centred: rotation about the control point c: p -> R (p - c) + c + t
    same = np.zeros((N, K), np.int64) + 5
    w, dx, dr, ds = _lbs(O, pts, ctrl, sp_t, sp_r, s0, d2, same, 0.01, True)
    assert np.abs(dx - ((pts - ctrl[5]) @ Rm.T + ctrl[5] + t - pts)).max() < 1e-12


def test_lbs_and_knn_backward_match_autograd(oracle_mod):
    """The oracle's hand-derived LBS / K-NN gradients against torch autograd (fp64) of the forward written a different
    way: rotation through Rodrigues' form R = (w^2 - v.v) I + 2 v v^T + 2 w [v]x of the normalised quaternion, weights
    through torch.softmax, distances through explicit differences."""
    O = oracle_mod
    g = torch.Generator().manual_seed(12)
    N, M, K, S, tau = 70, 9, 4, 2, 0.05
    for centred in (False, True):
        pts = torch.randn(N, 3, generator=g, dtype=torch.float64, requires_grad=True)
        ctrl = torch.randn(M, 3, generator=g, dtype=torch.float64, requires_grad=True)
        sp_t = (0.2 * torch.randn(M, 3, generator=g, dtype=torch.float64)).requires_grad_()
        sp_r = (0.4 * torch.randn(M, 4, generator=g, dtype=torch.float64)).requires_grad_()
        sp_s = (0.1 * torch.randn(M, S, generator=g, dtype=torch.float64)).requires_grad_()
        with torch.no_grad():
            idx = torch.cdist(pts, ctrl).topk(K, largest=False).indices.contiguous()
        diff = pts[:, None, :] - ctrl[idx]
        d2 = (diff * diff).sum(-1)
        d2_leaf = d2.detach().clone().requires_grad_()
        w = torch.softmax(-d2_leaf / tau, -1)
        q = sp_r + torch.tensor([0, 0, 0, 1.0], dtype=torch.float64)
        q = q / q.norm(dim=-1, keepdim=True)
        v, s = q[:, :3], q[:, 3:]
        zero = torch.zeros(M, dtype=torch.float64)
        skew = torch.stack([zero, -v[:, 2], v[:, 1], v[:, 2], zero, -v[:, 0], -v[:, 1], v[:, 0], zero], -1).view(M, 3, 3)
        eye = torch.eye(3, dtype=torch.float64)
        R = (s * s - (v * v).sum(-1, keepdim=True))[..., None] * eye + 2 * v[:, :, None] * v[:, None, :] + \
            2 * s[..., None] * skew
        t = sp_t + ctrl - torch.einsum('mab,mb->ma', R, ctrl) if centred else sp_t
        moved = torch.einsum('nkab,nb->nka', R[idx], pts) + t[idx]
        d_xyz = (w[..., None] * moved).sum(1) - pts
        d_rot = (w[..., None] * sp_r[idx]).sum(1)
        d_scale = (w[..., None] * sp_s[idx]).sum(1)
        gx, gr, gs = (torch.randn(*t_.shape, generator=g, dtype=torch.float64) for t_ in (d_xyz, d_rot, d_scale))
        loss = (d_xyz * gx).sum() + (d_rot * gr).sum() + (d_scale * gs).sum()
        a_pts, a_d2, a_ctrl, a_t, a_r, a_s = torch.autograd.grad(loss, [pts, d2_leaf, ctrl, sp_t, sp_r, sp_s],
                                                                  allow_unused=True)
        n = lambda x: np.ascontiguousarray(x.detach().numpy())
        o_pts, o_d2, o_ctrl = np.zeros((N, 3)), np.zeros((N, K)), np.zeros((M, 3))
        o_t, o_r, o_s = np.zeros((M, 3)), np.zeros((M, 4)), np.zeros((M, S))
        assert O.call("lbs_blend_backward_f64", N, M, K, int(centred), tau, n(pts), n(ctrl), n(sp_t), n(sp_r), n(sp_s),
                      S, n(d2), n(idx), n(gx), n(gr), n(gs), o_pts, o_d2, o_ctrl, o_t, o_r, o_s) == 0
        a_ctrl = torch.zeros(M, 3, dtype=torch.float64) if a_ctrl is None else a_ctrl
        for name, a, o in (("points", a_pts, o_pts), ("dist2", a_d2, o_d2), ("sp_points", a_ctrl, o_ctrl),
                           ("sp_t", a_t, o_t), ("sp_r", a_r, o_r), ("sp_s", a_s, o_s)):
            scale = max(float(a.abs().max()), 1e-30)
            assert np.abs(n(a) - o).max() < 1e-11 * max(scale, 1.0), (centred, name)
        assert centred or not o_ctrl.any()
        # K-NN distances: gradient of sum(g * d2) w.r.t. both point sets
        gd = torch.randn(N, K, generator=g, dtype=torch.float64)
        k_x, k_y = torch.autograd.grad((d2 * gd).sum(), [pts, ctrl])
        o_x, o_y = np.zeros((N, 3)), np.zeros((M, 3))
        assert O.call("knn_topk_backward_f64", N, M, 3, K, n(pts), n(ctrl), n(idx), n(gd), o_x, o_y) == 0
        assert np.abs(n(k_x) - o_x).max() < 1e-12 and np.abs(n(k_y) - o_y).max() < 1e-12


def _epilogue_torch(Tw2v, Tv2c, W, H, extras, opacity, images, bg, ratio):
    """renderer/gs_2d_render.py:608-617 + :439-470 + network.py:725-726 written with torch ops the way the reference
    writes them (matrix inverses, meshgrid, matmuls, torch.cross, F.normalize, nan_to_num)."""
    depths, normals, median, distortion, _ = extras.split([1, 3, 1, 1, 3], dim=0)
    normals = (normals.permute(1, 2, 0) @ Tw2v[:3, :3]).permute(2, 0, 1)
    median = torch.nan_to_num(median, 0, 0)
    depths = torch.nan_to_num(depths, 0, 0)
    surf_depth = depths * (1 - ratio) + ratio * median
    c2w = Tw2v.inverse()
    ndc2pix = torch.tensor([[W / 2, 0, 0, W / 2], [0, H / 2, 0, H / 2], [0, 0, 0, 1]], dtype=Tw2v.dtype).T
    projection_matrix = c2w.T @ (Tv2c @ Tw2v).T
    intrins = (projection_matrix @ ndc2pix)[:3, :3].T
    gx, gy = torch.meshgrid(torch.arange(W, dtype=Tw2v.dtype), torch.arange(H, dtype=Tw2v.dtype), indexing='xy')
    pix = torch.stack([gx, gy, torch.ones_like(gx)], dim=-1).reshape(-1, 3)
    rays_d = pix @ intrins.inverse().T @ c2w[:3, :3].T
    points = (surf_depth.reshape(-1, 1) * rays_d + c2w[:3, 3]).reshape(H, W, 3)
    out = torch.zeros_like(points)
    dx = points[2:, 1:-1] - points[:-2, 1:-1]
    dy = points[1:-1, 2:] - points[1:-1, :-2]
    out[1:-1, 1:-1, :] = torch.nn.functional.normalize(torch.cross(dx, dy, dim=-1), dim=-1)
    surf_normal = out.permute(2, 0, 1) * opacity.detach()
    comp = images + (1 - opacity) * bg[:, None, None]
    return normals, median, surf_depth, surf_normal, distortion, comp


def test_epilogue_matches_reference_formulation(oracle_mod):
    O = oracle_mod
    from fast_sp_gs_amd import scenes
    g = torch.Generator().manual_seed(15)
    W, H, ratio = 23, 17, 0.3
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0.7, -0.4, 3.5]))
    Tw2v, Tv2c = cam.Tw2v.double(), cam.Tv2c.double()
    extras = torch.randn(9, H, W, generator=g, dtype=torch.float64)
    extras[0] = 3.0 + 0.5 * torch.rand(H, W, generator=g, dtype=torch.float64)
    extras[4] = 3.0 + 0.5 * torch.rand(H, W, generator=g, dtype=torch.float64)
    extras[0, 2, 3], extras[4, 5, 6], extras[4, 7, 7] = float('nan'), float('inf'), float('nan')
    extras[0, 8:10, 8:10] = 0.0
    extras[4, 8:10, 8:10] = 0.0  # a flat patch at the camera centre: zero cross product, the eps branch
    opacity = torch.rand(H, W, generator=g, dtype=torch.float64)
    images = torch.rand(3, H, W, generator=g, dtype=torch.float64)
    bg = torch.tensor([0.2, 0.5, 0.9], dtype=torch.float64)
    ex, op, im = extras.clone().requires_grad_(), opacity.clone().requires_grad_(), images.clone().requires_grad_()
    want = _epilogue_torch(Tw2v, Tv2c, W, H, ex, op, im, bg, ratio)
    n = lambda t: np.ascontiguousarray(t.detach().numpy())
    z = lambda *shape: np.zeros(shape)
    normals, depths, sd, sn, comp = z(3, H, W), z(1, H, W), z(1, H, W), z(3, H, W), z(3, H, W)
    assert O.call("gs_2d_epilogue_forward_f64", W, H, ratio, n(Tw2v), n(Tv2c), n(extras), n(opacity), n(images), n(bg),
                  normals, depths, sd, sn, comp) == 0
    for name, a, b in (("normals", normals, want[0]), ("depths", depths, want[1]), ("surf_depth", sd, want[2]),
                       ("surf_normal", sn, want[3]), ("composite", comp, want[5])):
        assert np.abs(a - n(b)).max() < 1e-9, name
    assert np.abs(sn[:, 1:-1, 1:-1]).max() > 0.1 and not sn[:, 0].any() and not sn[:, :, -1].any()
    # backward against autograd of the same formulation
    grads = [torch.randn(*t.shape, generator=g, dtype=torch.float64) for t in want]
    loss = sum((t * g_).sum() for t, g_ in zip(want, grads))
    a_ex, a_op, a_im = torch.autograd.grad(loss, [ex, op, im])
    g_extras, g_opacity = z(9, H, W), z(H, W)
    assert O.call("gs_2d_epilogue_backward_f64", W, H, ratio, n(Tw2v), n(Tv2c), n(extras), n(opacity), n(bg),
                  n(grads[0]), n(grads[1]), n(grads[2]), n(grads[3]), n(grads[4]), n(grads[5]), g_extras,
                  g_opacity) == 0
    assert (np.abs(g_extras - n(a_ex)) <= 1e-8 * (1.0 + np.abs(n(a_ex)))).all()  # element-wise: the eps branch gives 1e12s
    assert np.abs(g_opacity - n(a_op)).max() < 1e-12  # the opacity only enters through the composite (detached elsewhere)
    assert torch.equal(a_im, grads[5])                # and the image gradient is the composite's, unchanged


def test_simple_knn_matches_kdtree(oracle_mod):
    """Exact 3-NN mean squared distance against scipy's k-d tree (k = 4 with the point itself first)."""
    O = oracle_mod
    from scipy.spatial import cKDTree
    rng = np.random.default_rng(17)
    pts = rng.normal(size=(3000, 3))
    pts[10] = pts[11]            # a duplicate pair: distance 0 counts
    out = np.zeros(3000)
    assert O.call("simple_knn_f64", 3000, pts, out) == 0
    d, _ = cKDTree(pts).query(pts, k=4)
    assert np.abs(out - (d[:, 1:] ** 2).mean(1)).max() < 1e-12
    assert out[10] < out.mean() and out[10] == out[11]
    # fewer than four points: missing neighbours stay at the largest float, as in the reference (FLT_MAX / 3 with one
    # missing, overflow to inf with two)
    few = np.ascontiguousarray(pts[:3].astype(np.float32))
    o32 = np.zeros(3, np.float32)
    assert O.call("simple_knn_f32", 3, few, o32) == 0
    assert np.allclose(o32, np.finfo(np.float32).max / 3, rtol=1e-6)
    assert O.call("simple_knn_f32", 2, few[:2].copy(), o32) == 0
    assert np.isinf(o32[:2]).all()


def test_masked_adam_matches_torch_adam(oracle_mod):
    O = oracle_mod
    rng = np.random.default_rng(4)
    N, M = 64, 6
    p0 = rng.normal(size=(N, M))
    param = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    opt = torch.optim.Adam([param], lr=1.6e-4, betas=(0.9, 0.999), eps=1e-15)
    p, m, v = p0.copy(), np.zeros((N, M)), np.zeros((N, M))
    mask = np.ones(N, np.uint8)
    for step in range(1, 4):
        g = rng.normal(size=(N, M))
        param.grad = torch.from_numpy(g.copy())
        opt.step()
        # SparseGaussianAdam folds the bias corrections into the learning rate (sparse_gaussian_adam.py:46)
        lr = 1.6e-4 * (1 - 0.999 ** step) ** 0.5 / (1 - 0.9 ** step)
        assert O.call("adam_masked_update_f64", N, M, mask, lr, 0.9, 0.999, 1e-15, p, np.ascontiguousarray(g), m, v) == 0
        assert np.abs(p - param.detach().numpy()).max() < 1e-12
    # masked rows are untouched, including their moments
    mask[::2] = 0
    before = (p.copy(), m.copy(), v.copy())
    O.call("adam_masked_update_f64", N, M, mask, 1e-3, 0.9, 0.999, 1e-15, p, np.ascontiguousarray(rng.normal(size=(N, M))), m, v)
    for a, b in zip(before, (p, m, v)):
        assert np.array_equal(a[::2], b[::2]) and not np.array_equal(a[1::2], b[1::2])


@pytest.mark.parametrize("include_input", [True, False])
def test_freq_encoder(oracle_mod, include_input):
    O = oracle_mod
    rng = np.random.default_rng(5)
    B, D, deg, scale = 37, 3, 10, 1.0
    x = np.ascontiguousarray(rng.uniform(-1, 1, size=(B, D)))
    Do = D * (2 * deg + int(include_input))
    out = np.zeros((B, Do))
    assert O.call("freq_encode_forward_f64", B, D, deg, int(include_input), scale, x, out) == 0
    parts = [torch.from_numpy(x)] if include_input else []
    for d in range(deg):
        parts += [torch.sin(torch.from_numpy(x) * 2.0 ** d * scale), torch.cos(torch.from_numpy(x) * 2.0 ** d * scale)]
    assert np.abs(out - torch.cat(parts, -1).numpy()).max() < 1e-9
    g = np.ascontiguousarray(rng.normal(size=(B, Do)))
    gin = np.zeros((B, D))
    assert O.call("freq_encode_backward_f64", B, D, deg, int(include_input), scale, g, out, gin) == 0
    xt = torch.from_numpy(x).requires_grad_()
    parts = [xt] if include_input else []
    for d in range(deg):
        parts += [torch.sin(xt * 2.0 ** d * scale), torch.cos(xt * 2.0 ** d * scale)]
    (torch.cat(parts, -1) * torch.from_numpy(g)).sum().backward()
    assert np.abs(gin - xt.grad.numpy()).max() < 1e-8


def test_deform_mlp_matches_torch(oracle_mod):
    import ctypes
    O = oracle_mod
    torch.manual_seed(0)
    B, Din, Wd, L, skip = 33, 84, 256, 8, 4
    x = torch.randn(B, Din)
    Ws, bs = [], []
    for i in range(L):
        din = Din if i == 0 else (Wd + Din if i == skip + 1 else Wd)
        Ws.append(torch.randn(Wd, din) / din ** 0.5)
        bs.append(torch.randn(Wd) * 0.1)
    heads = [(torch.randn(3, Wd) * 0.1, torch.randn(3)), (torch.randn(4, Wd) * 0.1, torch.randn(4)),
             (torch.randn(3, Wd) * 0.1, torch.randn(3))]
    h = x
    for i in range(L):  # network.py:1763-1767
        h = torch.relu(torch.nn.functional.linear(h, Ws[i], bs[i]))
        if i == skip:
            h = torch.cat([x, h], -1)
    ref = [torch.nn.functional.linear(h, w, b) for w, b in heads]
    arr = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    outs = [torch.zeros(B, w.shape[0]) for w, _ in heads]
    dims = (ctypes.c_int * 3)(3, 4, 3)
    lib = O.lib()
    lib.oracle_deform_mlp_f32.restype = ctypes.c_int
    rc = lib.oracle_deform_mlp_f32(B, Din, Wd, L, skip, ctypes.c_void_p(x.data_ptr()), arr(Ws), arr(bs), 3, dims,
                                   arr([w for w, _ in heads]), arr([b for _, b in heads]), arr(outs))
    assert rc == 0
    for o, r in zip(outs, ref):
        assert (o - r).abs().max() < 1e-4


def test_fusedssim_matches_conv2d_and_autograd(oracle_mod):
    """The oracle's fused SSIM against the textbook form the reference keeps as its fallback (losses/ssim.py:49-67):
    grouped conv2d with the normalised 11x11 Gaussian window (sigma 1.5, built here from its definition), zero padding;
    the backward against autograd of that form. Sizes are not multiples of the 32-pixel blocks."""
    import math
    import torch.nn.functional as F
    O = oracle_mod
    B, CH, H, W = 2, 3, 45, 70
    g = torch.Generator().manual_seed(0)
    img1 = torch.rand(B, CH, H, W, generator=g, dtype=torch.float64, requires_grad=True)
    img2 = torch.rand(B, CH, H, W, generator=g, dtype=torch.float64)
    gmap = torch.randn(B, CH, H, W, generator=g, dtype=torch.float64)
    w1 = torch.tensor([math.exp(-(x - 5) ** 2 / (2 * 1.5 ** 2)) for x in range(11)], dtype=torch.float64)
    w1 = w1 / w1.sum()
    win = (w1[:, None] * w1[None, :]).expand(CH, 1, 11, 11).contiguous()
    C1, C2 = 0.01 ** 2, 0.03 ** 2
    conv = lambda t: F.conv2d(t, win, padding=5, groups=CH)
    mu1, mu2 = conv(img1), conv(img2)
    s1, s2, s12 = conv(img1 * img1) - mu1 * mu1, conv(img2 * img2) - mu2 * mu2, conv(img1 * img2) - mu1 * mu2
    ref = ((2 * mu1 * mu2 + C1) * (2 * s12 + C2)) / ((mu1 * mu1 + mu2 * mu2 + C1) * (s1 + s2 + C2))
    (ref * gmap).sum().backward()

    a, b = img1.detach().numpy().copy(), img2.numpy().copy()
    out, d1, d2, d3 = (np.zeros_like(a) for _ in range(4))
    assert O.call("fusedssim_forward_f64", B, CH, H, W, C1, C2, a, b, out, d1, d2, d3) == 0
    # the kernel's weights are float literals: they differ from the exact Gaussian by float rounding
    assert np.abs(out - ref.detach().numpy()).max() < 1e-6
    grad = np.zeros_like(a)
    assert O.call("fusedssim_backward_f64", B, CH, H, W, a, b, gmap.numpy().copy(), d1, d2, d3, grad) == 0
    gref = img1.grad.numpy()
    assert np.abs(grad - gref).max() < 1e-5 * np.abs(gref).max()
    # without the partial-derivative maps only the SSIM map is produced
    out2 = np.zeros_like(a)
    assert O.call("fusedssim_forward_f64", B, CH, H, W, C1, C2, a, b, out2, None, None, None) == 0
    assert np.array_equal(out, out2)
    # identical images: SSIM is exactly 1 wherever the window is defined
    same = np.zeros_like(a)
    assert O.call("fusedssim_forward_f64", B, CH, H, W, C1, C2, a, a, same, None, None, None) == 0
    assert np.abs(same - 1.0).max() < 1e-12
