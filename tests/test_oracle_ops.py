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


def test_lbs_closed_forms(oracle_mod):
    """oracle/lbs.py (weights and warp of network.py:507-517, 545-573) against closed forms that a dropped term, a
    transposed rotation or a wrong branch would break."""
    from oracle import lbs as OL
    from scipy.spatial.transform import Rotation
    g = torch.Generator().manual_seed(3)
    N, M, K = 50, 8, 4
    f64 = dict(dtype=torch.float64, generator=g)
    pts, ctrl = torch.randn(N, 3, **f64), torch.randn(M, 3, **f64)
    idx = torch.stack([torch.randperm(M, generator=g)[:K] for _ in range(N)])
    d2 = torch.sort(torch.rand(N, K, **f64) * 0.05, 1).values
    zero3, zero4, s0 = torch.zeros(M, 3, dtype=torch.float64), torch.zeros(M, 4, dtype=torch.float64), \
        torch.zeros(M, 2, dtype=torch.float64)
    # identity transforms (local rotation 0 -> q = (0,0,0,1), t = 0) move nothing; 'dist' weights are a softmax
    dx, dr, ds, w = OL.lbs_blend(pts, ctrl, zero3, zero4, s0, zero4, d2, idx, 'dist', 0.01, 'LBS')
    assert float(dx.abs().max()) < 1e-14 and float(dr.abs().max()) == 0
    assert torch.allclose(w, torch.softmax(-d2 / 0.01, -1), atol=1e-14)
    # one rigid motion everywhere: p -> R p + t, with R from scipy (x, y, z, w convention)
    ang, axis = 0.7, np.array([0.0, 0.6, 0.8])
    q = np.concatenate([axis * np.sin(ang / 2), [np.cos(ang / 2)]])
    Rm = torch.from_numpy(Rotation.from_quat(q).as_matrix())
    t = torch.tensor([0.1, -0.2, 0.3], dtype=torch.float64)
    sp_rot = torch.from_numpy(2.5 * q - np.array([0, 0, 0, 1.0])).repeat(M, 1)  # normalize(rot + (0,0,0,1)) == q
    sp_r = torch.randn(M, 4, **f64)
    sp_t = t.repeat(M, 1)
    dx, dr, ds, w = OL.lbs_blend(pts, ctrl, sp_t, sp_r, s0 + 0.5, sp_rot, d2, idx, 'dist', 0.01, 'LBS')
    assert float((dx - (pts @ Rm.T + t - pts)).abs().max()) < 1e-12
    # the rotation that moves the points is sp_rot; sp_r is only blended into d_rotation (network.py:546-547, 565-566)
    assert float((dr - (w[..., None] * sp_r[idx]).sum(1)).abs().max()) < 1e-14 and torch.allclose(ds, ds * 0 + 0.5)
    # LBS_c: rotation about the control point c: p -> R (p - c) + c + t
    same = torch.full((N, K), 5)
    dx = OL.lbs_blend(pts, ctrl, sp_t, sp_r, s0, sp_rot, d2, same, 'dist', 0.01, 'LBS_c')[0]
    assert float((dx - ((pts - ctrl[5]) @ Rm.T + ctrl[5] + t - pts)).abs().max()) < 1e-12
    # 'largest' (network.py:555-561): ONE rigid transform per point, that of its assigned control point -- by default the
    # neighbour of largest weight (:594) -- written out here point by point with scipy rotations; residuals stay blended
    rots = torch.randn(M, 4, **f64) * 0.3
    t_each = torch.randn(M, 3, **f64)
    w_all = OL.lbs_weights(d2, idx, M, 'dist', 0.01)
    dx, dr, ds = OL.warp(pts, ctrl, t_each, sp_r, s0 + 0.5, rots, w_all, idx, 'largest')
    for n in range(N):
        m = int(idx[n, int(w_all[n].argmax())])
        qm = (rots[m] + torch.tensor([0, 0, 0, 1.0], dtype=torch.float64)).numpy()
        Rn = torch.from_numpy(Rotation.from_quat(qm / np.linalg.norm(qm)).as_matrix())
        assert float((dx[n] - (Rn @ pts[n] + t_each[m] - pts[n])).abs().max()) < 1e-12
    assert float((dr - (w_all[..., None] * sp_r[idx]).sum(1)).abs().max()) < 1e-14
    assigned = torch.randint(0, M, (N,), generator=g)
    dx2 = OL.warp(pts, ctrl, t_each, sp_r, s0, rots, w_all, idx, 'largest', p2sp=assigned)[0]
    one = OL.warp(pts, ctrl, t_each, sp_r, s0, rots, torch.ones(N, 1, dtype=torch.float64), assigned[:, None], 'LBS')[0]
    assert float((dx2 - one).abs().max()) < 1e-14  # == the blend over a single neighbour of weight one
    # no local rotation (the default configuration): the translations are blended, nothing else, whatever the method
    sp_t2 = torch.randn(M, 3, **f64)
    for method in ('LBS', 'LBS_c', 'largest'):
        dx, dr, ds, w = OL.lbs_blend(pts, ctrl, sp_t2, sp_r, s0, None, d2, idx, 'dist', 0.01, method)
        assert float((dx - (w[..., None] * sp_t2[idx]).sum(1)).abs().max()) < 1e-14
    # kernel weights by an explicit loop on the raw parameters (radius = exp(.), weight = sigmoid(.))
    rho, omega = 0.3 * torch.randn(M, **f64) - 2.0, torch.randn(M, **f64)
    for method in ('kernel', 'weighted_kernel'):
        w = OL.lbs_weights(d2, idx, M, method, 1.0, rho, omega)
        for n in range(0, N, 7):
            u = [np.exp(-float(d2[n, k]) / (2 * np.exp(float(rho[idx[n, k]])) ** 2)) *
                 (1 / (1 + np.exp(-float(omega[idx[n, k]]))) if method == 'weighted_kernel' else 1.0) + 1e-7
                 for k in range(K)]
            assert np.allclose(w[n].numpy(), np.array(u) / sum(u), atol=1e-14)
        assert torch.allclose(w.sum(-1), torch.ones(N, dtype=torch.float64))
    # limiting cases: equal radii and weights -> softmax(-d2 / (2 r^2)) up to the 1e-7 floor; a huge radius -> uniform
    w = OL.lbs_weights(d2, idx, M, 'kernel', 1.0, torch.full((M,), np.log(0.1), dtype=torch.float64), None)
    assert float((w - torch.softmax(-d2 / (2 * 0.1 ** 2), -1)).abs().max()) < 1e-6
    w = OL.lbs_weights(d2, idx, M, 'kernel', 1.0, torch.full((M,), 10.0, dtype=torch.float64), None)
    assert float((w - 1.0 / K).abs().max()) < 1e-6
    # 'W': softmax of the gathered rows; padded slots (index -1) get weight 0 and the rest still sums to 1
    sp_W = torch.randn(N, M, **f64)
    w = OL.lbs_weights(torch.gather(sp_W, 1, idx), idx, M, 'W')
    assert torch.allclose(w, torch.gather(sp_W, 1, idx).softmax(-1))
    padded = idx.clone()
    padded[:, -1] = -1
    w = OL.lbs_weights(d2, padded, M, 'dist', 0.01)
    assert float(w[:, -1].abs().max()) == 0 and torch.allclose(w.sum(-1), torch.ones(N, dtype=torch.float64))


def test_knn_backward_matches_autograd(oracle_mod):
    """K-NN squared distances: gradient of sum(g * d2) w.r.t. both point sets against torch autograd (fp64), with the 11
    columns the default configuration searches in (positions + 8 hyper features, exps/d_nerf.yaml:21-23)."""
    O = oracle_mod
    g = torch.Generator().manual_seed(12)
    for D in (3, 11):
        N, M, K = 70, 9, 3
        pts = torch.randn(N, D, generator=g, dtype=torch.float64, requires_grad=True)
        ctrl = torch.randn(M, D, generator=g, dtype=torch.float64, requires_grad=True)
        with torch.no_grad():
            idx = torch.cdist(pts, ctrl).topk(K, largest=False).indices.contiguous()
        diff = pts[:, None, :] - ctrl[idx]
        d2 = (diff * diff).sum(-1)
        gd = torch.randn(N, K, generator=g, dtype=torch.float64)
        k_x, k_y = torch.autograd.grad((d2 * gd).sum(), [pts, ctrl])
        n = lambda x: np.ascontiguousarray(x.detach().numpy())
        o_x, o_y = np.zeros((N, D)), np.zeros((M, D))
        assert O.call("knn_topk_backward_f64", N, M, D, K, n(pts), n(ctrl), n(idx), n(gd), o_x, o_y) == 0
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


def test_freq_encoder_double_tensor_goes_through_single_precision(oracle_mod):
    """freqencoder.cu:27-28 scales the angle with scalbnf, which narrows a double to float: for double tensors the
    forward is sinf / cosf of the float angle. Checked against numpy's float32 evaluation (one ulp of float), and shown
    to be a different function from the double-precision evaluation."""
    O = oracle_mod
    rng = np.random.default_rng(6)
    B, D, deg, scale = 41, 2, 10, 0.75
    x = np.ascontiguousarray(rng.uniform(-1, 1, size=(B, D)))
    out, exact = np.zeros((B, D * (2 * deg + 1))), np.zeros((B, D * (2 * deg + 1)))
    assert O.call("freq_encode_forward_double_via_single", B, D, deg, 1, scale, x, out) == 0
    assert O.call("freq_encode_forward_f64", B, D, deg, 1, scale, x, exact) == 0
    xf = (x * scale).astype(np.float32)
    parts = [x]
    for d in range(deg):
        v = np.ldexp(xf, d)
        assert v.dtype == np.float32
        parts += [np.sin(v).astype(np.float64), np.cos(v).astype(np.float64)]
    assert np.abs(out - np.concatenate(parts, -1)).max() < 1.5e-7
    assert np.array_equal(out[:, :D], x)  # the pass-through columns keep the double values
    assert np.abs(out - exact).max() > 4e-6
