"""GPU parity of the stand-alone operators against the CPU oracle (same seeded inputs), through the operator boundary
and the autograd wrappers. Indices are compared bit for bit; floats within 1e-5 abs / 1e-3 rel as stated per check."""
import numpy as np
import pytest
import torch

from util import abs_err, npy, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def c1():
    from fast_sp_gs_amd import scenes
    return scenes.config1(n_dirs=50_000, n_points=20_000, n_ctrl=512)


def test_sh_to_rgb_and_encoder(device, oracle_mod, c1):
    O = oracle_mod
    from fast_sp_gs_amd.ops import SH_to_RGB, sh_encode
    dirs, shs = c1['dirs'], c1['shs']
    P = dirs.shape[0]
    g = torch.Generator().manual_seed(3)
    grad_rgb, grad_enc = torch.randn(P, 3, generator=g), torch.randn(P, 16, generator=g)
    campos = torch.tensor([0.2, -0.1, 3.0])
    for cam in (None, campos):
        d = dirs.to(device).requires_grad_()
        s = shs.to(device).requires_grad_()
        c = None if cam is None else cam.to(device).requires_grad_()
        rgb = SH_to_RGB(s, d, c, 3, True)
        rgb.backward(grad_rgb.to(device))
        ref = np.zeros((P, 3), np.float32)
        O.call("sh_to_rgb_forward_f32", P, 16, 3, 1, npy(dirs), None if cam is None else npy(cam), npy(shs), ref)
        assert abs_err(npy(rgb), ref) < 2e-6
        gd, gs = np.zeros((P, 3), np.float32), np.zeros((P, 16, 3), np.float32)
        gc = None if cam is None else np.zeros(3, np.float32)
        O.call("sh_to_rgb_backward_f32", P, 16, 3, 1, npy(dirs), None if cam is None else npy(cam), npy(shs), ref,
               npy(grad_rgb), gd, gc, gs)
        assert rel_err(npy(s.grad), gs) < 1e-5 and rel_err(npy(d.grad), gd) < 1e-4
        if cam is not None:
            assert rel_err(npy(c.grad), gc) < 1e-3
    grad_enc = torch.randn(P, 64, generator=g)
    for degree in range(8):
        d = dirs.to(device).requires_grad_()
        enc = sh_encode(d, degree)
        n = (degree + 1) ** 2
        enc.backward(grad_enc[:, :n].contiguous().to(device))
        ref, gref = np.zeros((P, n), np.float32), np.zeros((P, 3), np.float32)
        O.call("sh_encode_forward_f32", P, 3, degree, npy(dirs), ref)
        O.call("sh_encode_backward_f32", P, 3, degree, npy(grad_enc[:, :n].contiguous()), npy(dirs), gref)
        assert abs_err(npy(enc), ref) < 2e-6 * max(1, degree) and rel_err(npy(d.grad), gref) < 1e-5
    # a degree above 3 through SH -> RGB (36 coefficients + one unused row)
    hi = torch.randn(2000, 37, 3, generator=g) * 0.2
    d, s = dirs[:2000].to(device).requires_grad_(), hi.to(device).requires_grad_()
    rgb = SH_to_RGB(s, d, None, 5, True)
    rgb.backward(grad_rgb[:2000].to(device))
    ref, gd, gs = np.zeros((2000, 3), np.float32), np.zeros((2000, 3), np.float32), np.zeros((2000, 37, 3), np.float32)
    O.call("sh_to_rgb_forward_f32", 2000, 37, 5, 1, npy(dirs[:2000]), None, npy(hi), ref)
    O.call("sh_to_rgb_backward_f32", 2000, 37, 5, 1, npy(dirs[:2000]), None, npy(hi), ref, npy(grad_rgb[:2000]), gd, None, gs)
    assert abs_err(npy(rgb), ref) < 5e-6 and rel_err(npy(s.grad), gs) < 1e-5 and rel_err(npy(d.grad), gd) < 1e-4


def test_freq_encoder(device, oracle_mod):
    O = oracle_mod
    from fast_sp_gs_amd.ops import FreqEncoder
    g = torch.Generator().manual_seed(4)
    for D, deg, inc in ((3, 10, True), (1, 10, True), (3, 4, False)):
        x = torch.rand(777, D, generator=g) * 2 - 1
        enc = FreqEncoder(D, deg, inc)
        xd = x.to(device).requires_grad_()
        out = enc(xd)
        gout = torch.randn(out.shape, generator=g)
        out.backward(gout.to(device))
        ref = np.zeros(tuple(out.shape), np.float32)
        O.call("freq_encode_forward_f32", 777, D, deg, int(inc), 1.0, npy(x), ref)
        # sin/cos of arguments up to 2^9 differ between libm and the GPU by a few ulp of the argument
        assert abs_err(npy(out), ref) < 5e-5
        gref = np.zeros((777, D), np.float32)
        O.call("freq_encode_backward_f32", 777, D, deg, int(inc), 1.0, npy(gout), ref, gref)
        assert rel_err(npy(xd.grad), gref) < 1e-3


def test_cdist_top(device, oracle_mod, c1):
    O = oracle_mod
    from fast_sp_gs_amd.ops import cdist_top
    g = torch.Generator().manual_seed(5)
    for shape1, shape2 in (((3, 1000, 3), (3, 257, 3)), ((1500, 7), (33, 7))):
        x1, x2 = torch.randn(shape1, generator=g), torch.randn(shape2, generator=g)
        x2.view(-1, shape2[-1])[5] = x2.view(-1, shape2[-1])[2]  # duplicate rows: tie rules decide
        B = x1.numel() // (shape1[-2] * shape1[-1])
        for largest in (False, True):
            a, b = x1.to(device).requires_grad_(), x2.to(device).requires_grad_()
            dist, idx = cdist_top(a, b, largest)
            gd = torch.randn(dist.shape, generator=g)
            dist.backward(gd.to(device))
            rd, ri = np.zeros(dist.shape, np.float32), np.zeros(dist.shape, np.int64)
            O.call("cdist_top_forward_f32", B, shape1[-2], shape2[-2], shape1[-1], int(largest), npy(x1), npy(x2), rd, ri)
            assert np.array_equal(npy(idx), ri) and idx.dtype == torch.int64
            assert np.array_equal(npy(dist), rd)
            g1, g2 = np.zeros(shape1, np.float32), np.zeros(shape2, np.float32)
            O.call("cdist_top_backward_f32", B, shape1[-2], shape2[-2], shape1[-1], npy(x1), npy(x2), rd, ri, npy(gd), g1, g2)
            assert rel_err(npy(a.grad), g1) < 1e-5 and rel_err(npy(b.grad), g2) < 1e-4


def test_small_operators_in_the_other_element_types(device, oracle_mod, c1):
    """The element types the reference dispatches these operators on beside float32 (shencoder.cu:667,688 float / double /
    half; freqencoder.cu:76,98 and cdist_top.cu:48,116 float / double). The outputs keep the inputs' type."""
    O = oracle_mod
    from fast_sp_gs_amd._C import get_C_function
    from fast_sp_gs_amd.ops import FreqEncoder, cdist_top, sh_encode
    g = torch.Generator().manual_seed(11)
    dirs = c1['dirs'][:4000].double()
    dirs = torch.nn.functional.normalize(dirs + 1e-3 * torch.randn(dirs.shape, generator=g, dtype=torch.float64), dim=-1)
    P = dirs.shape[0]
    # -- SH encoder, double: double arithmetic on single-precision coefficients. An axis direction shows the coefficient
    # itself: Y_1 = -(double)(0.48860251190291987f) * y exactly.
    axis = torch.tensor([[0.0, 1.0, 0.0]], dtype=torch.float64, device=device)
    enc = sh_encode(axis, 1)
    assert enc.dtype == torch.float64 and enc[0, 1].item() == -float(np.float32(0.48860251190291987))
    for degree in (0, 3, 7):
        n = (degree + 1) ** 2
        d = dirs.to(device).requires_grad_()
        enc = sh_encode(d, degree)
        genc = torch.randn(P, n, generator=g, dtype=torch.float64)
        enc.backward(genc.to(device))
        ref, gref = np.zeros((P, n)), np.zeros((P, 3))
        O.call("sh_encode_forward_f64", P, 3, degree, npy(dirs), ref)
        O.call("sh_encode_backward_f64", P, 3, degree, npy(genc), npy(dirs), gref)
        # the oracle's double coefficients are exact, the operator's are the reference's float literals: 6e-8 relative
        # per coefficient, which the cancelling monomials of degree 4..7 (coefficients up to 1e2) turn into 1e-6
        tol = 3e-7 if degree <= 3 else 3e-6
        assert enc.dtype == torch.float64 and d.grad.dtype == torch.float64
        assert abs_err(npy(enc), ref) < tol and rel_err(npy(d.grad), gref) < tol
        if degree >= 2:  # two entries re-evaluated in double with the float literals: the arithmetic itself is double
            x, y, z = (npy(dirs)[:, i] for i in range(3))
            y4 = float(np.float32(1.0925484305920792)) * (x * y)
            y6 = float(np.float32(0.94617469575755997)) * (z * z) - float(np.float32(0.31539156525251999))
            assert np.abs(npy(enc)[:, 4] - y4).max() < 1e-15 and np.abs(npy(enc)[:, 6] - y6).max() < 1e-15
        # -- half. Degree <= 3 follows the reference's at::Half instantiation, which keeps its monomials and its backward
        # sums in half (shencoder.cu:31-33, 188-193): checked against oracle/sh_half.py, the numpy restatement of exactly
        # that, element for element up to the float expressions' contraction (one half ulp, rare). Degrees 4 - 7 are float
        # arithmetic rounded once on store (2^-11 relative), checked against the float64 basis on the same half inputs.
        dh = dirs.half()
        d = dh.to(device).requires_grad_()
        enc = sh_encode(d, degree)
        gh = genc.half()
        enc.backward(gh.to(device))
        assert enc.dtype == torch.float16 and d.grad.dtype == torch.float16
        if degree <= 3:
            from oracle import sh_half as H
            want, gwant = H.sh_encode_half(npy(dh), degree), H.sh_encode_backward_half(npy(gh), npy(dh), degree)
            # a contraction moves one term by a float ulp, which can cross a half rounding boundary: one half ulp of that
            # TERM, whose size is bounded by 4 |upstream| for the sums of the backward and by the entry for the forward
            term = 4.0 * np.abs(npy(gh).astype(np.float64)).max(axis=1, keepdims=True) if degree else 1.0
            for got_, want_, size in ((npy(enc), want, None), (npy(d.grad), gwant, term)):
                a, b = got_.astype(np.float64), want_.astype(np.float64)
                ulp = np.maximum(np.abs(b) if size is None else np.maximum(np.abs(b), size), 2.0 ** -14) * 2.0 ** -10
                assert (np.abs(a - b) <= ulp).all()
                assert (got_ == want_).mean() > 0.98
        else:
            O.call("sh_encode_forward_f64", P, 3, degree, npy(dh.double()), ref)
            O.call("sh_encode_backward_f64", P, 3, degree, npy(gh.double()), npy(dh.double()), gref)
            assert np.abs(npy(enc.double()) - ref).max() <= 2.0 ** -11 * max(np.abs(ref).max(), 1) * 1.01
            assert np.abs(npy(d.grad.double()) - gref).max() <= 2.0 ** -11 * np.abs(gref).max() * 1.01
    with pytest.raises(RuntimeError, match='element type'):
        get_C_function('sh_encode_forward')(dirs.to(device).bfloat16(), torch.empty(P, 4, device=device).bfloat16(), P, 3, 1)
    with pytest.raises(RuntimeError, match='dtype'):
        get_C_function('sh_encode_forward')(dirs.to(device), torch.empty(P, 4, device=device), P, 3, 1)
    # -- frequency encoder, double: the angle, its sine and cosine are single precision as in the reference's kernel, so
    # the check is against the restatement of that, to the few ulp by which sinf of arguments up to 2^9 differs
    for D, deg, inc in ((3, 10, True), (2, 6, False)):
        x = torch.rand(777, D, generator=g, dtype=torch.float64) * 2 - 1
        xd = x.to(device).requires_grad_()
        out = FreqEncoder(D, deg, inc, scale=0.75)(xd)
        gout = torch.randn(out.shape, generator=g, dtype=torch.float64)
        out.backward(gout.to(device))
        ref, exact = np.zeros(tuple(out.shape)), np.zeros(tuple(out.shape))
        O.call("freq_encode_forward_double_via_single", 777, D, deg, int(inc), 0.75, npy(x), ref)
        O.call("freq_encode_forward_f64", 777, D, deg, int(inc), 0.75, npy(x), exact)
        assert out.dtype == torch.float64 and abs_err(npy(out), ref) < 5e-7
        if deg == 10:  # ... which a double-precision evaluation would miss by the rounding of the angle times 2^9
            assert abs_err(npy(out), exact) > 4e-6
        gref = np.zeros((777, D))
        O.call("freq_encode_backward_f64", 777, D, deg, int(inc), 0.75, npy(gout), npy(out), gref)
        assert xd.grad.dtype == torch.float64 and rel_err(npy(xd.grad), gref) < 1e-12
    with pytest.raises(RuntimeError, match='element type'):
        get_C_function('freq_encode_forward')(x.to(device).half(), 4, True, 1.0)
    # -- nearest / farthest point, double: same sequential sums, so bit for bit
    for shape1, shape2 in (((2, 700, 3), (2, 129, 3)), ((900, 5), (33, 5))):
        x1 = torch.randn(shape1, generator=g, dtype=torch.float64)
        x2 = torch.randn(shape2, generator=g, dtype=torch.float64)
        x2.view(-1, shape2[-1])[5] = x2.view(-1, shape2[-1])[2]
        B = x1.numel() // (shape1[-2] * shape1[-1])
        for largest in (False, True):
            a, b = x1.to(device).requires_grad_(), x2.to(device).requires_grad_()
            dist, idx = cdist_top(a, b, largest)
            gd = torch.randn(dist.shape, generator=g, dtype=torch.float64)
            dist.backward(gd.to(device))
            rd, ri = np.zeros(dist.shape), np.zeros(dist.shape, np.int64)
            O.call("cdist_top_forward_f64", B, shape1[-2], shape2[-2], shape1[-1], int(largest), npy(x1), npy(x2), rd, ri)
            assert dist.dtype == torch.float64 and np.array_equal(npy(idx), ri) and np.array_equal(npy(dist), rd)
            g1, g2 = np.zeros(shape1), np.zeros(shape2)
            O.call("cdist_top_backward_f64", B, shape1[-2], shape2[-2], shape1[-1], npy(x1), npy(x2), rd, ri, npy(gd), g1, g2)
            assert rel_err(npy(a.grad), g1) < 1e-14 and rel_err(npy(b.grad), g2) < 1e-13
    with pytest.raises(RuntimeError, match='dtype'):
        get_C_function('cdist_top')(x1.to(device), x2.to(device).float())


def test_knn_and_lbs(device, oracle_mod, c1):
    O = oracle_mod
    from fast_sp_gs_amd._C import get_C_function
    pts, ctrl = c1['points'], c1['ctrl']
    N, M = pts.shape[0], ctrl.shape[0]
    for K in (1, 4, 8):
        d2, idx = get_C_function('knn_topk')(pts.to(device), ctrl.to(device), K)
        rd, ri = np.zeros((N, K), np.float32), np.zeros((N, K), np.int64)
        O.call("knn_topk_f32", N, M, 3, K, npy(pts), npy(ctrl), rd, ri)
        assert np.array_equal(npy(idx), ri) and np.array_equal(npy(d2), rd)
    # 5-dimensional features (xyz + hyper coordinates) take the generic path
    g = torch.Generator().manual_seed(6)
    x5, y5 = torch.randn(3000, 5, generator=g), torch.randn(100, 5, generator=g)
    d2, idx = get_C_function('knn_topk')(x5.to(device), y5.to(device), 4)
    rd, ri = np.zeros((3000, 4), np.float32), np.zeros((3000, 4), np.int64)
    O.call("knn_topk_f32", 3000, 100, 5, 4, npy(x5), npy(y5), rd, ri)
    assert np.array_equal(npy(idx), ri) and np.array_equal(npy(d2), rd)

    # 11 columns, K = 3: positions + 8 hyper features, the default configuration's search (exps/d_nerf.yaml:21-23)
    x11, y11 = torch.randn(5000, 11, generator=g), torch.randn(512, 11, generator=g)
    d2, idx = get_C_function('knn_topk')(x11.to(device), y11.to(device), 3)
    rd, ri = np.zeros((5000, 3), np.float32), np.zeros((5000, 3), np.int64)
    O.call("knn_topk_f32", 5000, 512, 11, 3, npy(x11), npy(y11), rd, ri)
    assert np.array_equal(npy(idx), ri) and np.array_equal(npy(d2), rd)


LBS_CASES = [  # (warp method with a local rotation | None without one, weight method)
    (None, 'weighted_kernel'),   # the reference's default configuration: translations only, kernel weights
    (None, 'dist'), ('LBS', 'dist'), ('LBS_c', 'dist'), ('LBS_c', 'weighted_kernel'), ('LBS', 'kernel'),
    ('LBS_c', 'W'), (None, 'given'), ('LBS', 'given'),
]


def _lbs_inputs(pts, ctrl, sp_t, sp_r, sp_s, K, warp_method, weight_method, seed, device):
    """Device inputs of one LBS case + the same values in float64 for the oracle."""
    from fast_sp_gs_amd._C import get_C_function
    g = torch.Generator().manual_seed(seed)
    N, M = pts.shape[0], ctrl.shape[0]
    d = lambda t: None if t is None else t.to(device).contiguous()
    d2, idx = get_C_function('knn_topk')(d(pts), d(ctrl), K)
    sp_rot = 0.3 * torch.randn(M, 4, generator=g) if warp_method is not None else None
    # radii around the typical neighbour distance so that the kernel weights are neither uniform nor one-hot
    typical = float(d2[d2 >= 0].median().sqrt()) if N else 0.1
    rho = torch.log(torch.full((M,), max(typical, 1e-3))) + 0.3 * torch.randn(M, generator=g)
    omega = torch.randn(M, generator=g)
    if weight_method == 'W':
        pair = torch.randn(N, K, generator=g).to(device)  # the caller's gather of sp_W rows
    elif weight_method == 'given':
        pair = torch.rand(N, K, generator=g).to(device)
    else:
        pair = d2
    kw = dict(temperature=0.01 if typical < 0.3 else 0.05, warp_method=warp_method, sp_rot=d(sp_rot),
              weight_method=weight_method,
              sp_log_radius=d(rho) if 'kernel' in weight_method else None,
              sp_weight_logit=d(omega) if weight_method == 'weighted_kernel' else None)
    f64 = lambda t: None if t is None else t.detach().cpu().double()
    okw = dict(weight_method=weight_method, temperature=kw['temperature'], warp_method=warp_method or 'LBS',
               sp_radius=f64(rho) if 'kernel' in weight_method else None,
               sp_weight=f64(omega) if weight_method == 'weighted_kernel' else None)
    oargs = [f64(pts), f64(ctrl), f64(sp_t), f64(sp_r), f64(sp_s), f64(sp_rot), f64(pair), idx.cpu()]
    return (d(pts), d(ctrl), d(sp_t), d(sp_r), d(sp_s), pair, idx), kw, oargs, okw


@pytest.mark.parametrize("warp_method,weight_method", LBS_CASES)
def test_lbs_forward(warp_method, weight_method, device, c1):
    from fast_sp_gs_amd._C import get_C_function
    from oracle import lbs as OL
    args, kw, oargs, okw = _lbs_inputs(c1['points'], c1['ctrl'], c1['sp_t'], c1['sp_r'], c1['sp_s'], 3, warp_method,
                                       weight_method, 40, device)
    dx, dr, ds, w = get_C_function('lbs_blend')(*args, **kw)
    rx, rr, rs, rw = OL.lbs_blend(*oargs, **okw)
    assert abs_err(npy(w), rw.numpy()) < 1e-5 and abs_err(npy(dx), rx.numpy()) < 1e-5
    assert abs_err(npy(dr), rr.numpy()) < 1e-5 and abs_err(npy(ds), rs.numpy()) < 1e-6
    assert float(w.max(dim=1).values.mean()) < 0.98 or weight_method == 'given'  # the weights really mix neighbours


def _lbs_backward_case(device, pts, ctrl, sp_t, sp_r, sp_s, K, warp_method, weight_method, seed):
    from fast_sp_gs_amd._C import get_C_function
    from oracle import lbs as OL
    N, M = pts.shape[0], ctrl.shape[0]
    S = 0 if sp_s is None else sp_s.shape[1]
    args, kw, oargs, okw = _lbs_inputs(pts, ctrl, sp_t, sp_r, sp_s, K, warp_method, weight_method, seed, device)
    g = torch.Generator().manual_seed(seed + 1000)
    gx, gr = torch.randn(N, 3, generator=g), torch.randn(N, 4, generator=g)
    gs = torch.randn(N, S, generator=g) if S else None
    d = lambda t: None if t is None else t.to(device).contiguous()
    print(f"[lbs backward] N={N} M={M} K={K} S={S} warp={warp_method} weights={weight_method}", flush=True)
    out = get_C_function('lbs_blend_backward')(*args, d(gx), d(gr), d(gs), **kw)
    torch.cuda.synchronize()
    ref = OL.lbs_blend_backward(*oargs, gx.double(), gr.double(), None if gs is None else gs.double(), **okw)
    pairs = [('g_points', 'points'), ('g_pair', 'pair_in'), ('g_sp_points', 'sp_points'), ('g_sp_t', 'sp_t'),
             ('g_sp_rot', 'sp_rot'), ('g_sp_r', 'sp_r'), ('g_sp_s', 'sp_s'), ('g_log_radius', 'sp_radius'),
             ('g_weight_logit', 'sp_weight')]
    for mine, theirs in pairs:
        a, b = out[mine], ref[theirs]
        assert (a is None) == (b is None), mine
        if a is None:
            continue
        b = b.numpy()
        if not np.abs(b).max() > 0:
            assert not npy(a).any(), mine   # e.g. no pivot term outside LBS_c, no position gradient without a rotation
            continue
        # sums of thousands of fp32 terms in a different association than the oracle's float64 sum
        assert rel_err(npy(a), b) < 2e-4, (mine, rel_err(npy(a), b))
    if weight_method in ('dist', 'kernel', 'weighted_kernel'):
        # the squared-distance gradient continues into both point sets
        O = __import__('oracle')
        gd = out['g_pair']
        g_x, g_y = get_C_function('knn_topk_backward')(args[0], args[1], args[6], gd)
        torch.cuda.synchronize()
        rx, ry = np.zeros((N, 3), np.float32), np.zeros((M, 3), np.float32)
        O.call("knn_topk_backward_f32", N, M, 3, K, npy(pts), npy(ctrl), npy(args[6]), npy(gd), rx, ry)
        assert rel_err(npy(g_x), rx) < 1e-5 and rel_err(npy(g_y), ry) < 2e-4


@pytest.mark.parametrize("warp_method,weight_method", LBS_CASES)
def test_lbs_backward_modes(warp_method, weight_method, device, oracle_mod, c1):
    """Every weight / warp combination at the default configuration's K = 3 (binned, atomic-free sums)."""
    _lbs_backward_case(device, c1['points'][:30011], c1['ctrl'], c1['sp_t'], c1['sp_r'], c1['sp_s'], 3, warp_method,
                       weight_method, seed=21)


def test_lbs_and_knn_backward_shapes(device, oracle_mod, c1):
    pts, ctrl = c1['points'][:30011], c1['ctrl']
    g = torch.Generator().manual_seed(22)
    # three scale residuals (what the network predicts before the caller slices them), K = 4
    s3 = 0.1 * torch.randn(512, 3, generator=g)
    _lbs_backward_case(device, pts, ctrl, c1['sp_t'], c1['sp_r'], s3, 4, 'LBS_c', 'weighted_kernel', seed=28)
    # no scale residuals, K = 8, fewer points than one block (LDS float atomics: not binned)
    small_ctrl = torch.rand(40, 3, generator=g) * 2 - 1
    _lbs_backward_case(device, pts[:100], small_ctrl, 0.1 * torch.randn(40, 3, generator=g),
                       0.2 * torch.randn(40, 4, generator=g), None, 8, 'LBS_c', 'weighted_kernel', seed=23)
    # more neighbours asked for than control points exist: the padded slots (index -1) carry nothing
    tiny_ctrl = torch.rand(3, 3, generator=g) * 2 - 1
    _lbs_backward_case(device, pts[:500], tiny_ctrl, 0.1 * torch.randn(3, 3, generator=g),
                       0.2 * torch.randn(3, 4, generator=g), 0.1 * torch.randn(3, 2, generator=g), 5, 'LBS', 'dist',
                       seed=24)
    # K = 4 with a padded slot (3 control points), through the binned variant
    for wm in ('dist', 'kernel'):
        _lbs_backward_case(device, pts[:700], tiny_ctrl, 0.1 * torch.randn(3, 3, generator=g),
                           0.2 * torch.randn(3, 4, generator=g), 0.1 * torch.randn(3, 2, generator=g), 4, 'LBS_c', wm,
                           seed=26)
    # more points than one pass of the launch covers: every block bins several chunks into its table
    many = torch.rand(280_001, 3, generator=g) * 2 - 1
    _lbs_backward_case(device, many, ctrl, c1['sp_t'], c1['sp_r'], c1['sp_s'], 3, None, 'weighted_kernel', seed=27)
    # a control set whose table exceeds LDS takes the device-scope atomic path
    big_ctrl = torch.rand(2500, 3, generator=g) * 2 - 1
    _lbs_backward_case(device, pts[:20000], big_ctrl, 0.1 * torch.randn(2500, 3, generator=g),
                       0.2 * torch.randn(2500, 4, generator=g), 0.1 * torch.randn(2500, 2, generator=g), 4, 'LBS_c',
                       'weighted_kernel', seed=25)


@pytest.mark.parametrize("local_frame,is_blender", [(True, True), (False, False)])
def test_deform_branch_autograd(local_frame, is_blender, device):
    """superpoint_deform and the MLP are differentiable end to end: gradients through the HIP backward kernels equal
    torch autograd of the same formulas written with torch ops on the device. With a local-rotation head the warp is
    the rigid blend about the control points (LBS_c), without one the translations are blended (the reference's default
    configuration); with the D-NeRF time network in front, its parameters get their gradient through the MLP's input."""
    from fast_sp_gs_amd.deform import DeformNetwork, superpoint_deform
    g = torch.Generator().manual_seed(31)
    N, M, K = 5000, 64, 3
    pts = (torch.rand(N, 3, generator=g) * 2 - 1).to(device)
    ctrl = (torch.rand(M, 3, generator=g) * 2 - 1).to(device).requires_grad_()
    hyper = (0.1 * torch.randn(N, 8, generator=g)).to(device).requires_grad_()
    sp_hyper = (0.1 * torch.randn(M, 8, generator=g)).to(device).requires_grad_()
    rho = torch.full((M,), float(np.log(0.25)), device=device).requires_grad_()
    omega = torch.randn(M, generator=g).to(device).requires_grad_()
    torch.manual_seed(32)
    net = DeformNetwork(t_degree=6 if is_blender else 10, is_blender=is_blender, local_frame=local_frame).to(device)
    for head in net._heads():
        torch.nn.init.normal_(head.weight, std=0.05)  # the default 1e-5 would make every gradient vanish
    t = torch.full((1,), 0.3, device=device)
    gx, gr, gs = (torch.randn(N, c, generator=g).to(device) for c in (3, 4, 2))

    def loss_of(d_xyz, d_rot, d_scale):
        return (d_xyz * gx).sum() + (d_rot * gr).sum() + (d_scale * gs).sum()

    c_xyz, c_rot, c_scale, c_local = net(ctrl.detach(), t)
    assert c_xyz.requires_grad and (c_local is not None) == local_frame
    d_xyz, d_rot, d_scale, w, idx = superpoint_deform(
        pts, ctrl, c_xyz, c_rot, c_scale[:, :2], sp_rot=c_local, K=K, warp_method='LBS_c',
        LBS_method='weighted_kernel', sp_radius=rho, sp_weight=omega, feature=hyper, sp_feature=sp_hyper)
    leaves = [ctrl, hyper, sp_hyper, rho, omega]
    leaf_names = ['sp_points', 'hyper', 'sp_hyper', 'sp_radius', 'sp_weight']
    params = list(net.parameters())
    grads = torch.autograd.grad(loss_of(d_xyz, d_rot, d_scale), leaves + params, allow_unused=True)

    # the same computation with torch ops (fp32 network, the reference's expressions: network.py:498-573)
    r_xyz, r_rot, r_scale, r_local = net.forward_fp32(ctrl.detach(), t)
    x = torch.cat([pts, hyper], -1)
    y = torch.cat([ctrl.detach(), sp_hyper], -1)
    diff = x[:, None, :] - y[idx]
    nn_dist = (diff * diff).sum(-1)
    wt = torch.exp(-nn_dist / (2 * torch.exp(rho)[idx] ** 2)) * torch.sigmoid(omega)[idx] + 1e-7
    wt = wt / wt.sum(-1, keepdim=True)
    assert float((wt.detach() - w).abs().max()) < 1e-4
    if local_frame:
        q = r_local + torch.tensor([0, 0, 0, 1.0], device=device)
        q = q / q.norm(dim=-1, keepdim=True)
        qx, qy, qz, qs = q.unbind(-1)
        R = torch.stack([1 - 2 * (qy * qy + qz * qz), 2 * (qx * qy - qz * qs), 2 * (qy * qs + qx * qz),
                         2 * (qx * qy + qz * qs), 1 - 2 * (qx * qx + qz * qz), 2 * (qy * qz - qx * qs),
                         2 * (qx * qz - qy * qs), 2 * (qx * qs + qy * qz), 1 - 2 * (qx * qx + qy * qy)], -1).view(M, 3, 3)
        tt = r_xyz + ctrl - torch.einsum('mab,mb->ma', R, ctrl)
        moved = torch.einsum('nkab,nb->nka', R[idx], pts) + tt[idx]
        e_xyz = (wt[..., None] * moved).sum(1) - pts
    else:
        e_xyz = (wt[..., None] * r_xyz[idx]).sum(1)
    e_rot = (wt[..., None] * r_rot[idx]).sum(1)
    e_scale = (wt[..., None] * r_scale[:, :2][idx]).sum(1)
    assert float((e_xyz - d_xyz).detach().abs().max()) < 2e-2 * float(e_xyz.detach().abs().max())  # bf16 forward
    ref = torch.autograd.grad(loss_of(e_xyz, e_rot, e_scale), leaves + params, allow_unused=True)
    seen_timenet = False
    for name, a, b in zip(leaf_names + [n for n, _ in net.named_parameters()], grads, ref):
        if b is None or not float(b.abs().max()) > 0:
            assert a is None or not float(a.abs().max()) > 0, name  # e.g. sp_points without a pivot or a rotation
            continue
        assert a is not None, name
        if name in leaf_names:
            # the HIP forward runs the layers in bf16, so the values the chain rule is evaluated at differ by ~1e-2 rel
            scale = float(b.abs().max())
            assert float((a - b).abs().max()) <= 5e-2 * scale + 1e-12, (name, float((a - b).abs().max()), scale)
        else:
            # network parameters: the bf16 and fp32 forwards mask a few near-zero ReLU units differently, which moves
            # sums of random-sign terms element-wise; the direction of the gradient is what has to agree
            cos = float((a * b).sum() / (a.norm() * b.norm()).clamp_min(1e-30))
            assert cos > 0.97, (name, cos)
            seen_timenet |= name.startswith('timenet')
    assert seen_timenet == is_blender


def test_calc_LBS_weight_and_warp_mirror_the_fused_path(device):
    """`calc_LBS_weight` (K-NN on the HIP kernel, the reference's torch weight expressions) followed by `warp` on those
    weights gives what `superpoint_deform` computes in one kernel, values and gradients."""
    from fast_sp_gs_amd.deform import calc_LBS_weight, superpoint_deform, warp
    g = torch.Generator().manual_seed(33)
    N, M, K = 3000, 40, 3
    dev = lambda t: t.to(device)
    pts = dev(torch.rand(N, 3, generator=g) * 2 - 1)
    mk = lambda *shape, s=0.2: dev(s * torch.randn(*shape, generator=g)).requires_grad_()
    ctrl, sp_t, sp_r, sp_s, sp_rot = mk(M, 3, s=0.6), mk(M, 3), mk(M, 4), mk(M, 3), mk(M, 4)
    rho, omega = (dev(torch.full((M,), float(np.log(0.3))))).requires_grad_(), mk(M, s=1.0)
    gx, gr, gs = (dev(torch.randn(N, c, generator=g)) for c in (3, 4, 3))
    leaves = [ctrl, sp_t, sp_r, sp_s, sp_rot, rho, omega]
    for rot, method in ((sp_rot, 'LBS_c'), (sp_rot, 'LBS'), (None, 'LBS')):
        use = [l for l in leaves if not (l is sp_rot and rot is None)]
        a = superpoint_deform(pts, ctrl, sp_t, sp_r, sp_s, sp_rot=rot, K=K, warp_method=method,
                              LBS_method='weighted_kernel', sp_radius=rho, sp_weight=omega)
        ga = torch.autograd.grad((a[0] * gx).sum() + (a[1] * gr).sum() + (a[2] * gs).sum(), use, allow_unused=True)
        w, idx = calc_LBS_weight(pts, ctrl, K=K, LBS_method='weighted_kernel', sp_radius=rho, sp_weight=omega)
        b = warp(pts, ctrl, sp_t, sp_r, sp_s, rot, w, idx, method)
        gb = torch.autograd.grad((b[0] * gx).sum() + (b[1] * gr).sum() + (b[2] * gs).sum(), use, allow_unused=True)
        assert torch.equal(idx, a[4]) and float((w - a[3]).abs().max()) < 1e-5
        for x, y in zip(a[:3], b):
            assert float((x - y).abs().max()) < 1e-5
        for x, y in zip(ga, gb):
            assert (x is None) == (y is None)
            if x is not None:
                assert float((x - y).abs().max()) <= 2e-4 * max(float(y.abs().max()), 1e-6)


def test_warp_largest_matches_oracle(device):
    """warp_method 'largest' (network.py:555-561, assignment :594): values and gradients of `warp` / `superpoint_deform`
    against the float64 oracle and its autograd; the assignment defaults to the neighbour of largest weight and can be
    handed in."""
    from oracle import lbs as OL
    from fast_sp_gs_amd.deform import assign_superpoints, superpoint_deform, warp
    g = torch.Generator().manual_seed(71)
    N, M, K = 4000, 48, 4
    mk = lambda *shape, s=0.2: (s * torch.randn(*shape, generator=g))
    pts = torch.rand(N, 3, generator=g) * 2 - 1
    ctrl, sp_t, sp_r, sp_s, sp_rot = mk(M, 3, s=0.6), mk(M, 3), mk(M, 4), mk(M, 2), mk(M, 4, s=0.4)
    gx, gr, gs = mk(N, 3, s=1.0), mk(N, 4, s=1.0), mk(N, 2, s=1.0)
    names = ['ctrl', 'sp_t', 'sp_r', 'sp_s', 'sp_rot']
    dev_leaves = [t.to(device).requires_grad_() for t in (ctrl, sp_t, sp_r, sp_s, sp_rot)]
    d_xyz, d_rot, d_scale, w, idx = superpoint_deform(pts.to(device), *dev_leaves[:4], sp_rot=dev_leaves[4], K=K,
                                                      temperature=0.05, warp_method='largest', LBS_method='dist')
    got = torch.autograd.grad((d_xyz * gx.to(device)).sum() + (d_rot * gr.to(device)).sum() +
                              (d_scale * gs.to(device)).sum(), dev_leaves, allow_unused=True)
    p2sp = assign_superpoints(w, idx)
    # oracle on the GPU's neighbour lists (float64), distances recomputed there
    leaves = [t.double().requires_grad_() for t in (ctrl, sp_t, sp_r, sp_s, sp_rot)]
    idx_c = idx.cpu()
    d2 = ((pts.double()[:, None] - leaves[0][idx_c]) ** 2).sum(-1)
    w_ref = OL.lbs_weights(d2, idx_c, M, 'dist', 0.05)
    assert float((w.cpu().double() - w_ref.detach()).abs().max()) < 1e-5
    assert torch.equal(p2sp.cpu(), torch.gather(idx_c, -1, w_ref.argmax(-1, keepdim=True))[:, 0])
    r_xyz, r_rot, r_scale = OL.warp(pts.double(), *leaves[:4], leaves[4], w_ref, idx_c, 'largest')
    for a, b in ((d_xyz, r_xyz), (d_rot, r_rot), (d_scale, r_scale)):
        assert float((a.detach().cpu().double() - b.detach()).abs().max()) <= 2e-5 * max(float(b.abs().max()), 1.0)
    want = torch.autograd.grad((r_xyz * gx.double()).sum() + (r_rot * gr.double()).sum() + (r_scale * gs.double()).sum(),
                               leaves, allow_unused=True)
    for name, a, b in zip(names, got, want):
        assert a is not None and b is not None, name
        assert float((a.cpu().double() - b).abs().max()) <= 1e-3 * float(b.abs().max()) + 1e-9, name
    # an assignment handed in is used as it is: points follow control point 7 rigidly
    fixed = torch.full((N,), 7, dtype=torch.int64, device=device)
    d_fixed = warp(pts.to(device), *[t.detach() for t in dev_leaves[:4]], dev_leaves[4].detach(), w, idx, 'largest',
                   p2sp=fixed)[0]
    r_fixed = OL.warp(pts.double(), ctrl.double(), sp_t.double(), sp_r.double(), sp_s.double(), sp_rot.double(), w_ref,
                      idx_c, 'largest', p2sp=fixed.cpu())[0]
    assert float((d_fixed.cpu().double() - r_fixed).abs().max()) < 2e-5


@pytest.mark.parametrize("B,D,p_degree,t_degree", [(512, 8, 10, 10), (500, 8, 10, 6), (70, 4, 4, 2), (1, 3, 2, 1)])
def test_deform_mlp_backward_mfma(B, D, p_degree, t_degree, device):
    """Weight / bias / input gradients from the MFMA backward kernels. The checkers for this floating-point kernel:
      * oracle/mlp.py with the kernels' roundings -- the chain rule evaluated at the stored bf16 hidden states (their
        zeros are the ReLU mask) with bf16 operands where the matrix cores take them and every dZ rounded to bf16, in
        float64; without the roundings that function equals torch.autograd (tests/test_oracle_mlp.py): agreement to
        1e-3 of each tensor's largest entry;
      * torch autograd of the fp32 network: same direction (cosine > 0.98); element-wise it differs more because a
        hidden unit whose pre-activation is within bf16 rounding of zero is masked differently by the two forwards and
        each such unit moves a sum of B random-sign terms by a whole term.
    Batch sizes cover a partial 32-row block and a single row."""
    from fast_sp_gs_amd._C import get_C_function
    from fast_sp_gs_amd.deform import DeformNetwork
    torch.manual_seed(41)
    net = DeformNetwork(D=D, p_degree=p_degree, t_degree=t_degree).to(device)
    for head in (net.gaussian_warp, net.gaussian_rotation, net.gaussian_scaling):
        torch.nn.init.normal_(head.weight, std=0.05)
        torch.nn.init.normal_(head.bias, std=0.05)
    for l in net.linear:
        torch.nn.init.normal_(l.bias, std=0.05)
    g = torch.Generator().manual_seed(42)
    x = (torch.rand(B, 3, generator=g) * 2 - 1).to(device)
    t = torch.full((1,), 0.7, device=device)
    go = [torch.randn(B, c, generator=g).to(device) for c in (3, 4, 3)]
    print(f"[mlp backward] B={B} D={D} Din={net.input_ch}", flush=True)
    outs = net(x, t)[:3]
    params = list(net.parameters())
    names = [n for n, _ in net.named_parameters()]
    got = dict(zip(names, torch.autograd.grad(sum((o * g_).sum() for o, g_ in zip(outs, go)), params)))
    torch.cuda.synchronize()

    # The checker is oracle/mlp.py with its rounding switch on: the chain rule written out by hand in float64 (pinned on
    # the CPU against torch.autograd, tests/test_oracle_mlp.py) with bf16 operands where the matrix cores take them,
    # evaluated at the hidden states the forward kernel stored (their zeros are the ReLU mask). What is left is fp32
    # summation order plus the rare dZ element whose fp32 sum sits on a bf16 rounding boundary (one bf16 ulp of one term
    # of a B-term sum): 1e-3 of each tensor's largest entry.
    from oracle import mlp as OM
    from fast_sp_gs_amd.deform import _DeformMlp
    cpu = lambda t_: t_.detach().cpu()
    with torch.no_grad():
        x_enc = net.encode(x, t)
        packed, bias = net._packed
        _, saved = get_C_function('mlp_forward')(x_enc, packed, bias, D, net.skip, 10, True)
        hidden = list(cpu(saved.view(torch.bfloat16)).double())  # D x [B, 256]
        Wh = torch.cat([net.gaussian_warp.weight, net.gaussian_rotation.weight, net.gaussian_scaling.weight], 0)
        g_out = torch.cat(go, -1)
        ref = OM.mlp_backward(cpu(x_enc), [cpu(l.weight) for l in net.linear], cpu(Wh), net.skip, cpu(g_out), hidden,
                              round_bf16=True)
        want = {}
        for name, lo, hi in (('gaussian_warp', 0, 3), ('gaussian_rotation', 3, 7), ('gaussian_scaling', 7, 10)):
            want[name + '.weight'], want[name + '.bias'] = ref['head_w'][lo:hi], ref['head_b'][lo:hi]
        for l in range(D):
            want[f'linear.{l}.weight'], want[f'linear.{l}.bias'] = ref['weights'][l], ref['biases'][l]
    for name in names:
        a, b = cpu(got[name]).double(), want[name]
        assert a.shape == b.shape and bool(torch.isfinite(a).all()), name
        scale = float(b.abs().max())
        assert float((a - b).abs().max()) <= 1e-3 * scale + 1e-9, (name, float((a - b).abs().max()), scale)
    # the gradient of the encoded input (what reaches the time network): dZ_0 W_0 + dZ_{skip+1} W_{skip+1}[:, :Din]
    leaf = x_enc.detach().clone().requires_grad_()
    out = _DeformMlp.apply(leaf, packed, bias, net._packed_t, net._heads_w, D, net.skip, 10, *net._mlp_parameters())
    g_leaf, = torch.autograd.grad((out * g_out).sum(), [leaf])
    # (a row of it is a sum over 2 x 256 hidden units of dZ, each of which may sit on a bf16 rounding boundary: 3e-3)
    scale = float(ref['x'].abs().max())
    assert float((cpu(g_leaf).double() - ref['x']).abs().max()) <= 3e-3 * scale + 1e-9

    refs = net.forward_fp32(x, t)[:3]
    auto = torch.autograd.grad(sum((o * g_).sum() for o, g_ in zip(refs, go)), params)
    for name, b in zip(names, auto):
        a = got[name]
        if B >= 64:
            cos = float((a * b).sum() / (a.norm() * b.norm()).clamp_min(1e-30))
            assert cos > 0.98, (name, cos)
    # a second call after an optimiser step re-packs the weights (version counters changed)
    with torch.no_grad():
        for p_ in params:
            p_.add_(0.01 * torch.randn_like(p_))
    outs2 = net(x, t)[:3]
    refs2 = net.forward_fp32(x, t)[:3]
    for a, b in zip(outs2, refs2):
        assert float((a - b).abs().max()) <= 3e-2 * float(b.abs().max()) + 1e-6


def test_sparse_adam(device, oracle_mod):
    O = oracle_mod
    from fast_sp_gs_amd.sparse_gaussian_adam import SparseGaussianAdam
    g = torch.Generator().manual_seed(7)
    N = 5000
    shapes = [(N, 3), (N, 16, 3), (N, 1), (N, 2), (N, 4)]  # xyz, sh, opacity, scales, rotations: M = 3, 48, 1, 2, 4
    params = [torch.nn.Parameter(torch.randn(s, generator=g).to(device)) for s in shapes]
    opt = SparseGaussianAdam([{'params': [p], 'lr': 1.6e-4, 'eps': 1e-15} for p in params], lr=1.6e-4, eps=1e-15)
    ref_p = [npy(p) for p in params]
    ref_m = [np.zeros_like(p) for p in ref_p]
    ref_v = [np.zeros_like(p) for p in ref_p]
    for step in range(1, 4):
        vis = torch.rand(N, generator=g) < 0.6
        grads = [torch.randn(s, generator=g) for s in shapes]
        for p, gr in zip(params, grads):
            p.grad = gr.to(device)
        opt.set_before_step(vis.to(device), N)
        opt.step()
        # the reference forms the rate on a float32 step TENSOR (sparse_gaussian_adam.py:42-46): float32 arithmetic,
        # widened to double when it is handed to the kernel
        step_t = torch.tensor(float(step), dtype=torch.float32)
        lr = float(1.6e-4 * (1 - 0.999 ** step_t) ** 0.5 / (1 - 0.9 ** step_t))
        assert lr != 1.6e-4 * (1 - 0.999 ** step) ** 0.5 / (1 - 0.9 ** step)  # ... which is not the double expression
        for k, s in enumerate(shapes):
            Mk = int(np.prod(s[1:]))
            O.call("adam_masked_update_f32", N, Mk, npy(vis.to(torch.uint8)), lr, 0.9, 0.999, 1e-15, ref_p[k],
                   npy(grads[k]), ref_m[k], ref_v[k])
    for p, r in zip(params, ref_p):
        assert np.array_equal(npy(p), r)  # same operation order, contraction off on both sides: bit exact
    for p, r in zip(params, ref_m):
        assert np.array_equal(npy(opt.state[p]['exp_avg']), r)


def test_multi_tensor_entry_points_match_the_single_ones(device):
    """`AdamMasksedUpdatedMulti` against `AdamMasksedUpdated` tensor by tensor (own rate and eps each, more tensors than
    one launch takes through the optimiser class), and `mlp_pack_all` against the separate packing operators plus
    torch.cat: bit for bit."""
    from fast_sp_gs_amd._C import get_C_function
    from fast_sp_gs_amd.deform import DeformNetwork
    from fast_sp_gs_amd.sparse_gaussian_adam import SparseGaussianAdam
    g = torch.Generator().manual_seed(17)
    N = 3001
    shapes = [(N, 3), (N, 16, 3), (N, 1), (N, 2), (N, 4), (N, 5), (N, 8)]
    mk = lambda: [torch.randn(s, generator=g).to(device) for s in shapes]
    p1, gr, m1 = mk(), mk(), mk()
    v1 = [t.abs() for t in mk()]
    p2, m2, v2 = [t.clone() for t in p1], [t.clone() for t in m1], [t.clone() for t in v1]
    vis = (torch.rand(N, generator=g) < 0.5).to(device)
    lrs = [1e-3 * (k + 1) for k in range(len(shapes))]
    epss = [1e-15 * 10 ** k for k in range(len(shapes))]
    get_C_function('AdamMasksedUpdatedMulti')(p1, gr, m1, v1, vis, lrs, 0.9, 0.999, epss, N)
    for k, s_ in enumerate(shapes):
        get_C_function('AdamMasksedUpdated')(p2[k], gr[k], m2[k], v2[k], vis, lrs[k], 0.9, 0.999, epss[k], N,
                                             p2[k].numel() // N)
    for a, b in zip(p1 + m1 + v1, p2 + m2 + v2):
        assert torch.equal(a, b)
    assert not torch.equal(p1[1][vis], mk()[1][vis])  # something moved
    # 14 groups: two launches inside the optimiser
    params = [torch.nn.Parameter(torch.randn(N, 1 + k % 4, generator=g).to(device)) for k in range(14)]
    before = [p_.detach().clone() for p_ in params]
    opt = SparseGaussianAdam([{'params': [p_], 'lr': 1e-3 * (k + 1)} for k, p_ in enumerate(params)], lr=1e-3, eps=1e-15)
    for p_ in params:
        p_.grad = torch.randn(p_.shape, generator=g).to(device)
    opt.set_before_step(vis, N)
    opt.step()
    for k, (p_, b) in enumerate(zip(params, before)):
        assert torch.equal(p_[~vis], b[~vis]) and not torch.equal(p_[vis], b[vis]), k
        # first step of Adam: |update| = lr * sqrt(1 - b2) / (1 - b1) * (1 - b1) |g| / (sqrt((1 - b2) g^2) + eps) = lr
        assert float(((p_ - b)[vis].abs() - 1e-3 * (k + 1)).abs().max()) < 1e-3 * (k + 1) * 1e-3
    with pytest.raises(RuntimeError):
        get_C_function('AdamMasksedUpdatedMulti')(p1, gr[:-1], m1, v1, vis, lrs, 0.9, 0.999, epss, N)

    net = DeformNetwork().to(device)
    with torch.no_grad():
        for p_ in net.parameters():
            p_.add_(0.05 * torch.randn(p_.shape, generator=g).to(device))
    heads = (net.gaussian_warp, net.gaussian_rotation, net.gaussian_scaling)
    weights = [l.weight.detach() for l in net.linear]
    packed, packed_t, bias, heads_w = get_C_function('mlp_pack_all')(
        weights, [l.bias.detach() for l in net.linear], [h.weight.detach() for h in heads],
        [h.bias.detach() for h in heads], net.skip)
    hw = torch.cat([h.weight.detach() for h in heads], 0).contiguous()
    assert torch.equal(packed, get_C_function('mlp_pack_weights')(weights, hw, net.skip))
    assert torch.equal(packed_t, get_C_function('mlp_pack_transposed')(weights))
    assert torch.equal(bias, torch.cat([l.bias.detach() for l in net.linear] + [h.bias.detach() for h in heads]))
    assert torch.equal(heads_w, hw)
    only = get_C_function('mlp_pack_all')(weights, [l.bias.detach() for l in net.linear],
                                          [h.weight.detach() for h in heads], [h.bias.detach() for h in heads],
                                          net.skip, False)
    assert only[1] is None and torch.equal(only[0], packed)


@pytest.mark.parametrize("S,log_scales", [(2, False), (3, True), (2, True)])
def test_deform_apply_matches_the_torch_operators(S, log_scales, device):
    """points + d_xyz, act(scales) + d_scale, normalize(rot + d_rot) (network.py:630, :643, :645) in one kernel each way
    against the torch operators the reference runs, forward and through autograd; one rotation row sums to zero."""
    from fast_sp_gs_amd.deform import deform_apply
    g = torch.Generator().manual_seed(23)
    N = 7001
    mk = lambda *s_: torch.randn(*s_, generator=g).to(device)
    base = [mk(N, 3), mk(N, 3) * 0.1, mk(N, S) * 0.5, mk(N, S) * 0.1, mk(N, 4), mk(N, 4) * 0.1]
    base[5][7] = -base[4][7]  # rot + d_rot == 0 there: normalize's floor on the norm decides
    a = [t.clone().requires_grad_(True) for t in base]
    b = [t.clone().requires_grad_(True) for t in base]
    out = deform_apply(*a, log_scales=log_scales)
    ref = (b[0] + b[1], (torch.exp(b[2]) if log_scales else b[2]) + b[3],
           torch.nn.functional.normalize(b[4] + b[5], dim=-1))
    for o, r in zip(out, ref):
        assert o.shape == r.shape and float((o - r).abs().max()) <= 2e-6 * max(1.0, float(r.abs().max()))
    assert not out[2][7].any()
    go = [mk(*o.shape) for o in out]
    go[2][7] *= 1e-9  # keeps g / 1e-12 finite in float32
    sum((o * g_).sum() for o, g_ in zip(out, go)).backward()
    sum((r * g_).sum() for r, g_ in zip(ref, go)).backward()
    for k, (x, y) in enumerate(zip(a, b)):
        assert rel_err(npy(x.grad), npy(y.grad)) < 1e-5, k
    # only the deltas need gradients (parameters detached)
    c = [t.clone().requires_grad_(k % 2 == 1) for k, t in enumerate(base)]
    out2 = deform_apply(*c, log_scales=log_scales)
    sum((o * g_).sum() for o, g_ in zip(out2, go)).backward()
    assert all((t.grad is None) == (k % 2 == 0) for k, t in enumerate(c))
    assert torch.equal(c[5].grad, a[5].grad) and torch.equal(c[1].grad, a[1].grad)


def test_full_size_properties(device):
    """Full benchmark-size runs checked through size-independent properties (no oracle at this size)."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function
    c = scenes.config1(n_dirs=1_000_000, n_points=200_000, n_ctrl=512)
    pts, ctrl = c['points'].to(device), c['ctrl'].to(device)
    d2, idx = get_C_function('knn_topk')(pts, ctrl, 4)
    assert bool((d2[:, 1:] >= d2[:, :-1]).all()) and int(idx.min()) >= 0 and int(idx.max()) < 512
    # distances recomputed from the returned indices, and the nearest one agrees with cdist_top's minimum
    rec = (pts[:, None, :] - ctrl[idx]).square().sum(-1)
    assert float((rec - d2).abs().max()) < 1e-6
    dist, i1 = get_C_function('cdist_top')(pts, ctrl, False)
    assert float((dist.square() - d2[:, 0]).abs().max()) < 1e-6
    # SH encoder at 1M directions: rows are orthonormal-basis evaluations, so |Y|^2 sums to (degree+1)^2 / (4 pi)
    dirs = c['dirs'].to(device)
    enc = torch.empty(dirs.shape[0], 16, device=device)
    get_C_function('sh_encode_forward')(dirs, enc, dirs.shape[0], 3, 3)
    assert float((enc.square().sum(-1) - 16 / (4 * np.pi)).abs().max()) < 1e-5
    # SH encoder backward at 1M directions. |Y(d)|^2 is constant on the sphere, so with the encoding itself as upstream
    # gradient (the gradient of |Y|^2 / 2) nothing may be left tangentially to the sphere, whatever polynomial extension
    # off the sphere the basis is written in; and the backward is linear in the upstream gradient.
    B = dirs.shape[0]
    g1, g2 = torch.empty(B, 3, device=device), torch.empty(B, 3, device=device)
    get_C_function('sh_encode_backward')(enc, dirs, B, 3, 3, g1)
    tangential = g1 - (g1 * dirs).sum(-1, keepdim=True) * dirs
    assert float(tangential.abs().max()) < 2e-5
    up = torch.randn(B, 16, generator=torch.Generator().manual_seed(2)).to(device)
    get_C_function('sh_encode_backward')(up, dirs, B, 3, 3, g1)
    get_C_function('sh_encode_backward')(up * -3.0, dirs, B, 3, 3, g2)
    assert float((g2 + 3.0 * g1).abs().max()) < 1e-5 * max(1.0, float(g1.abs().max()))
    # SH -> RGB at 1M points through the other kernel family: positions on the unit sphere seen from the origin give
    # the directions themselves, so the colours are the encoder's rows contracted with the coefficients, + 0.5, clamped;
    # the backward's coefficient gradient is the outer product of the clamped upstream gradient and the same rows
    shs = c['shs'].to(device)
    origin = torch.zeros(3, device=device)
    rgb = get_C_function('SH_to_RGB_forward')(dirs, origin, shs, 3, True)
    want = torch.clamp_min(torch.einsum('pk,pkc->pc', enc.double(), shs.double()) + 0.5, 0.0)
    assert float((rgb.double() - want).abs().max()) < 2e-6
    g_rgb = torch.randn(B, 3, generator=torch.Generator().manual_seed(3)).to(device)
    g_sh, g_pos, g_cam = torch.empty_like(shs), torch.empty_like(dirs), torch.zeros(3, device=device)
    get_C_function('SH_to_RGB_backward')(3, True, dirs, origin, shs, rgb, g_rgb, g_pos, g_cam, g_sh)
    masked = (g_rgb * (rgb > 0)).double()
    assert float((g_sh.double() - enc.double()[:, :, None] * masked[:, None, :]).abs().max()) < 2e-6 * float(g_rgb.abs().max())
    assert float((g_pos * dirs).sum(-1).abs().max()) < 1e-4  # a direction's gradient has no radial part
    assert float((g_cam.double() + g_pos.double().sum(0)).abs().max()) < 1e-3 * max(1.0, float(g_pos.abs().sum(0).max()))


def test_full_size_against_the_oracle(device, oracle_mod):
    """The stand-alone operators at the benchmark's sizes against the oracle itself: SH encoder forward / backward at
    1M directions, K-NN at 200 000 x 512 (k = 4) bit for bit, its distances' backward, the LBS blend forward against the
    float64 restatement, and the masked Adam at 300 000 x 58 floats bit for bit."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    import oracle.lbs as OL
    O = oracle_mod
    c = scenes.config1(n_dirs=1_000_000, n_points=200_000, n_ctrl=512)
    dirs = c['dirs']
    B = dirs.shape[0]
    g = torch.Generator().manual_seed(21)
    enc, g_dirs = torch.empty(B, 16, device=device), torch.empty(B, 3, device=device)
    up = torch.randn(B, 16, generator=g)
    f('sh_encode_forward')(dirs.to(device), enc, B, 3, 3)
    f('sh_encode_backward')(up.to(device), dirs.to(device), B, 3, 3, g_dirs)
    ref, gref = np.zeros((B, 16), np.float32), np.zeros((B, 3), np.float32)
    O.call("sh_encode_forward_f32", B, 3, 3, npy(dirs), ref)
    O.call("sh_encode_backward_f32", B, 3, 3, npy(up), npy(dirs), gref)
    print(f"[full config 1] sh_encode 1M: forward abs err {abs_err(npy(enc), ref):.2e}, backward rel err "
          f"{rel_err(npy(g_dirs), gref):.2e}", flush=True)
    assert abs_err(npy(enc), ref) < 6e-6 and rel_err(npy(g_dirs), gref) < 1e-5

    pts, ctrl = c['points'], c['ctrl']
    N, M, K = pts.shape[0], ctrl.shape[0], 4
    d2, idx = f('knn_topk')(pts.to(device), ctrl.to(device), K)
    rd, ri = np.zeros((N, K), np.float32), np.zeros((N, K), np.int64)
    O.call("knn_topk_f32", N, M, 3, K, npy(pts), npy(ctrl), rd, ri)
    assert np.array_equal(npy(idx), ri) and np.array_equal(npy(d2), rd)
    gd = torch.randn(N, K, generator=g)
    gx, gy = f('knn_topk_backward')(pts.to(device), ctrl.to(device), idx, gd.to(device))
    rx, ry = np.zeros((N, 3), np.float32), np.zeros((M, 3), np.float32)
    O.call("knn_topk_backward_f32", N, M, 3, K, npy(pts), npy(ctrl), ri, npy(gd), rx, ry)
    assert rel_err(npy(gx), rx) < 1e-5 and rel_err(npy(gy), ry) < 2e-4
    out = f('lbs_blend')(pts.to(device), ctrl.to(device), c['sp_t'].to(device), c['sp_r'].to(device),
                         c['sp_s'].to(device), d2, idx, 0.01, 'LBS', c['sp_r'].to(device), 'dist')
    want = OL.lbs_blend(pts.double(), ctrl.double(), c['sp_t'].double(), c['sp_r'].double(), c['sp_s'].double(),
                        c['sp_r'].double(), d2.cpu().double(), idx.cpu(), 'dist', 0.01, 'LBS')
    for a, b, name in zip(out[:3], want[:3], ('d_xyz', 'd_rot', 'd_scale')):
        assert rel_err(npy(a), b.numpy()) < 2e-5, name
    print(f"[full config 1] knn 200000 x 512 bit-exact, lbs_blend within 2e-5", flush=True)

    P, widths = 300_000, (3, 3, 45, 1, 2, 4)
    mask = torch.rand(P, generator=g) < 0.9
    params = [torch.randn(P, w, generator=g) for w in widths]
    grads = [torch.randn(P, w, generator=g) for w in widths]
    dev = [[t.to(device) for t in group] for group in (params, grads)]
    m1, m2 = [torch.zeros_like(t) for t in dev[0]], [torch.zeros_like(t) for t in dev[0]]
    f('AdamMasksedUpdatedMulti')(dev[0], dev[1], m1, m2, mask.to(device), [1.6e-4] * 6, 0.9, 0.999, [1e-15] * 6, P)
    for k, w in enumerate(widths):
        rp, rm, rv = npy(params[k]).copy(), np.zeros((P, w), np.float32), np.zeros((P, w), np.float32)
        O.call("adam_masked_update_f32", P, w, npy(mask.to(torch.uint8)), 1.6e-4, 0.9, 0.999, 1e-15, rp, npy(grads[k]),
               rm, rv)
        assert np.array_equal(npy(dev[0][k]), rp) and np.array_equal(npy(m1[k]), rm) and np.array_equal(npy(m2[k]), rv)


def test_deform_mlp_mfma(device, oracle_mod):
    """Fused bf16 MFMA MLP against (a) the fp32 oracle on bf16-rounded weights and inputs -- isolates the kernel's own
    arithmetic up to the per-layer bf16 re-rounding of activations, tolerance 1e-2 relative -- and (b) the plain fp32 network, tolerance 2e-2 relative (bf16 rounding of
    weights and activations, the stated mixed-precision tolerance)."""
    import ctypes
    from fast_sp_gs_amd.deform import DeformNetwork
    O = oracle_mod
    torch.manual_seed(0)
    net = DeformNetwork().to(device)
    # heads are initialised at 1e-5 scale in the reference; give them weight so the comparison is meaningful
    for head in (net.gaussian_warp, net.gaussian_rotation, net.gaussian_scaling):
        torch.nn.init.normal_(head.weight, std=0.05)
        torch.nn.init.normal_(head.bias, std=0.1)
    for l in net.linear:
        torch.nn.init.normal_(l.bias, std=0.05)
    for B in (512, 77):
        x = torch.rand(B, 3, device=device) * 2 - 1
        t = torch.rand(1, device=device)
        net.pack()
        d_xyz, rot, scale, _ = net(x, t)
        got = torch.cat([d_xyz, rot, scale], -1).cpu()
        with torch.no_grad():
            ref32 = torch.cat(net.forward_fp32(x, t)[:3], -1)
            ref32 = torch.cat([ref32[:, 0:3], ref32[:, 3:7], ref32[:, 7:10]], -1).cpu()
        assert float((got - ref32).abs().max() / ref32.abs().max()) < 2e-2
        # oracle on bf16-rounded operands
        rb = lambda w: w.detach().to(torch.bfloat16).float().cpu().contiguous()
        inp = net.encode(x, t).to(torch.bfloat16).float().cpu().contiguous()
        Ws, bs = [rb(l.weight) for l in net.linear], [l.bias.detach().cpu().contiguous() for l in net.linear]
        heads = [net.gaussian_warp, net.gaussian_rotation, net.gaussian_scaling]
        hW, hb = [rb(h.weight) for h in heads], [h.bias.detach().cpu().contiguous() for h in heads]
        outs = [torch.zeros(B, h.weight.shape[0]) for h in heads]
        arr = lambda ts: (ctypes.c_void_p * len(ts))(*[v.data_ptr() for v in ts])
        dims = (ctypes.c_int * 3)(3, 4, 3)
        lib = O.lib()
        lib.oracle_deform_mlp_f32.restype = ctypes.c_int
        assert lib.oracle_deform_mlp_f32(B, inp.shape[1], 256, 8, 4, ctypes.c_void_p(inp.data_ptr()), arr(Ws), arr(bs),
                                         3, dims, arr(hW), arr(hb), arr(outs)) == 0
        ref = torch.cat(outs, -1)
        # remaining difference: activations are re-rounded to bf16 between layers on the GPU only
        assert float((got - ref).abs().max() / ref.abs().max()) < 1e-2


@pytest.mark.parametrize("P,kind", [(20000, "ball"), (5000, "clusters"), (777, "plane"), (3, "ball"), (2, "ball"),
                                    (1, "ball"), (4097, "same"), (5000, "halo"), (7000, "halo"), (20001, "halo")])
def test_simple_knn(P, kind, device, oracle_mod):
    """Mean squared 3-NN distance: bit-exact against the all-pairs oracle (the search is exact and both sides add the
    squares in the same order with contraction off) on clouds that stress the pruning: clusters far apart, a flat
    cloud (degenerate bounding box), duplicates, fewer points than neighbours, and a tight cluster inside a sparse halo
    (a wavefront whose queries have very different pruning bounds: the widest of all 64 has to be used)."""
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    g = torch.Generator().manual_seed(60 + P)
    if kind == "ball":
        pts = torch.randn(P, 3, generator=g)
    elif kind == "clusters":
        centres = torch.randn(7, 3, generator=g) * 50.0
        pts = centres[torch.randint(0, 7, (P,), generator=g)] + 0.01 * torch.randn(P, 3, generator=g)
    elif kind == "plane":
        pts = torch.cat([torch.rand(P, 2, generator=g), torch.full((P, 1), 0.25)], 1)
    elif kind == "halo":
        dense = 0.002 * torch.randn(P - P // 8, 3, generator=g)
        pts = torch.cat([dense, torch.rand(P // 8, 3, generator=g) * 4 - 2])[torch.randperm(P, generator=g)]
    else:
        pts = torch.ones(P, 3) * 0.5  # every point identical: all distances 0, the curve order is all ties
    pts = pts.contiguous()
    print(f"[simple_knn] P={P} {kind}", flush=True)
    got = get_C_function('simple_knn')(pts.to(device))
    torch.cuda.synchronize()
    ref = np.zeros(P, np.float32)
    with np.errstate(over='ignore'):
        O.call("simple_knn_f32", P, npy(pts), ref)
    assert np.array_equal(npy(got), ref)


def test_simple_knn_full_size(device):
    """3 M points: every result equals the 3-NN mean recomputed by brute force for a sample of queries."""
    from fast_sp_gs_amd._C import get_C_function
    g = torch.Generator().manual_seed(71)
    P = 3_000_000
    pts = (torch.rand(P, 3, generator=g) * 2 - 1).to(device)
    print(f"[simple_knn] P={P}", flush=True)
    got = get_C_function('simple_knn')(pts)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got).all()) and float(got.min()) >= 0
    sample = torch.randint(0, P, (256,), generator=g).to(device)
    d2 = ((pts[sample][:, None, :] - pts[None, :, :]) ** 2).sum(-1)  # [256, P]
    best = d2.topk(4, dim=1, largest=False).values[:, 1:]            # drop the point itself (distance 0)
    assert float((best.mean(1) - got[sample]).abs().max()) <= 1e-6 * float(best.max())


def test_simple_knn_mixed_density_large(device):
    """More points than one round of 64 x 64 boxes covers (so the group level runs a partial last round), most of them in
    a tight cluster, the rest a sparse halo: the halo points' results against brute force."""
    from fast_sp_gs_amd._C import get_C_function
    g = torch.Generator().manual_seed(72)
    P, n_halo = 300_001, 3_000
    pts = torch.cat([0.002 * torch.randn(P - n_halo, 3, generator=g), torch.rand(n_halo, 3, generator=g) * 4 - 2])
    perm = torch.randperm(P, generator=g)
    pts = pts[perm].contiguous().to(device)
    halo = torch.nonzero(perm >= P - n_halo).flatten()[:1024].to(device)
    sample = torch.cat([halo, torch.randint(0, P, (256,), generator=g).to(device)])
    print(f"[simple_knn] mixed density P={P}", flush=True)
    got = get_C_function('simple_knn')(pts)
    torch.cuda.synchronize()
    for part in sample.split(256):
        d2 = ((pts[part][:, None, :] - pts[None, :, :]) ** 2).sum(-1)
        best = d2.topk(4, dim=1, largest=False).values[:, 1:]
        want = best.mean(1)
        assert float(((want - got[part]).abs() / want.clamp_min(1e-30)).max()) <= 1e-5
