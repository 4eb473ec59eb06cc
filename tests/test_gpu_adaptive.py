"""GPU parity of the density-control kernels against oracle/adaptive.py through the operators: selections, masks and
gathered rows bit for bit, the children of a split to 1e-6, and the host methods (`prune_points`, `densify_and_clone`,
`densify_and_split`, the one-table `densify`, `prune`) against the reference's operation sequence restated on arrays,
including optimiser parameter groups and Adam moments."""
import numpy as np
import pytest
import torch

from oracle import adaptive as A
from util import npy

pytestmark = pytest.mark.gpu


def _points(P, S, seed):
    rng = np.random.default_rng(seed)
    f = np.float32
    return {'xyz': rng.normal(size=(P, 3)).astype(f), 'f_dc': rng.normal(size=(P, 1, 3)).astype(f),
            'f_rest': rng.normal(size=(P, 15, 3)).astype(f), 'scaling': np.log(rng.uniform(0.005, 0.2, (P, S))).astype(f),
            'rotation': rng.normal(size=(P, 4)).astype(f), 'opacity': rng.normal(size=(P, 1)).astype(f)}


@pytest.mark.parametrize("P,frac", [(0, 0.5), (1, 1.0), (63, 0.5), (4096, 0.0), (4097, 1.0), (100003, 0.3),
                                    (3000000, 0.9)])
def test_select_indices(P, frac, device):
    from fast_sp_gs_amd._C import get_C_function
    rng = np.random.default_rng(P)
    mask = rng.random(P) < frac
    print(f"[select_indices] P={P} frac={frac}", flush=True)
    m = torch.from_numpy(mask).to(device)
    for invert in (False, True):
        got = get_C_function('select_indices')(m, invert)
        assert got.dtype == torch.int32 and np.array_equal(npy(got), A.select_indices(mask, invert))
    got = get_C_function('select_indices')(m.to(torch.uint8) * 7)  # any non-zero byte counts
    assert np.array_equal(npy(got), A.select_indices(mask))


def test_gather_rows(device):
    from fast_sp_gs_amd._C import get_C_function
    rng = np.random.default_rng(3)
    P, n = 50000, 61234
    shapes = [(3,), (1, 3), (15, 3), (2,), (4,), (1,), (), (16,), (5,)]
    tensors = [rng.normal(size=(P,) + s).astype(np.float32) for s in shapes]
    tensors += [rng.integers(0, 2, (P,)).astype(bool), rng.integers(-9, 9, (P, 3)).astype(np.int32),
                rng.integers(0, 255, (P, 3)).astype(np.uint8), rng.integers(-9, 9, (P,)).astype(np.int64)]
    tensors = tensors * 3  # 39 tensors: more than one launch
    rows = rng.integers(-1, P, n).astype(np.int32)
    print(f"[gather_rows] {len(tensors)} tensors, {P} -> {n} rows", flush=True)
    dev = [torch.from_numpy(t).to(device) for t in tensors]
    dev[2] = dev[2][:, :, :]  # contiguous view
    out = get_C_function('gather_rows')(dev, torch.from_numpy(rows).to(device))
    for t, o in zip(tensors, out):
        assert o.dtype == torch.from_numpy(t).dtype and np.array_equal(npy(o), A.gather_rows(t, rows))
    # a sliced (misaligned) source: rows of 12 bytes starting 4 bytes into an allocation
    base = torch.from_numpy(rng.normal(size=(P * 3 + 1,)).astype(np.float32)).to(device)
    view = base[1:].view(P, 3)
    o = get_C_function('gather_rows')([view], torch.from_numpy(rows).to(device))[0]
    assert np.array_equal(npy(o), A.gather_rows(npy(view), rows))
    assert get_C_function('gather_rows')([dev[0]], torch.empty(0, dtype=torch.int32, device=device))[0].shape == (0, 3)


@pytest.mark.parametrize("S", [2, 3])
def test_masks_children_statistics(S, device):
    from fast_sp_gs_amd._C import get_C_function as f
    rng = np.random.default_rng(7 + S)
    P, N = 200001, 2
    print(f"[masks / children / statistics] P={P} S={S}", flush=True)
    acc = rng.uniform(0, 1e-2, (P, 1)).astype(np.float32)
    den = rng.integers(0, 5, (P, 1)).astype(np.float32)
    acc[den == 0] = 0
    scaling = rng.uniform(0.001, 0.1, (P, S)).astype(np.float32)
    d = lambda a: torch.from_numpy(a).to(device)
    clone, split = f('densify_masks')(d(acc), d(den), d(scaling), 2e-3, 0.04)
    want_c, want_s = A.densify_masks(acc, den, scaling, 2e-3, 0.04)
    assert clone.dtype == torch.bool and np.array_equal(npy(clone), want_c) and np.array_equal(npy(split), want_s)
    assert want_c.any() and want_s.any()
    none_c, none_s = f('densify_masks')(d(acc), d(den), d(scaling), float('inf'), 0.04)
    assert not none_c.any() and not none_s.any()

    opacity = rng.uniform(0, 0.05, (P, 1)).astype(np.float32)
    radii = rng.uniform(0, 40, P).astype(np.float32)
    for size in (20.0, None, 0):
        got = f('prune_mask')(d(opacity), d(radii), d(scaling), 0.005, size, 0.09)
        assert np.array_equal(npy(got), A.prune_mask(opacity, radii, scaling, 0.005, size, 0.09))

    xyz = rng.normal(size=(P, 3)).astype(np.float32)
    rot = rng.normal(size=(P, 4)).astype(np.float32)
    sel = A.select_indices(want_s)
    noise = rng.normal(size=(N * len(sel), 3)).astype(np.float32)
    cx, cs = f('split_children')(d(sel), N, d(xyz), d(scaling), d(rot), d(noise))
    wx, ws = A.split_children(sel, N, xyz.astype(np.float64), scaling.astype(np.float64), rot.astype(np.float64), noise)
    np.testing.assert_allclose(npy(cx), wx, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(npy(cs), ws, rtol=1e-6, atol=1e-6)

    r = rng.integers(-1, 30, P).astype(np.int32)
    r[rng.random(P) < 0.4] = 0
    grad = rng.normal(size=(P, 3)).astype(np.float32)
    fac = rng.uniform(0.5, 2, (P, 1)).astype(np.float32)
    for factor in (None, fac):
        mr, a, dn = d(radii), d(acc), d(den)
        vis = f('densification_stats')(d(r), d(grad), mr, a, dn, None if factor is None else d(factor))
        wmr, wa, wd, wv = A.densification_stats(r, grad, radii, acc, den, factor)
        assert np.array_equal(npy(vis), wv) and np.array_equal(npy(mr), wmr) and np.array_equal(npy(dn), wd)
        assert np.array_equal(npy(a), wa)  # contraction is off in the kernel, as in the restatement


def _model(pts, device, lr=1e-2, steps=2):
    """A point holder with torch Adam whose moments are populated by a few steps."""
    from fast_sp_gs_amd.adaptive_control import GaussianPoints
    t = {k: torch.from_numpy(v).to(device) for k, v in pts.items()}
    model = GaussianPoints(t['xyz'], t['f_dc'], t['f_rest'], t['scaling'], t['rotation'], t['opacity'])
    opt = torch.optim.Adam(model.param_groups(lr), eps=1e-15)
    g = torch.Generator(device='cpu').manual_seed(0)
    for _ in range(steps):
        for group in opt.param_groups:
            p = group['params'][0]
            p.grad = torch.randn(p.shape, generator=g).to(device) * 1e-3
        opt.step()
    names = model.param_names_map
    params = {n: npy(getattr(model, a)) for a, n in names.items()}
    moments = {n: (npy(opt.state[getattr(model, a)]['exp_avg']), npy(opt.state[getattr(model, a)]['exp_avg_sq']))
               for a, n in names.items()}
    return model, opt, A.PointSet(params, moments)


def _same(model, opt, ps, exact=True):
    assert model._xyz.shape[0] == ps.P
    for a, n in model.param_names_map.items():
        p = getattr(model, a)
        group = [g for g in opt.param_groups if g['name'] == n][0]
        assert group['params'][0] is p and p.requires_grad and isinstance(p, torch.nn.Parameter)
        if exact or n not in ('xyz', 'scaling'):
            assert np.array_equal(npy(p), ps.params[n]), n
        else:
            np.testing.assert_allclose(npy(p), ps.params[n], rtol=2e-6, atol=2e-6)
        st = opt.state[p]
        assert np.array_equal(npy(st['exp_avg']), ps.moments[n][0]) and np.array_equal(npy(st['exp_avg_sq']), ps.moments[n][1])
        assert 'step' in st
    assert len(opt.state) == 6
    assert np.array_equal(npy(model.xyz_gradient_accum), ps.grad_accum) and np.array_equal(npy(model.denom), ps.denom)
    assert np.array_equal(npy(model.max_radii2D), ps.max_radii2D)


def _statistics(model, ps, seed):
    rng = np.random.default_rng(seed)
    P = ps.P
    ps.grad_accum = rng.uniform(0, 4e-3, (P, 1)).astype(np.float32)
    ps.denom = rng.integers(0, 3, (P, 1)).astype(np.float32)
    ps.grad_accum[ps.denom == 0] = 0
    ps.max_radii2D = rng.uniform(0, 30, P).astype(np.float32)
    dev = model._xyz.device
    model.xyz_gradient_accum = torch.from_numpy(ps.grad_accum).to(dev)
    model.denom = torch.from_numpy(ps.denom).to(dev)
    model.max_radii2D = torch.from_numpy(ps.max_radii2D).to(dev)


@pytest.mark.parametrize("S", [2, 3])
def test_density_control_methods(S, device):
    P, N = 30011, 2
    thr, extent, pd = 1e-3, 5.0, 0.01
    print(f"[density control] P={P} S={S}", flush=True)
    pts = _points(P, S, 11)
    rng = np.random.default_rng(12)

    # prune_points
    model, opt, ps = _model(pts, device)
    _statistics(model, ps, 1)
    mask = rng.random(P) < 0.2
    model.prune_points(opt, torch.from_numpy(mask).to(device))
    ps.prune_points(mask)
    _same(model, opt, ps)
    opt.zero_grad()
    model._xyz.sum().backward()
    opt.step()  # the optimiser still steps on the new parameters

    # the reference's two-step densify, then prune
    model, opt, ps = _model(pts, device)
    _statistics(model, ps, 2)
    grads = np.nan_to_num(ps.grad_accum / ps.denom, nan=0.0).astype(np.float32)
    g = torch.from_numpy(grads).to(device)
    model.densify_and_clone(opt, g, thr, pd * extent)
    ps.densify_and_clone(grads, thr, pd * extent)
    _same(model, opt, ps)
    n_split = int(((np.pad(grads.reshape(-1), (0, ps.P - P)) >= np.float32(thr))
                   & (ps.scaling().max(1) > np.float32(pd * extent))).sum())
    noise = rng.normal(size=(N * n_split, 3)).astype(np.float32)
    model.densify_and_split(opt, g, thr, pd * extent, N, torch.from_numpy(noise).to(device))
    ps.densify_and_split(grads, thr, pd * extent, noise, N)
    _same(model, opt, ps, exact=False)
    two_step = {a: npy(getattr(model, a)) for a in model.param_names_map}

    # densify as one table gives the same point set
    model, opt, ps = _model(pts, device)
    _statistics(model, ps, 2)
    model.densify(opt, thr, extent, pd, N, torch.from_numpy(noise).to(device))
    ps.densify(thr, extent, noise, pd, N)
    _same(model, opt, ps, exact=False)
    for a, v in two_step.items():
        assert np.array_equal(npy(getattr(model, a)), v), a
    assert model._xyz.shape[0] > P

    # prune with and without the size tests; thresholds sit away from every value by construction of the check below
    for size in (20.0, None):
        _statistics(model, ps, 3)
        op, sc = ps.opacity().reshape(-1), ps.scaling().max(1)
        assert np.abs(op - 0.3).min() > 1e-6 and np.abs(sc - 0.1 * 1.5).min() > 1e-7
        model.prune(opt, 0.3, 1.5, size, 0.1)
        ps.prune(0.3, 1.5, size, 0.1)
        _same(model, opt, ps, exact=False)

    # per-step statistics through the host method
    radii = torch.randint(0, 20, (ps.P,), dtype=torch.int32, device=device)
    grad = torch.randn(ps.P, 3, device=device)
    vis = model.update_statistics(radii, grad)
    mr, acc, den, wv = A.densification_stats(npy(radii), npy(grad), ps.max_radii2D, ps.grad_accum, ps.denom)
    assert np.array_equal(npy(vis), wv) and np.array_equal(npy(model.max_radii2D), mr)
    assert np.array_equal(npy(model.xyz_gradient_accum), acc) and np.array_equal(npy(model.denom), den)

    # reset_opacity keeps the groups consistent
    model.reset_opacity(opt)
    assert float(torch.sigmoid(model._opacity).max()) <= 0.01 + 1e-6
    assert not opt.state[model._opacity]['exp_avg'].any()


def test_superpoint_extras_follow_the_points(device):
    """The superpoint model's per-point extras -- per-frame culling flags, the visibility factor, the superpoint
    assignment -- through clone, split and prune, against the reference's own expressions for them
    (network.py:1195-1215: `t[valid]`, `cat((t, t[mask]))`, `cat((t, t[mask].repeat(N, 1)))`, and the prune of the split
    parents, :1190-1191), evaluated with torch indexing on the same masks; and the visibility factor inside the gradient
    statistics (:1153)."""
    P, N, F = 20011, 2, 7
    thr, extent, pd = 1e-3, 5.0, 0.01
    pts = _points(P, 2, 21)
    model, opt, ps = _model(pts, device)
    _statistics(model, ps, 5)
    g = torch.Generator().manual_seed(9)
    model._culling = (torch.rand(P, F, generator=g) < 0.3).to(device)
    model.factor_culling = torch.rand(P, 1, generator=g).to(device)
    model.p2sp = torch.randint(0, 512, (P,), generator=g, dtype=torch.int32).to(device)
    ref = {k: getattr(model, k).clone() for k in ('_culling', 'factor_culling', 'p2sp')}

    def carry(mask, n=None):  # densification_postfix of the superpoint model
        for k, t in ref.items():
            extra = t[mask] if n is None else t[mask].repeat(n, *[1] * (t.ndim - 1))
            ref[k] = torch.cat((t, extra))

    def drop(mask):  # prune_points of the superpoint model
        for k, t in ref.items():
            ref[k] = t[~mask]

    def check():
        for k, t in ref.items():
            got = getattr(model, k)
            assert got.dtype == t.dtype and got.shape == t.shape and torch.equal(got, t), k
        assert model._culling.shape[0] == model._xyz.shape[0]

    grads = torch.from_numpy(np.nan_to_num(ps.grad_accum / ps.denom, nan=0.0).astype(np.float32)).to(device)
    scaling = model.get_scaling.detach()
    clone_mask = (torch.norm(grads, dim=-1) >= thr) & (scaling.amax(1) <= pd * extent)
    model.densify_and_clone(opt, grads, thr, pd * extent)
    carry(clone_mask)
    check()
    P1 = model._xyz.shape[0]
    padded = torch.zeros(P1, device=device)
    padded[:P] = grads.squeeze(-1)
    split_mask = (padded >= thr) & (model.get_scaling.detach().amax(1) > pd * extent)
    assert int(clone_mask.sum()) > 0 and int(split_mask.sum()) > 0
    model.densify_and_split(opt, grads, thr, pd * extent, N)
    carry(split_mask, N)
    drop(torch.cat((split_mask, split_mask.new_zeros(N * int(split_mask.sum())))))
    check()
    prune = torch.rand(model._xyz.shape[0], generator=g).to(device) < 0.25
    model.prune_points(opt, prune)
    drop(prune)
    check()
    # gradient statistics weighted by the visibility factor
    Pn = model._xyz.shape[0]
    vs = torch.zeros(Pn, 3, device=device, requires_grad=True)
    vs.grad = torch.randn(Pn, 3, generator=g).to(device)
    upd = torch.rand(Pn, generator=g).to(device) < 0.6
    acc0, den0 = model.xyz_gradient_accum.clone(), model.denom.clone()
    model.add_densification_stats(vs, upd)
    want = acc0.clone()
    want[upd] += torch.norm(vs.grad[upd, :2], dim=-1, keepdim=True) * model.factor_culling[upd]
    assert float((model.xyz_gradient_accum - want).abs().max()) <= 1e-6 * float(want.abs().max())
    assert torch.equal(model.denom, den0 + upd[:, None].float())
