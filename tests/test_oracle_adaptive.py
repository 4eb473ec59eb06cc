"""Pins oracle/adaptive.py (density control restated in numpy) by checks that do not reuse its expressions: explicit
Python loops for the selections, scipy rotations and closed forms for the children of a split, and an independent
list-of-records model for the densify / prune sequence of fast_2d_gs/gaussian_splatting.py:557-636."""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

from oracle import adaptive as A


def _points(P, S, seed):
    rng = np.random.default_rng(seed)
    f = np.float32
    return {'xyz': rng.normal(size=(P, 3)).astype(f), 'f_dc': rng.normal(size=(P, 1, 3)).astype(f),
            'f_rest': rng.normal(size=(P, 15, 3)).astype(f), 'scaling': np.log(rng.uniform(0.005, 0.2, (P, S))).astype(f),
            'rotation': rng.normal(size=(P, 4)).astype(f), 'opacity': rng.normal(size=(P, 1)).astype(f)}


def test_select_and_gather_against_loops():
    rng = np.random.default_rng(0)
    for P in (0, 1, 7, 1000):
        mask = rng.random(P) < 0.3
        want = [i for i in range(P) if mask[i]]
        assert A.select_indices(mask).tolist() == want
        assert A.select_indices(mask, True).tolist() == [i for i in range(P) if not mask[i]]
    t = rng.normal(size=(50, 2, 3)).astype(np.float32)
    rows = np.array([3, -1, 49, 3, 0, -1], np.int32)
    out = A.gather_rows(t, rows)
    for r, s in enumerate(rows):
        assert np.array_equal(out[r], t[s] if s >= 0 else np.zeros((2, 3), np.float32))


def test_masks_against_loops():
    rng = np.random.default_rng(1)
    P = 500
    acc = rng.uniform(0, 1e-2, (P, 1)).astype(np.float32)
    den = rng.integers(0, 5, (P, 1)).astype(np.float32)
    acc[den == 0] = 0  # a point never seen has no accumulated gradient: 0 / 0 -> NaN -> 0
    scaling = rng.uniform(0.001, 0.1, (P, 3)).astype(np.float32)
    clone, split = A.densify_masks(acc, den, scaling, 2e-3, 0.04)
    for i in range(P):
        g = 0.0 if den[i, 0] == 0 else float(np.float32(acc[i, 0]) / np.float32(den[i, 0]))
        big = max(scaling[i])
        assert clone[i] == (g >= np.float32(2e-3) and big <= np.float32(0.04))
        assert split[i] == (g >= np.float32(2e-3) and big > np.float32(0.04))
    assert not (clone & split).any() and clone.any() and split.any()
    opacity = rng.uniform(0, 0.05, (P, 1)).astype(np.float32)
    radii = rng.uniform(0, 40, P).astype(np.float32)
    m = A.prune_mask(opacity, radii, scaling, 0.005, 20, 0.09)
    m0 = A.prune_mask(opacity, radii, scaling, 0.005, None, 0.09)
    for i in range(P):
        low = opacity[i, 0] < np.float32(0.005)
        assert m0[i] == low
        assert m[i] == (low or radii[i] > 20 or max(scaling[i]) > np.float32(0.09))


@pytest.mark.parametrize('S', [2, 3])
def test_split_children_closed_forms(S):
    rng = np.random.default_rng(2)
    P, N = 40, 2
    pts = _points(P, S, 3)
    pts = {k: v.astype(np.float64) for k, v in pts.items()}
    scaling = np.exp(pts['scaling'])
    sel = np.array([1, 5, 6, 30], np.int32)
    noise = rng.normal(size=(N * len(sel), 3))
    xyz, sc = A.split_children(sel, N, pts['xyz'], scaling, pts['rotation'], noise)
    assert xyz.shape == (N * len(sel), 3) and sc.shape == (N * len(sel), S)
    for j in range(N * len(sel)):
        p = sel[j % len(sel)]
        s3 = np.concatenate([scaling[p], np.zeros(3 - S)])
        R = Rotation.from_quat(pts['rotation'][p]).as_matrix()  # scipy: xyzw, normalises
        np.testing.assert_allclose(xyz[j], R @ (noise[j] * s3) + pts['xyz'][p], rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(np.exp(sc[j]), scaling[p] / (0.8 * N), rtol=1e-12)
    # no noise: children sit on their parents; identity rotation: the offset is the scaled noise itself
    xyz0, _ = A.split_children(sel, N, pts['xyz'], scaling, pts['rotation'], np.zeros_like(noise))
    np.testing.assert_array_equal(xyz0, np.tile(pts['xyz'][sel], (N, 1)))
    ident = np.tile(np.array([0, 0, 0, 2.0]), (P, 1))  # unnormalised on purpose
    xyz1, _ = A.split_children(sel, N, pts['xyz'], scaling, ident, noise)
    s3 = np.concatenate([scaling, np.zeros((P, 3 - S))], 1)
    np.testing.assert_allclose(xyz1 - np.tile(pts['xyz'][sel], (N, 1)), noise * np.tile(s3[sel], (N, 1)), atol=1e-15)


def test_statistics_against_loop():
    rng = np.random.default_rng(4)
    P = 300
    radii = rng.integers(-1, 30, P).astype(np.int32)
    radii[rng.random(P) < 0.4] = 0
    grad = rng.normal(size=(P, 3)).astype(np.float32)
    mr = rng.uniform(0, 20, P).astype(np.float32)
    acc, den = rng.uniform(0, 1, (P, 1)).astype(np.float32), rng.integers(0, 9, (P, 1)).astype(np.float32)
    fac = rng.uniform(0.5, 2, (P, 1)).astype(np.float32)
    for factor in (None, fac):
        mr2, acc2, den2, vis = A.densification_stats(radii, grad, mr, acc, den, factor)
        for i in range(P):
            if radii[i] > 0:
                n = np.hypot(np.float64(grad[i, 0]), np.float64(grad[i, 1])) * (1 if factor is None else factor[i, 0])
                assert vis[i] and mr2[i] == max(mr[i], radii[i]) and den2[i, 0] == den[i, 0] + 1
                assert abs(acc2[i, 0] - (acc[i, 0] + n)) < 1e-6
            else:
                assert not vis[i] and mr2[i] == mr[i] and acc2[i, 0] == acc[i, 0] and den2[i, 0] == den[i, 0]


def test_densify_prune_sequence_against_record_model():
    """The reference's clone -> split -> prune sequence on a list of per-point records (one dict per point), written
    without masks or concatenation: what each point becomes is decided point by point."""
    P, N, S = 400, 2, 2
    pts = _points(P, S, 5)
    rng = np.random.default_rng(6)
    moments = {k: (rng.normal(size=v.shape).astype(np.float32), rng.uniform(size=v.shape).astype(np.float32))
               for k, v in pts.items()}
    ps = A.PointSet(pts, moments)
    ps.grad_accum = rng.uniform(0, 4e-3, (P, 1)).astype(np.float32)
    ps.denom = rng.integers(0, 3, (P, 1)).astype(np.float32)
    ps.grad_accum[ps.denom == 0] = 0
    grads = np.where(ps.denom > 0, ps.grad_accum / np.maximum(ps.denom, 1), 0).reshape(-1)
    thr, extent, pd = 1e-3, 5.0, 0.01
    big = np.exp(pts['scaling']).max(1)
    clone = [i for i in range(P) if grads[i] >= np.float32(thr) and big[i] <= np.float32(pd * extent)]
    split = [i for i in range(P) if grads[i] >= np.float32(thr) and big[i] > np.float32(pd * extent)]
    assert clone and split
    noise = rng.normal(size=(N * len(split), 3)).astype(np.float32)
    ps.densify(thr, extent, noise, pd, N)

    records = []  # (source point, kind, child number)
    records += [(i, 'kept', 0) for i in range(P) if i not in set(split)]
    records += [(i, 'clone', 0) for i in clone]
    records += [(i, 'child', r * len(split) + k) for r in range(N) for k, i in enumerate(split)]
    assert ps.P == len(records) == P - len(split) + len(clone) + N * len(split)
    for row, (i, kind, j) in enumerate(records):
        for k in pts:
            if kind == 'child' and k in ('xyz', 'scaling'):
                continue
            assert np.array_equal(ps.params[k][row], pts[k][i]), (row, k)
            m, v = ps.moments[k][0][row], ps.moments[k][1][row]
            if kind == 'kept':
                assert np.array_equal(m, moments[k][0][i]) and np.array_equal(v, moments[k][1][i])
            else:
                assert not m.any() and not v.any()
        if kind == 'child':
            s3 = np.concatenate([np.exp(pts['scaling'][i]), [0.0]])
            R = Rotation.from_quat(pts['rotation'][i].astype(np.float64)).as_matrix()
            np.testing.assert_allclose(ps.params['xyz'][row], R @ (noise[j] * s3) + pts['xyz'][i], atol=2e-6)
            np.testing.assert_allclose(ps.params['scaling'][row], pts['scaling'][i] - np.log(0.8 * N), atol=2e-6)
    assert not ps.grad_accum.any() and not ps.denom.any() and not ps.max_radii2D.any()
    assert ps.grad_accum.shape == (ps.P, 1) and ps.max_radii2D.shape == (ps.P,)

    # prune: statistics follow the kept rows
    ps.max_radii2D = rng.uniform(0, 30, ps.P).astype(np.float32)
    before = {k: v.copy() for k, v in ps.params.items()}
    radii = ps.max_radii2D.copy()
    op = 1 / (1 + np.exp(-before['opacity'].astype(np.float64).reshape(-1)))
    drop = [i for i in range(ps.P) if op[i] < 0.3 or radii[i] > 20 or np.exp(before['scaling'][i]).max() > 0.1 * 1.5]
    ps.prune(0.3, 1.5, 20, 0.1)
    keep = [i for i in range(len(radii)) if i not in set(drop)]
    assert 0 < len(keep) < len(radii) and ps.P == len(keep)
    for k in before:
        assert np.array_equal(ps.params[k], before[k][keep])
    assert np.array_equal(ps.max_radii2D, radii[keep])
