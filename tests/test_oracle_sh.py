"""Pins the oracle's spherical-harmonic code (oracle/sh_basis.h and its users) without the reference:
orthonormality of the basis under sphere quadrature, the degree-0 closed form, the l=1 sign convention (-y, +z, -x),
central finite differences for every derivative, and the clamp mask of SH -> RGB."""
import numpy as np
import pytest


def _sphere_quadrature(n_theta=64, n_phi=128):
    # Gauss-Legendre in cos(theta) x uniform in phi integrates polynomials up to high degree exactly
    ct, wt = np.polynomial.legendre.leggauss(n_theta)
    phi = (np.arange(n_phi) + 0.5) * (2 * np.pi / n_phi)
    CT, PH = np.meshgrid(ct, phi, indexing="ij")
    ST = np.sqrt(1 - CT ** 2)
    dirs = np.stack([ST * np.cos(PH), ST * np.sin(PH), CT], -1).reshape(-1, 3)
    w = (wt[:, None] * np.full((1, n_phi), 2 * np.pi / n_phi)).reshape(-1)
    return np.ascontiguousarray(dirs), w


def _encode(O, dirs, degree):
    out = np.zeros((dirs.shape[0], (degree + 1) ** 2), dirs.dtype)
    suffix = "f64" if dirs.dtype == np.float64 else "f32"
    assert O.call(f"sh_encode_forward_{suffix}", dirs.shape[0], 3, degree, dirs, out) == 0
    return out


def test_basis_is_orthonormal(oracle_mod):
    dirs, w = _sphere_quadrature()
    Y = _encode(oracle_mod, dirs, 7)  # degrees 4..7 come from the generated table
    gram = (Y * w[:, None]).T @ Y
    assert np.abs(gram - np.eye(64)).max() < 1e-12
    for degree in range(7):  # lower degrees are prefixes of the same table
        assert np.array_equal(_encode(oracle_mod, dirs, degree), Y[:, :(degree + 1) ** 2])


def test_degree0_and_l1_signs(oracle_mod):
    d = np.array([[0.3, -0.5, 0.81]], np.float64)
    Y = _encode(oracle_mod, d, 1)[0]
    c1 = np.sqrt(3 / (4 * np.pi))
    assert abs(Y[0] - 0.5 / np.sqrt(np.pi)) < 1e-15
    assert np.allclose(Y[1:4], [-c1 * d[0, 1], c1 * d[0, 2], -c1 * d[0, 0]], atol=1e-15)


def test_float_matches_double(oracle_mod):
    rng = np.random.default_rng(0)
    d = rng.normal(size=(1000, 3))
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    assert np.abs(_encode(oracle_mod, d.astype(np.float32), 3) - _encode(oracle_mod, d, 3)).max() < 2e-6
    assert np.abs(_encode(oracle_mod, d.astype(np.float32), 7) - _encode(oracle_mod, d, 7)).max() < 2e-5


@pytest.mark.parametrize("degree", [0, 1, 2, 3, 4, 5, 6, 7])
def test_encoder_backward_is_the_gradient(oracle_mod, degree):
    rng = np.random.default_rng(degree)
    B, n = 50, (degree + 1) ** 2
    x = np.ascontiguousarray(rng.normal(size=(B, 3)))
    g = np.ascontiguousarray(rng.normal(size=(B, n)))
    gin = np.zeros((B, 3))
    assert oracle_mod.call("sh_encode_backward_f64", B, 3, degree, g, x, gin) == 0
    eps = 1e-6
    fd = np.zeros((B, 3))
    for a in range(3):
        xp, xm = x.copy(), x.copy()
        xp[:, a] += eps
        xm[:, a] -= eps
        fd[:, a] = ((_encode(oracle_mod, xp, degree) - _encode(oracle_mod, xm, degree)) * g).sum(1) / (2 * eps)
    assert np.abs(gin - fd).max() < 1e-8 * max(1.0, np.abs(fd).max())


@pytest.mark.parametrize("degree", [3, 6])
@pytest.mark.parametrize("use_campos", [False, True])
def test_sh_to_rgb_forward_backward(oracle_mod, use_campos, degree):
    O = oracle_mod
    rng = np.random.default_rng(7)
    P, F = 40, (degree + 1) ** 2 + 1
    pos = np.ascontiguousarray(rng.normal(size=(P, 3)))
    if not use_campos:
        pos /= np.linalg.norm(pos, axis=1, keepdims=True)
    cam = np.array([0.1, -0.2, 3.0]) if use_campos else None
    sh = np.ascontiguousarray(rng.normal(size=(P, F, 3)) * 0.4)
    grad = np.ascontiguousarray(rng.normal(size=(P, 3)))

    def fwd(pos_, cam_, sh_, clamp=1):
        rgb = np.zeros((P, 3))
        assert O.call("sh_to_rgb_forward_f64", P, F, degree, clamp, pos_, cam_, sh_, rgb) == 0
        return rgb

    rgb = fwd(pos, cam, sh)
    # forward = max(0, 0.5 + sum_l Y_l c_l) with the (optionally normalised) direction
    d = pos - cam if use_campos else pos
    if use_campos:
        d = d / np.sqrt((d * d).sum(1, keepdims=True) + 1e-12)
    Y = _encode(O, np.ascontiguousarray(d), degree)
    assert np.abs(rgb - np.maximum(0, 0.5 + np.einsum("pl,plc->pc", Y, sh[:, :Y.shape[1]]))).max() < 1e-12
    assert (rgb == 0).any() and (rgb > 0).any()  # the clamp is exercised

    g_dir, g_sh = np.zeros((P, 3)), np.zeros((P, F, 3))
    g_cam = np.zeros(3) if use_campos else None
    assert O.call("sh_to_rgb_backward_f64", P, F, degree, 1, pos, cam, sh, rgb, grad, g_dir, g_cam, g_sh) == 0
    eps = 1e-6
    loss = lambda pos_, cam_, sh_: (fwd(pos_, cam_, sh_) * grad).sum()
    # coefficients
    for (p, l, c) in [(0, 0, 0), (3, 5, 1), (7, (degree + 1) ** 2 - 1, 2), (11, 9, 0)]:
        shp, shm = sh.copy(), sh.copy()
        shp[p, l, c] += eps
        shm[p, l, c] -= eps
        assert abs((loss(pos, cam, shp) - loss(pos, cam, shm)) / (2 * eps) - g_sh[p, l, c]) < 1e-7
    # position / direction, and the camera position (sum over points, opposite sign)
    cam_fd = np.zeros(3)
    for a in range(3):
        for p in range(0, P, 7):
            pp, pm = pos.copy(), pos.copy()
            pp[p, a] += eps
            pm[p, a] -= eps
            assert abs((loss(pp, cam, sh) - loss(pm, cam, sh)) / (2 * eps) - g_dir[p, a]) < 1e-6
        if use_campos:
            cp, cm = cam.copy(), cam.copy()
            cp[a] += eps
            cm[a] -= eps
            cam_fd[a] = (loss(pos, cp, sh) - loss(pos, cm, sh)) / (2 * eps)
    if use_campos:
        assert np.abs(cam_fd - g_cam).max() < 1e-6
        assert np.abs(g_cam + g_dir.sum(0)).max() < 1e-9


def test_half_encoder_restatement(oracle_mod):
    """oracle/sh_half.py (the reference's at::Half instantiation of the SH encoder, degree <= 3): stays within the
    accumulated half roundings of the float64 basis / gradient on the same half inputs, really rounds its monomials
    (a value the unrounded evaluation would give differently), and agrees with a scalar evaluation whose half
    conversions go through `struct` ('e' format) instead of numpy's float16."""
    import struct
    from oracle import sh_half as H
    O = oracle_mod
    rng = np.random.default_rng(5)
    d = rng.normal(size=(3000, 3))
    d16 = (d / np.linalg.norm(d, axis=1, keepdims=True)).astype(np.float16)
    g16 = rng.normal(size=(3000, 16)).astype(np.float16)
    for degree in (0, 1, 2, 3):
        n = (degree + 1) ** 2
        ref, gref = np.zeros((3000, n)), np.zeros((3000, 3))
        O.call("sh_encode_forward_f64", 3000, 3, degree, np.ascontiguousarray(d16, np.float64), ref)
        O.call("sh_encode_backward_f64", 3000, 3, degree, np.ascontiguousarray(g16[:, :n], np.float64),
               np.ascontiguousarray(d16, np.float64), gref)
        enc = H.sh_encode_half(d16, degree)
        back = H.sh_encode_backward_half(np.ascontiguousarray(g16[:, :n]), d16, degree)
        assert enc.dtype == np.float16 and back.dtype == np.float16
        # forward: one rounding of a monomial + one on store; backward: up to 9 rounded terms and 9 rounded sums
        assert np.abs(enc.astype(np.float64) - ref).max() <= 3 * 2.0 ** -11 * max(np.abs(ref).max(), 1.0)
        if degree:
            assert np.abs(back.astype(np.float64) - gref).max() <= 12 * 2.0 ** -11 * np.abs(gref).max()
    # the monomials are rounded: recomputing entry 4 from the unrounded product differs somewhere
    x, y = d16[:, 0].astype(np.float32), d16[:, 1].astype(np.float32)
    unrounded = (np.float32(1.0925484305920792) * (x * y)).astype(np.float16)
    assert (H.sh_encode_half(d16, 2)[:, 4] != unrounded).any()
    # scalar evaluation with struct's half conversion
    h = lambda v: struct.unpack('e', struct.pack('e', float(v)))[0]
    f = lambda v: float(np.float32(v))
    for i in range(0, 3000, 97):
        xs, ys, zs = (float(v) for v in d16[i])
        xy, zz = h(f(xs * ys)), h(f(zs * zs))
        assert float(enc[i, 4]) == h(f(np.float32(1.0925484305920792) * np.float32(xy)))
        want = h(f(np.float32(0.3731763325901154) * np.float32(zs)) * f(np.float32(5.0) * np.float32(zz) - np.float32(3.0)))
        assert abs(float(enc[i, 12]) - want) <= abs(want) * 2.0 ** -10
