"""TEST INFRASTRUCTURE ONLY: the reference's SH encoder on half tensors, degree <= 3, restated in numpy.

With scalar_t = at::Half (fast_2d_gs/_C/src/nerf/shencoder.cu, dispatch :667, :688) the kernels keep some intermediates in
half: the monomials `scalar_t xy = x * y, ...` (:31-33 forward, :190-193 backward; a product of two halves is formed in
float and rounded to half) and, in the backward, the running sums `scalar_t dx, dy, dz` (:188), where `dx += term`
rounds the float term to half and then the sum (:204-281). Everything else is float arithmetic on those values, rounded
once on store. numpy's float16 multiplies and adds the same way (float32 arithmetic, one rounding), so the restatement
below is plain numpy with explicit astype calls. Whether the reference's float expressions are contracted into fused
multiply-adds is the CUDA compiler's choice; results that differ by that choice differ by at most one half ulp.

Pinned by tests/test_oracle_sh.py: against the float64 basis and its gradient within the accumulated half roundings, and
exactly against a scalar Python evaluation with `struct`-level half conversions.
"""
import numpy as np

f16, f32 = np.float16, np.float32
C1 = f32(0.48860251190291987)
C1B = f32(0.48860251190291992)


def _monomials(x, y, z):
    """x, y, z: float16 arrays -> the six half-rounded products as float32."""
    h = lambda a, b: (a.astype(f32) * b.astype(f32)).astype(f16).astype(f32)
    return h(x, y), h(x, z), h(y, z), h(x, x), h(y, y), h(z, z)


def sh_encode_half(dirs16: np.ndarray, degree: int) -> np.ndarray:
    """dirs16 [B, D >= 3] float16 -> [B, (degree + 1)^2] float16 (shencoder.cu:18-73 with scalar_t = at::Half)."""
    assert dirs16.dtype == f16 and 0 <= degree <= 3
    x16, y16, z16 = dirs16[:, 0], dirs16[:, 1], dirs16[:, 2]
    x, y, z = (a.astype(f32) for a in (x16, y16, z16))
    Y = np.zeros((dirs16.shape[0], (degree + 1) ** 2), f32)
    Y[:, 0] = f32(0.28209479177387814)
    if degree >= 1:
        Y[:, 1], Y[:, 2], Y[:, 3] = -C1 * y, C1 * z, -C1 * x
    if degree >= 2:
        xy, xz, yz, xx, yy, zz = _monomials(x16, y16, z16)
        Y[:, 4] = f32(1.0925484305920792) * xy
        Y[:, 5] = f32(-1.0925484305920792) * yz
        Y[:, 6] = f32(0.94617469575755997) * zz - f32(0.31539156525251999)
        Y[:, 7] = f32(-1.0925484305920792) * xz
        Y[:, 8] = f32(0.54627421529603959) * xx - f32(0.54627421529603959) * yy
    if degree >= 3:
        Y[:, 9] = f32(0.59004358992664352) * y * (f32(-3.0) * xx + yy)
        Y[:, 10] = f32(2.8906114426405538) * xy * z
        Y[:, 11] = f32(0.45704579946446572) * y * (f32(1.0) - f32(5.0) * zz)
        Y[:, 12] = f32(0.3731763325901154) * z * (f32(5.0) * zz - f32(3.0))
        Y[:, 13] = f32(0.45704579946446572) * x * (f32(1.0) - f32(5.0) * zz)
        Y[:, 14] = f32(1.4453057213202769) * z * (xx - yy)
        Y[:, 15] = f32(0.59004358992664352) * x * (-xx + f32(3.0) * yy)
    return Y.astype(f16)


def sh_encode_backward_half(grad16: np.ndarray, dirs16: np.ndarray, degree: int) -> np.ndarray:
    """-> grad_inputs [B, 3] float16 (shencoder.cu:178-281 with scalar_t = at::Half): half running sums, every term
    rounded to half before it is added; terms with a literal zero factor are left out (they add +0)."""
    assert grad16.dtype == f16 and dirs16.dtype == f16 and 0 <= degree <= 3
    x16, y16, z16 = dirs16[:, 0], dirs16[:, 1], dirs16[:, 2]
    x, y, z = (a.astype(f32) for a in (x16, y16, z16))
    t = grad16.astype(f32)
    B = dirs16.shape[0]
    acc = {k: np.zeros(B, f16) for k in 'xyz'}

    def add(k, term):
        acc[k] = (acc[k].astype(f32) + term.astype(f32).astype(f16).astype(f32)).astype(f16)

    if degree >= 1:
        add('x', t[:, 3] * -C1B), add('y', t[:, 1] * -C1B), add('z', t[:, 2] * C1B)
    if degree >= 2:
        c = f32(1.0925484305920792)
        add('x', t[:, 4] * (c * y)), add('x', t[:, 7] * (-c * z)), add('x', t[:, 8] * (c * x))
        add('y', t[:, 4] * (c * x)), add('y', t[:, 5] * (-c * z)), add('y', t[:, 8] * (-c * y))
        add('z', t[:, 5] * (-c * y)), add('z', t[:, 6] * (f32(1.8923493915151204) * z)), add('z', t[:, 7] * (-c * x))
    if degree >= 3:
        xy, xz, yz, xx, yy, zz = _monomials(x16, y16, z16)
        a, b, c2 = f32(3.5402615395598609), f32(2.8906114426405538), f32(1.7701307697799304)
        d, e = f32(0.45704579946446572), f32(2.2852289973223288)
        add('x', t[:, 9] * (-a * xy)), add('x', t[:, 10] * (b * yz)), add('x', t[:, 13] * (d - e * zz))
        add('x', t[:, 14] * (b * xz)), add('x', t[:, 15] * (-c2 * xx + c2 * yy))
        add('y', t[:, 9] * (-c2 * xx + c2 * yy)), add('y', t[:, 10] * (b * xz)), add('y', t[:, 11] * (d - e * zz))
        add('y', t[:, 14] * (-b * yz)), add('y', t[:, 15] * (a * xy))
        add('z', t[:, 10] * (b * xy)), add('z', t[:, 11] * (f32(-4.5704579946446566) * yz))
        add('z', t[:, 12] * (f32(5.597644988851731) * zz - f32(1.1195289977703462)))
        add('z', t[:, 13] * (f32(-4.5704579946446566) * xz))
        add('z', t[:, 14] * (f32(1.4453057213202769) * xx - f32(1.4453057213202769) * yy))
    return np.stack([acc['x'], acc['y'], acc['z']], 1)
