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
