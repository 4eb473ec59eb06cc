"""CPU restatement (numpy) of the reference's adaptive density control. TEST INFRASTRUCTURE ONLY: nothing in the product
imports this module.

Follows fast_2d_gs/gaussian_splatting.py:497-637 and fast_2d_gs/network.py:1152-1215, 1276-1282 one operation at a time,
the way the reference performs them (boolean indexing, concatenation, repetition), so that the table-driven device
version can be checked against the sequence of host operations it replaces.

Pinned by tests/test_oracle_adaptive.py: selections against explicit Python loops, the children of a split against
scipy's rotations and closed forms (a child drawn with zero noise sits on its parent, an identity rotation leaves the
scaled noise as the offset, log-scales drop by log(0.8 N)), the whole densify / prune sequence against an independent
list-of-records model.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import numpy as np


def select_indices(mask: np.ndarray, invert: bool = False) -> np.ndarray:
    """`torch.nonzero(mask)` / `torch.nonzero(~mask)`: what `tensor[mask]` reads, in order
    (gaussian_splatting.py:526-527, :558)."""
    m = np.asarray(mask).astype(bool)
    return np.flatnonzero(~m if invert else m).astype(np.int32)


def gather_rows(tensor: np.ndarray, source_row: np.ndarray) -> np.ndarray:
    """out[r] = tensor[source_row[r]], zeros where source_row[r] < 0 (the zero Adam moments of new points,
    gaussian_splatting.py:539-543)."""
    out = np.zeros((len(source_row),) + tensor.shape[1:], dtype=tensor.dtype)
    ok = source_row >= 0
    out[ok] = tensor[source_row[ok]]
    return out


def densify_masks(grad_accum: np.ndarray, denom: np.ndarray, scaling: np.ndarray, grad_threshold: float,
                  scale_threshold: float) -> Tuple[np.ndarray, np.ndarray]:
    """gaussian_splatting.py:623-626 (grads = accum / denom, NaN -> 0), :612-615 (clone: norm >= threshold and largest
    scale <= extent threshold), :585-589 (split: grad >= threshold and largest scale > extent threshold)."""
    with np.errstate(divide='ignore', invalid='ignore'):
        g = (grad_accum.reshape(-1).astype(np.float32) / denom.reshape(-1).astype(np.float32)).astype(np.float32)
    g[np.isnan(g)] = 0.0
    big = scaling.max(axis=1)
    thr, ext = np.float32(grad_threshold), np.float32(scale_threshold)
    return (np.abs(g) >= thr) & (big <= ext), (g >= thr) & (big > ext)


def prune_mask(opacity: np.ndarray, max_radii2D: np.ndarray, scaling: np.ndarray, min_opacity: float,
               max_screen_size: Optional[float], world_threshold: float) -> np.ndarray:
    """gaussian_splatting.py:630-635."""
    m = opacity.reshape(-1) < np.float32(min_opacity)
    if max_screen_size:
        m = m | (max_radii2D > np.float32(max_screen_size)) | (scaling.max(axis=1) > np.float32(world_threshold))
    return m


def quaternion_to_R(q: np.ndarray) -> np.ndarray:
    """utils/ops_3d/quaternion.py:164-174 (xyzw, normalised with F.normalize's 1e-12 floor)."""
    n = np.maximum(np.sqrt((q * q).sum(-1, keepdims=True)), q.dtype.type(1e-12))
    x, y, z, w = np.moveaxis(q / n, -1, 0)
    R = np.stack([1 - 2 * y * y - 2 * z * z, 2 * x * y - 2 * w * z, 2 * w * y + 2 * x * z,
                  2 * x * y + 2 * w * z, 1 - 2 * x * x - 2 * z * z, 2 * y * z - 2 * w * x,
                  2 * x * z - 2 * w * y, 2 * w * x + 2 * y * z, 1 - 2 * x * x - 2 * y * y], -1)
    return R.reshape(q.shape[:-1] + (3, 3))


def split_children(selected: np.ndarray, N: int, xyz: np.ndarray, scaling: np.ndarray, rotations: np.ndarray,
                   noise: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """gaussian_splatting.py:591-597 / network.py:1170-1183: stds = scale[selected].repeat(N, 1) (a surfel gets a zero
    third axis), samples = noise * stds (`torch.normal(0, std)`), xyz' = R samples + xyz[selected].repeat(N, 1),
    scale' = log(scale[selected].repeat(N, 1) / (0.8 N))."""
    stds = np.tile(scaling[selected], (N, 1))
    stds3 = stds if stds.shape[1] == 3 else np.concatenate([stds, np.zeros_like(stds[:, :1])], 1)
    samples = noise.astype(xyz.dtype) * stds3
    R = np.tile(quaternion_to_R(rotations[selected]), (N, 1, 1))
    new_xyz = np.einsum('nij,nj->ni', R, samples) + np.tile(xyz[selected], (N, 1))
    return new_xyz.astype(xyz.dtype), np.log(stds / xyz.dtype.type(0.8 * N)).astype(xyz.dtype)


def densification_stats(radii: np.ndarray, grad: np.ndarray, max_radii2D: np.ndarray, grad_accum: np.ndarray,
                        denom: np.ndarray, factor: Optional[np.ndarray] = None):
    """network.py:1276-1282 with gaussian_splatting.py:486-495 (network.py:1152-1154 multiplies by factor_culling).
    Returns the updated (max_radii2D, grad_accum, denom, visible)."""
    vis = radii > 0
    mr, acc, den = max_radii2D.copy(), grad_accum.copy().reshape(-1), denom.copy().reshape(-1)
    mr[vis] = np.maximum(mr[vis], radii[vis].astype(np.float32))
    gx, gy = grad[:, 0].astype(np.float32), grad[:, 1].astype(np.float32)
    n = np.sqrt((gx * gx).astype(np.float32) + (gy * gy).astype(np.float32)).astype(np.float32)
    if factor is not None:
        n = (n * factor.reshape(-1)).astype(np.float32)
    acc[vis] = acc[vis] + n[vis]
    den[vis] = den[vis] + np.float32(1)
    return mr, acc.reshape(grad_accum.shape), den.reshape(denom.shape), vis


class PointSet:
    """Parameters, Adam moments and statistics as plain arrays, changed the way the reference changes them."""

    def __init__(self, params: Dict[str, np.ndarray], moments: Optional[Dict[str, Tuple[np.ndarray, np.ndarray]]] = None):
        self.params = {k: v.copy() for k, v in params.items()}
        self.moments = {k: (m.copy(), v.copy()) for k, (m, v) in (moments or {}).items()}
        P = len(self.params['xyz'])
        self.grad_accum = np.zeros((P, 1), np.float32)
        self.denom = np.zeros((P, 1), np.float32)
        self.max_radii2D = np.zeros((P,), np.float32)

    @property
    def P(self):
        return len(self.params['xyz'])

    def scaling(self):
        return np.exp(self.params['scaling'])  # gaussian_splatting.py:142, :460

    def opacity(self):
        return (1 / (1 + np.exp(-self.params['opacity'].astype(np.float64)))).astype(np.float32)  # :145

    def prune_points(self, mask):
        """gaussian_splatting.py:557-568 with change_optimizer op='prune' (:526-527, :544-546)."""
        keep = ~mask
        self.params = {k: v[keep] for k, v in self.params.items()}
        self.moments = {k: (m[keep], v[keep]) for k, (m, v) in self.moments.items()}
        self.grad_accum, self.denom, self.max_radii2D = self.grad_accum[keep], self.denom[keep], self.max_radii2D[keep]

    def densification_postfix(self, new: Dict[str, np.ndarray]):
        """gaussian_splatting.py:570-579 with change_optimizer op='concat' (:524-525, :539-543)."""
        self.params = {k: np.concatenate([v, new[k]], 0) for k, v in self.params.items()}
        self.moments = {k: (np.concatenate([m, np.zeros_like(new[k])], 0), np.concatenate([v, np.zeros_like(new[k])], 0))
                        for k, (m, v) in self.moments.items()}
        P = self.P
        self.grad_accum, self.denom = np.zeros((P, 1), np.float32), np.zeros((P, 1), np.float32)
        self.max_radii2D = np.zeros((P,), np.float32)

    def densify_and_clone(self, grads, grad_threshold, scale_threshold):
        """gaussian_splatting.py:610-621."""
        sel = (np.abs(grads.reshape(-1)) >= np.float32(grad_threshold)) & \
              (self.scaling().max(1) <= np.float32(scale_threshold))
        self.densification_postfix({k: v[sel] for k, v in self.params.items()})
        return sel

    def densify_and_split(self, grads, grad_threshold, scale_threshold, noise, N=2):
        """gaussian_splatting.py:581-608; `noise` [N * selected, 3] stands for the standard normal draws."""
        padded = np.zeros((self.P,), np.float32)
        padded[:len(grads)] = grads.reshape(-1)
        sel = (padded >= np.float32(grad_threshold)) & (self.scaling().max(1) > np.float32(scale_threshold))
        idx = np.flatnonzero(sel)
        new_xyz, new_scaling = split_children(idx, N, self.params['xyz'], self.scaling(), self.params['rotation'], noise)
        new = {k: np.tile(v[sel], (N,) + (1,) * (v.ndim - 1)) for k, v in self.params.items()}
        new['xyz'], new['scaling'] = new_xyz, new_scaling
        self.densification_postfix(new)
        self.prune_points(np.concatenate([sel, np.zeros(N * int(sel.sum()), bool)]))
        return sel

    def densify(self, max_grad, extent, noise, percent_dense=0.01, N=2):
        """gaussian_splatting.py:623-628."""
        with np.errstate(divide='ignore', invalid='ignore'):
            grads = (self.grad_accum / self.denom).astype(np.float32)
        grads[np.isnan(grads)] = 0.0
        self.densify_and_clone(grads, max_grad, percent_dense * extent)
        self.densify_and_split(grads, max_grad, percent_dense * extent, noise, N)

    def prune(self, min_opacity, extent, max_screen_size, percent_dense=0.1):
        """gaussian_splatting.py:630-636."""
        self.prune_points(prune_mask(self.opacity(), self.max_radii2D, self.scaling(), min_opacity, max_screen_size,
                                     percent_dense * extent))
