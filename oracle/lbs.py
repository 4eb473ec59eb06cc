"""TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's superpoint weights and warp in plain torch.

The reference's path for this stage IS torch code (fast_2d_gs/network.py:498-573), differentiated by torch autograd, so
the restatement is torch too: `lbs_weights` follows calc_LBS_weight's weight branches (:507-517), `warp` follows warp()
(:545-573) for apply_rotate == 'add' (the only value that completes: 'qmul' raises NotImplementedError at :569) and
methods 'LBS' / 'LBS_c', and the backward is torch.autograd of these functions. Run in float64 for parity checks.

Third-party conventions (parity unpinned: lietorch is neither vendored nor version-pinned by the reference):
`SE3.InitFromVec(cat([t, q]))` with q = (x, y, z, w) and `.act(p) = R(q) p + t`; `SO3.InitFromVec(q).act(p) = R(q) p`.

What the build adds to the reference's semantics: neighbour slots whose index is outside [0, M) (the -1 padding a K-NN
returns when K > M; the reference always has K <= M) get weight 0 and take no part in the normalisation.

Pinned by tests/test_oracle_ops.py: closed forms (identity -> 0, one control point -> rigid motion through
scipy.spatial.transform.Rotation, rotation about the control point for LBS_c, translation-only without a local
rotation), weights against torch.softmax / explicit per-row loops, limiting cases of the kernel weights.
"""
from __future__ import annotations

import torch


def quat_to_matrix(q: torch.Tensor) -> torch.Tensor:
    """Rotation matrix of unit quaternions (x, y, z, w) (utils/ops_3d/quaternion.py:164-174)."""
    x, y, z, w = q.unbind(-1)
    R = torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (y * w + x * z),
                     2 * (x * y + z * w), 1 - 2 * (x * x + z * z), 2 * (y * z - x * w),
                     2 * (x * z - y * w), 2 * (x * w + y * z), 1 - 2 * (x * x + y * y)], -1)
    return R.reshape(*q.shape[:-1], 3, 3)


def lbs_weights(pair_in: torch.Tensor, indices: torch.Tensor, M: int, method: str, temperature: float = 1.0,
                sp_radius: torch.Tensor = None, sp_weight: torch.Tensor = None) -> torch.Tensor:
    """network.py:507-517. `pair_in`: squared distances for 'dist' / 'kernel' / 'weighted_kernel', the gather
    sp_W[n, indices[n, k]] for 'W' (:515), the finished weights for 'given'. `sp_radius` / `sp_weight` are the raw
    parameters (_sp_radius, _sp_weight): radius = exp(.) (:255-256), weight = sigmoid(.) (:259-260)."""
    valid = (indices >= 0) & (indices < M)
    safe = indices.clamp(0, M - 1)
    if method in ('kernel', 'weighted_kernel'):
        radius = torch.exp(sp_radius)[safe]
        weights = torch.exp(-pair_in / (2 * radius ** 2))
        if method == 'weighted_kernel':
            weights = weights * torch.sigmoid(sp_weight)[safe]
        weights = (weights + 1e-7) * valid
        return weights / weights.sum(dim=-1, keepdim=True)
    if method == 'W':
        return torch.softmax(pair_in.masked_fill(~valid, float('-inf')), dim=-1)
    if method == 'dist':
        return torch.softmax((-pair_in / temperature).masked_fill(~valid, float('-inf')), dim=-1)
    if method == 'given':
        return pair_in * valid
    raise ValueError(method)


def warp(points, sp_points, sp_t, sp_r, sp_s, sp_rot, weights, indices, method='LBS', p2sp=None):
    """network.py:545-573 -> (d_points, d_rotation, d_scales). sp_rot None: translations only (:563-564). Any method
    other than 'LBS' / 'LBS_c' takes the reference's last branch (:555-561): every point is moved by the transform of its
    assigned control point `p2sp` ([N] indices; sp_stage assigns the neighbour of largest weight, :594)."""
    M = sp_points.shape[0]
    safe = indices.clamp(0, M - 1)
    if sp_rot is not None:
        q = sp_rot + sp_rot.new_tensor([0, 0, 0, 1.])
        q = q / q.norm(dim=-1, keepdim=True).clamp_min(1e-12)
        R = quat_to_matrix(q)
        if method == 'LBS_c':
            sp_t = sp_t + sp_points + torch.einsum('mab,mb->ma', R, -sp_points)
        if method in ('LBS', 'LBS_c'):
            moved = torch.einsum('nkab,nb->nka', R[safe], points) + sp_t[safe]
            d_points = (moved * weights[..., None]).sum(dim=1) - points
        else:
            if p2sp is None:
                p2sp = torch.gather(indices, -1, weights.argmax(dim=-1, keepdim=True))[:, 0]
            d_points = torch.einsum('nab,nb->na', R[p2sp], points) + sp_t[p2sp] - points
    else:
        d_points = (sp_t[safe] * weights[..., None]).sum(dim=1)
    d_rotation = (sp_r[safe] * weights[..., None]).sum(dim=1)
    d_scales = (sp_s[safe] * weights[..., None]).sum(dim=1) if sp_s is not None else None
    return d_points, d_rotation, d_scales


def lbs_blend(points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, indices, weight_method='dist', temperature=1.0,
              warp_method='LBS', sp_radius=None, sp_weight=None):
    """Weights + warp -> (d_points, d_rotation, d_scales, weights)."""
    w = lbs_weights(pair_in, indices, sp_points.shape[0], weight_method, temperature, sp_radius, sp_weight)
    return (*warp(points, sp_points, sp_t, sp_r, sp_s, sp_rot, w, indices, warp_method), w)


def lbs_blend_backward(points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, indices, g_xyz, g_rot, g_scale,
                       weight_method='dist', temperature=1.0, warp_method='LBS', sp_radius=None, sp_weight=None):
    """torch.autograd of `lbs_blend`, which is how the reference differentiates this stage. Returns a dict of gradients
    (None for absent inputs): points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, sp_radius, sp_weight."""
    names = ['points', 'sp_points', 'sp_t', 'sp_r', 'sp_s', 'sp_rot', 'pair_in', 'sp_radius', 'sp_weight']
    vals = [points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, sp_radius, sp_weight]
    leaves = {n: (None if v is None else v.detach().clone().requires_grad_(True)) for n, v in zip(names, vals)}
    L = leaves
    d_xyz, d_rot, d_scale, _ = lbs_blend(L['points'], L['sp_points'], L['sp_t'], L['sp_r'], L['sp_s'], L['sp_rot'],
                                         L['pair_in'], indices, weight_method, temperature, warp_method,
                                         L['sp_radius'], L['sp_weight'])
    loss = (d_xyz * g_xyz).sum() + (d_rot * g_rot).sum()
    if d_scale is not None:
        loss = loss + (d_scale * g_scale).sum()
    present = [n for n in names if leaves[n] is not None]
    grads = torch.autograd.grad(loss, [leaves[n] for n in present], allow_unused=True)
    out = {n: None for n in names}
    for n, g in zip(present, grads):
        out[n] = torch.zeros_like(leaves[n]) if g is None else g
    return out
