"""Host side of the superpoint deformation branch: frequency encoders + fused MFMA MLP, K-NN of Gaussians to control
points, and LBS skinning -- the reference's `SC_GS_DeformNetwork` (fast_2d_gs/network.py:1670-1776) and
`calc_LBS_weight` / `warp` (network.py:498-573) on the HIP operators, differentiable like the reference's torch code:
K-NN distances, the LBS blend and the MLP (bf16 MFMA, fp32 accumulation) all have HIP backward kernels."""
from __future__ import annotations

import math
from typing import List, Tuple

import torch
from torch import Tensor, nn

from fast_sp_gs_amd._C import get_C_function
from fast_sp_gs_amd.ops import FreqEncoder

__all__ = ['DeformNetwork', 'superpoint_deform', 'deform_apply', 'calc_LBS_weight', 'warp', 'knn_points']


class DeformNetwork(nn.Module):
    """The reference's SC_GS_DeformNetwork (network.py:1670-1776): D x Linear(W)+ReLU with the encoded input
    re-concatenated after layer D//2, heads warp(3) / rotation(4) / scaling(3) and, with `local_frame`, a fourth head
    local_rotation(4). `is_blender` puts the reference's small time network (Linear(.., 256) + ReLU + Linear(256, 30),
    :1707-1713) between the time encoding and the trunk, as the D-NeRF configuration does (exps/d_nerf.yaml:15).
    Parameters are fp32 torch tensors initialised as the reference does (:1741-1755); the trunk and the heads run in
    bf16 on the matrix cores through `mlp_forward`, the time network (one row per step) in torch."""

    def __init__(self, D=8, W=256, p_degree=10, t_degree=10, is_blender=False, local_frame=False, max_d_scale=-1.0):
        super().__init__()
        self.D, self.W, self.skip = D, W, D // 2
        self.pos_enc_p = FreqEncoder(3, p_degree, True)
        self.pos_enc_t = FreqEncoder(1, t_degree, True)
        self.is_blender, self.local_frame, self.max_d_scale = is_blender, local_frame, max_d_scale
        if is_blender:
            self.time_out = 30
            self.timenet = nn.Sequential(nn.Linear(self.pos_enc_t.output_dim, 256), nn.ReLU(inplace=True),
                                         nn.Linear(256, self.time_out))
            self.input_ch = self.pos_enc_p.output_dim + self.time_out
        else:
            self.input_ch = self.pos_enc_p.output_dim + self.pos_enc_t.output_dim
        self.linear = nn.ModuleList(
            [nn.Linear(self.input_ch, W)] +
            [nn.Linear(W, W) if i != self.skip else nn.Linear(W + self.input_ch, W) for i in range(D - 1)])
        self.gaussian_warp = nn.Linear(W, 3)
        self.gaussian_scaling = nn.Linear(W, 3)
        self.gaussian_rotation = nn.Linear(W, 4)
        if local_frame:
            self.local_rotation = nn.Linear(W, 4)
            nn.init.normal_(self.local_rotation.weight, mean=0, std=1e-4)
            nn.init.zeros_(self.local_rotation.bias)
        for layer in self.linear:
            nn.init.kaiming_uniform_(layer.weight, mode='fan_in', nonlinearity='relu')
            nn.init.zeros_(layer.bias)
        nn.init.normal_(self.gaussian_warp.weight, mean=0, std=1e-5)
        nn.init.normal_(self.gaussian_scaling.weight, mean=0, std=1e-8)
        nn.init.normal_(self.gaussian_rotation.weight, mean=0, std=1e-5)
        for head in (self.gaussian_warp, self.gaussian_scaling, self.gaussian_rotation):
            nn.init.zeros_(head.bias)
        self._packed = None

    def _heads(self):
        """Head order inside the fused kernel's stacked output: warp, rotation, scaling (, local rotation)."""
        heads = [self.gaussian_warp, self.gaussian_rotation, self.gaussian_scaling]
        return heads + [self.local_rotation] if self.local_frame else heads

    def pack(self, transposed: bool = True):
        """Refresh the bf16 weight buffers, the bias vector and the stacked head rows from the parameters in one launch
        (call after every optimiser step on these parameters). `transposed` also makes the copy the backward reads."""
        heads = self._heads()
        packed, packed_t, bias, heads_w = get_C_function('mlp_pack_all')(
            [l.weight.detach() for l in self.linear], [l.bias.detach() for l in self.linear],
            [h.weight.detach() for h in heads], [h.bias.detach() for h in heads], self.skip, transposed)
        self._packed = (packed, bias)
        self._packed_t = packed_t
        self._heads_w = heads_w
        return self._packed

    def encode(self, x: Tensor, t: Tensor) -> Tensor:
        t_emb = self.pos_enc_t(t.view(-1, 1))
        if self.is_blender:
            t_emb = self.timenet(t_emb)
        return torch.cat([self.pos_enc_p(x), t_emb.expand(x.shape[0], t_emb.shape[-1])], dim=-1).contiguous()

    def _mlp_parameters(self) -> List[Tensor]:
        return [p for l in list(self.linear) + self._heads() for p in (l.weight, l.bias)]

    def _split(self, out: Tensor):
        d_xyz, rotation, scaling = out[:, 0:3], out[:, 3:7], out[:, 7:10]
        if self.max_d_scale > 0:
            scaling = torch.tanh(scaling) * math.log(self.max_d_scale)
        return d_xyz, rotation, scaling, (out[:, 10:14] if self.local_frame else None)

    def forward(self, x: Tensor, t: Tensor):
        """bf16 MFMA forward -> (d_xyz, rotation, scaling, local_rotation | None), the reference's return order
        (network.py:1776). With gradients enabled the weights are re-packed when they changed since the last call and
        the output carries a backward (see `_DeformMlp`); under `torch.no_grad()` the cached pack is used."""
        params = self._mlp_parameters()
        x_enc = self.encode(x, t)
        n_out = 14 if self.local_frame else 10
        track = torch.is_grad_enabled() and (x_enc.requires_grad or any(p.requires_grad for p in params))
        versions = tuple(p._version for p in params)
        if self._packed is None or (track and (getattr(self, '_packed_versions', None) != versions or
                                               self._packed_t is None)):
            self.pack(transposed=track)
            self._packed_versions = versions
        packed, bias = self._packed
        if track:
            out = _DeformMlp.apply(x_enc, packed, bias, self._packed_t, self._heads_w, self.D, self.skip, n_out,
                                   *params)
        else:
            out = get_C_function('mlp_forward')(x_enc.detach(), packed, bias, self.D, self.skip, n_out)
        return self._split(out)

    def forward_fp32(self, x: Tensor, t: Tensor):
        """The same network in plain fp32 torch (what the reference computes); used to state the bf16 tolerance."""
        x0 = self.encode(x, t)
        h = x0
        for i, l in enumerate(self.linear):
            h = torch.relu(l(h))
            if i == self.skip:
                h = torch.cat([x0, h], -1)
        return self._split(torch.cat([head(h) for head in self._heads()], -1))


class _DeformMlp(torch.autograd.Function):
    """Forward: the fused bf16 MFMA kernel, which also stores every layer's post-ReLU state. Backward: the chain and
    weight-gradient MFMA kernels; gradients come back in one flat buffer and are handed out as views in parameter
    order (weight, bias per layer, then the heads). The encoded input gets a gradient only when it asks for one (the
    reference feeds detached control points, network.py:586, so that is the time network's output, the same row for
    every control point): dZ_0 W_0 + dZ_{skip+1} W_{skip+1}[:, :Din] from the pre-activation gradients the chain
    kernel leaves behind, as two small torch products."""

    @staticmethod
    def forward(ctx, x_enc, packed, bias, packed_t, heads_w, D, skip, n_out, *params):
        out, saved = get_C_function('mlp_forward')(x_enc, packed, bias, D, skip, n_out, True)
        ctx.save_for_backward(x_enc, packed_t, heads_w, saved, params[0], params[2 * (skip + 1)])
        ctx.D, ctx.skip = D, skip
        ctx.head_rows = [p.shape[0] for p in params[2 * D::2]]
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x_enc, packed_t, heads_w, saved, w_first, w_skip = ctx.saved_tensors
        D, skip, Din = ctx.D, ctx.skip, x_enc.shape[1]
        need_in = ctx.needs_input_grad[0]
        res = get_C_function('mlp_backward')(x_enc, packed_t, heads_w, saved, grad_out.contiguous(), D, skip, need_in)
        g_w, g_b = res[0], res[1]
        g_in = None
        if need_in:
            dz = res[2]
            g_in = dz[0].float() @ w_first.detach() + dz[skip + 1].float() @ w_skip.detach()[:, :Din]
        grads, off = [], 0
        for i in range(D):
            K = Din if i == 0 else (Din + 256 if i == skip + 1 else 256)
            grads += [g_w[off:off + 256 * K].view(256, K), g_b[256 * i:256 * (i + 1)]]
            off += 256 * K
        lo = 0
        for n in ctx.head_rows:  # rows of the stacked heads, in the order of DeformNetwork._heads()
            grads += [g_w[off + 256 * lo:off + 256 * (lo + n)].view(n, 256), g_b[256 * D + lo:256 * D + lo + n]]
            lo += n
        need = ctx.needs_input_grad[8:]
        return (g_in,) + (None,) * 7 + tuple(g if n else None for g, n in zip(grads, need))


class _KnnTopk(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, y, K):
        d2, idx = get_C_function('knn_topk')(x, y, K)
        ctx.save_for_backward(x, y, idx)
        ctx.mark_non_differentiable(idx)
        return d2, idx

    @staticmethod
    def backward(ctx, g_d2, _):
        x, y, idx = ctx.saved_tensors
        g_x, g_y = get_C_function('knn_topk_backward')(x, y, idx, g_d2.contiguous(), ctx.needs_input_grad[0])
        return g_x, (g_y if ctx.needs_input_grad[1] else None), None


class _LbsBlend(torch.autograd.Function):
    """lbs_blend / lbs_blend_backward as one differentiable operator. Optional tensors are passed as None."""

    @staticmethod
    def forward(ctx, points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, idx, sp_log_radius, sp_weight_logit,
                temperature, warp_method, weight_method):
        c = lambda t: None if t is None else t.contiguous()
        args = [c(t) for t in (points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, idx, sp_log_radius,
                               sp_weight_logit)]
        points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, idx, sp_log_radius, sp_weight_logit = args
        d_xyz, d_rot, d_scale, w = get_C_function('lbs_blend')(
            points, sp_points, sp_t, sp_r, sp_s, pair_in, idx, temperature, warp_method, sp_rot, weight_method,
            sp_log_radius, sp_weight_logit)
        ctx.save_for_backward(*[t for t in args if t is not None])
        ctx.present = [t is not None for t in args]
        ctx.cfg = (temperature, warp_method, weight_method)
        ctx.mark_non_differentiable(w)
        return d_xyz, d_rot, d_scale, w

    @staticmethod
    def backward(ctx, g_xyz, g_rot, g_scale, _):
        it = iter(ctx.saved_tensors)
        points, sp_points, sp_t, sp_r, sp_s, sp_rot, pair_in, idx, sp_log_radius, sp_weight_logit = [
            next(it) if p else None for p in ctx.present]
        temperature, warp_method, weight_method = ctx.cfg
        need = ctx.needs_input_grad
        zeros = lambda ref: torch.zeros_like(ref)
        g = get_C_function('lbs_blend_backward')(
            points, sp_points, sp_t, sp_r, sp_s, pair_in, idx,
            (zeros(points) if g_xyz is None else g_xyz.contiguous()),
            (points.new_zeros(points.shape[0], 4) if g_rot is None else g_rot.contiguous()),
            None if sp_s is None else (points.new_zeros(points.shape[0], sp_s.shape[1]) if g_scale is None
                                       else g_scale.contiguous()),
            temperature, warp_method, sp_rot, weight_method, sp_log_radius, sp_weight_logit, need[0])
        pick = lambda key, k: g[key] if need[k] and g[key] is not None else None
        return (pick('g_points', 0), pick('g_sp_points', 1), pick('g_sp_t', 2), pick('g_sp_r', 3), pick('g_sp_s', 4),
                pick('g_sp_rot', 5), pick('g_pair', 6), None, pick('g_log_radius', 8), pick('g_weight_logit', 9),
                None, None, None)


def knn_points(points: Tensor, sp_points: Tensor, K: int):
    """Squared distances (ascending) and indices of the K nearest rows of `sp_points` for every row of `points`: the
    reference's `pytorch3d.ops.knn_points(points[None], sp_points[None], K=K)` (network.py:504) without the batch
    dimension. Differentiable in both point sets through the distances."""
    return _KnnTopk.apply(points.contiguous(), sp_points.contiguous(), K)


def calc_LBS_weight(points: Tensor, sp_points: Tensor, feature: Tensor = None, sp_feature: Tensor = None, K: int = 3,
                    temperature: float = 1.0, LBS_method: str = 'dist', sp_radius: Tensor = None,
                    sp_weight: Tensor = None, sp_W: Tensor = None):
    """The reference's `calc_LBS_weight` (network.py:498-521) -> (weights[N,K], indices[N,K]). The K-NN runs on the HIP
    kernel (positions detached and concatenated with the hyper features when both are given, :500-502); the weights
    are the reference's torch expressions on its raw parameters (`sp_radius` = _sp_radius, `sp_weight` = _sp_weight).
    `superpoint_deform` fuses these weights into the blend kernel; this function is for callers that want them alone."""
    if feature is not None and sp_feature is not None:
        points = torch.cat([points.detach(), feature], dim=-1)
        sp_points = torch.cat([sp_points.detach(), sp_feature], dim=-1)
    nn_dist, indices = knn_points(points, sp_points, K)
    if LBS_method in ('kernel', 'weighted_kernel'):
        radius = torch.exp(sp_radius)[indices]
        weights = torch.exp(-nn_dist / (2 * radius ** 2))
        if LBS_method == 'weighted_kernel':
            weights = weights * torch.sigmoid(sp_weight)[indices]
        weights = weights + 1e-7
        weights = weights / weights.sum(dim=-1, keepdim=True)
    elif LBS_method == 'W':
        weights = torch.gather(sp_W, dim=1, index=indices).softmax(dim=-1)
    else:
        weights = torch.softmax(-nn_dist / temperature, dim=-1)
    return weights, indices


def assign_superpoints(weights: Tensor, indices: Tensor) -> Tensor:
    """p2sp of the reference (network.py:594): for every Gaussian the neighbour that carries its largest weight."""
    return torch.gather(indices, -1, weights.argmax(dim=-1, keepdim=True))[:, 0]


def _rigid_by_assignment(points, sp_points, sp_t, sp_r, sp_rot, p2sp):
    """warp_method 'largest' (network.py:555-561): every Gaussian is moved by the rigid transform of ONE control point,
    `spT[p2sp].act(points) - points`, no blend. The blend kernel with K = 1 and a weight of one is exactly that gather
    (and its backward the scatter of the gradients to the assigned control points)."""
    one = points.new_ones(points.shape[0], 1)
    d_xyz, _, _, _ = _LbsBlend.apply(points, sp_points, sp_t, sp_r, None, sp_rot, one, p2sp.long()[:, None].contiguous(),
                                     None, None, 1.0, 'LBS', 'given')
    return d_xyz


def warp(points: Tensor, sp_points: Tensor, sp_t: Tensor, sp_r: Tensor, sp_s: Tensor, sp_rot: Tensor, weights: Tensor,
         indices: Tensor, method: str = 'LBS', p2sp: Tensor = None):
    """The reference's `warp` (network.py:523-573) for apply_rotate == 'add' on finished weights ->
    (d_points, d_rotation, d_scales). Without `sp_rot` (no local rotation, the default configuration) the translations
    are blended whatever the method; with it every Gaussian is moved by rigid transforms
    (normalize(sp_rot + (0,0,0,1)), sp_t): blended over its neighbours for 'LBS', blended about the control points
    for 'LBS_c', and for 'largest' the one transform of its assigned control point `p2sp` (default: the neighbour with
    the largest weight, as sp_stage assigns it, :594). Rotation and scale residuals are blended in every case.
    Differentiable in everything but the indices."""
    if method not in ('LBS', 'LBS_c', 'largest'):
        raise ValueError(f'unknown warp method {method!r}')  # the reference's assert, network.py:205
    blended = method if (sp_rot is not None and method != 'largest') else None
    d_xyz, d_rot, d_scale, _ = _LbsBlend.apply(points, sp_points, sp_t, sp_r, sp_s, sp_rot if blended else None, weights,
                                               indices, None, None, 1.0, blended, 'given')
    if method == 'largest' and sp_rot is not None:
        if p2sp is None:
            p2sp = assign_superpoints(weights.detach(), indices)
        d_xyz = _rigid_by_assignment(points, sp_points, sp_t, sp_r, sp_rot, p2sp)
    return d_xyz, d_rot, d_scale


def superpoint_deform(points: Tensor, sp_points: Tensor, sp_t: Tensor, sp_r: Tensor, sp_s: Tensor,
                      sp_rot: Tensor = None, K: int = 3, temperature: float = 1.0, warp_method: str = 'LBS',
                      LBS_method: str = 'dist', sp_radius: Tensor = None, sp_weight: Tensor = None,
                      sp_W: Tensor = None, feature: Tensor = None, sp_feature: Tensor = None, p2sp: Tensor = None):
    """`calc_LBS_weight` + `warp` of the reference's `sp_stage` (network.py:576-599) with the weights formed inside the
    blend kernels: K-NN of the Gaussians to the control points (on positions, or on positions + hyper features when
    `feature` / `sp_feature` are given, :500-504), weights by `LBS_method` ('dist', 'kernel', 'weighted_kernel', 'W'),
    then the warp ('LBS', 'LBS_c', or 'largest' with the assignment `p2sp`, by default the neighbour of largest
    weight). Returns (d_xyz, d_rot, d_scale, weights, indices). Differentiable with respect to sp_points and the
    hyper features (through the distances, and sp_points also through the pivot of 'LBS_c'), sp_t, sp_r, sp_s, sp_rot,
    sp_radius, sp_weight and sp_W; the returned weights are detached. As in the reference the Gaussians' positions are
    detached (:577, :501)."""
    points = points.detach()
    if feature is not None and sp_feature is not None:
        x = torch.cat([points, feature], dim=-1)
        y = torch.cat([sp_points.detach(), sp_feature], dim=-1)
    else:
        x, y = points, sp_points
    d2, idx = _KnnTopk.apply(x.contiguous(), y.contiguous(), K)
    if LBS_method == 'W':
        pair_in, radius, weight = torch.gather(sp_W, dim=1, index=idx), None, None
    elif LBS_method in ('kernel', 'weighted_kernel'):
        pair_in, radius, weight = d2, sp_radius, (sp_weight if LBS_method == 'weighted_kernel' else None)
    elif LBS_method == 'dist':
        pair_in, radius, weight = d2, None, None
    else:
        raise ValueError(f'unknown LBS_method {LBS_method!r}')
    if warp_method not in ('LBS', 'LBS_c', 'largest'):
        raise ValueError(f'unknown warp method {warp_method!r}')
    blended = warp_method if (sp_rot is not None and warp_method != 'largest') else None
    d_xyz, d_rot, d_scale, w = _LbsBlend.apply(points, sp_points, sp_t, sp_r, sp_s, sp_rot if blended else None, pair_in,
                                               idx, radius, weight, temperature, blended, LBS_method)
    if warp_method == 'largest' and sp_rot is not None:
        p2sp = assign_superpoints(w, idx) if p2sp is None else p2sp
        d_xyz = _rigid_by_assignment(points, sp_points, sp_t, sp_r, sp_rot, p2sp)
    return d_xyz, d_rot, d_scale, w, idx


class _DeformApply(torch.autograd.Function):
    """points + d_xyz, act(scales) + d_scale, normalize(rotations + d_rotation) (network.py:630, :643, :645) as one
    kernel forward and one backward; sums hand their upstream gradient to both addends unchanged."""

    @staticmethod
    def forward(ctx, points, d_xyz, scales, d_scale, rotations, d_rotation, log_scales):
        args = [t.contiguous() for t in (points, d_xyz, scales, d_scale, rotations, d_rotation)]
        out = get_C_function('deform_apply_forward')(*args, log_scales)
        ctx.save_for_backward(args[2], args[4], args[5])
        ctx.log_scales = log_scales
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, g_points, g_scales, g_rot):
        scales, rotations, d_rotation = ctx.saved_tensors
        need = ctx.needs_input_grad
        gs = g_r = None
        if need[4] or need[5] or (ctx.log_scales and need[2]):
            gs, g_r = get_C_function('deform_apply_backward')(
                scales, rotations, d_rotation, g_scales.contiguous() if ctx.log_scales else None, g_rot.contiguous(),
                ctx.log_scales)
        if not ctx.log_scales:
            gs = g_scales
        pick = lambda g, k: g if need[k] else None
        return pick(g_points, 0), pick(g_points, 1), pick(gs, 2), pick(g_scales, 3), pick(g_r, 4), pick(g_r, 5), None


def deform_apply(points: Tensor, d_xyz: Tensor, scales: Tensor, d_scale: Tensor, rotations: Tensor, d_rotation: Tensor,
                 log_scales: bool = False):
    """The deformed parameters handed to the renderer (reference: fast_2d_gs/network.py:630, :643, :645 with
    apply_rotate == 'add'): (points + d_xyz, scales + d_scale, normalize(rotations + d_rotation)); with `log_scales`
    the scales are stored as logarithms and exp is applied first (gaussian_splatting.py:142)."""
    return _DeformApply.apply(points, d_xyz, scales, d_scale, rotations, d_rotation, bool(log_scales))
