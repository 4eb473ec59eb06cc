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

__all__ = ['DeformNetwork', 'superpoint_deform', 'deform_apply']


class DeformNetwork(nn.Module):
    """D x Linear(W)+ReLU with the encoded input re-concatenated after layer D//2, heads warp(3) / rotation(4) /
    scaling(3). Parameters are fp32 torch tensors initialised as the reference does (network.py:1741-1755); the forward
    runs in bf16 on the matrix cores through `mlp_forward`."""

    def __init__(self, D=8, W=256, p_degree=10, t_degree=10):
        super().__init__()
        self.D, self.W, self.skip = D, W, D // 2
        self.pos_enc_p = FreqEncoder(3, p_degree, True)
        self.pos_enc_t = FreqEncoder(1, t_degree, True)
        self.input_ch = self.pos_enc_p.output_dim + self.pos_enc_t.output_dim
        self.linear = nn.ModuleList(
            [nn.Linear(self.input_ch, W)] +
            [nn.Linear(W, W) if i != self.skip else nn.Linear(W + self.input_ch, W) for i in range(D - 1)])
        self.gaussian_warp = nn.Linear(W, 3)
        self.gaussian_scaling = nn.Linear(W, 3)
        self.gaussian_rotation = nn.Linear(W, 4)
        for layer in self.linear:
            nn.init.kaiming_uniform_(layer.weight, mode='fan_in', nonlinearity='relu')
            nn.init.zeros_(layer.bias)
        nn.init.normal_(self.gaussian_warp.weight, mean=0, std=1e-5)
        nn.init.normal_(self.gaussian_scaling.weight, mean=0, std=1e-8)
        nn.init.normal_(self.gaussian_rotation.weight, mean=0, std=1e-5)
        for head in (self.gaussian_warp, self.gaussian_scaling, self.gaussian_rotation):
            nn.init.zeros_(head.bias)
        self._packed = None

    def pack(self, transposed: bool = True):
        """Refresh the bf16 weight buffers, the bias vector and the stacked head rows from the parameters in one launch
        (call after every optimiser step on these parameters). `transposed` also makes the copy the backward reads."""
        heads = (self.gaussian_warp, self.gaussian_rotation, self.gaussian_scaling)
        packed, packed_t, bias, heads_w = get_C_function('mlp_pack_all')(
            [l.weight.detach() for l in self.linear], [l.bias.detach() for l in self.linear],
            [h.weight.detach() for h in heads], [h.bias.detach() for h in heads], self.skip, transposed)
        self._packed = (packed, bias)
        self._packed_t = packed_t
        self._heads_w = heads_w
        return self._packed

    def encode(self, x: Tensor, t: Tensor) -> Tensor:
        t_emb = self.pos_enc_t(t.view(-1, 1)).expand(x.shape[0], self.pos_enc_t.output_dim)
        return torch.cat([self.pos_enc_p(x), t_emb], dim=-1).contiguous()

    def _mlp_parameters(self) -> List[Tensor]:
        layers = list(self.linear) + [self.gaussian_warp, self.gaussian_rotation, self.gaussian_scaling]
        return [p for l in layers for p in (l.weight, l.bias)]

    def forward(self, x: Tensor, t: Tensor):
        """bf16 MFMA forward. With gradients enabled the weights are re-packed when they changed since the last call
        and the output carries a backward (see `_DeformMlp`); under `torch.no_grad()` the cached pack is used."""
        params = self._mlp_parameters()
        x_enc = self.encode(x, t)
        track = torch.is_grad_enabled() and (x_enc.requires_grad or any(p.requires_grad for p in params))
        versions = tuple(p._version for p in params)
        if self._packed is None or (track and (getattr(self, '_packed_versions', None) != versions or
                                               self._packed_t is None)):
            self.pack(transposed=track)
            self._packed_versions = versions
        packed, bias = self._packed
        if track:
            out = _DeformMlp.apply(x_enc, packed, bias, self._packed_t, self._heads_w, self.D, self.skip, *params)
        else:
            out = get_C_function('mlp_forward')(x_enc.detach(), packed, bias, self.D, self.skip, 10)
        d_xyz, rotation, scaling = out[:, 0:3], out[:, 3:7], out[:, 7:10]
        return d_xyz, rotation, scaling, None

    def forward_fp32(self, x: Tensor, t: Tensor):
        """The same network in plain fp32 torch (what the reference computes); used to state the bf16 tolerance."""
        x0 = self.encode(x, t)
        h = x0
        for i, l in enumerate(self.linear):
            h = torch.relu(l(h))
            if i == self.skip:
                h = torch.cat([x0, h], -1)
        return self.gaussian_warp(h), self.gaussian_rotation(h), self.gaussian_scaling(h), None


class _DeformMlp(torch.autograd.Function):
    """Forward: the fused bf16 MFMA kernel, which also stores every layer's post-ReLU state. Backward: the chain and
    weight-gradient MFMA kernels; gradients come back in one flat buffer and are handed out as views in parameter
    order (weight, bias per layer, then the warp / rotation / scaling heads). The encoded input gets no gradient (the
    reference feeds detached control points, network.py:586)."""

    @staticmethod
    def forward(ctx, x_enc, packed, bias, packed_t, heads_w, D, skip, *params):
        out, saved = get_C_function('mlp_forward')(x_enc, packed, bias, D, skip, 10, True)
        ctx.save_for_backward(x_enc, packed_t, heads_w, saved)
        ctx.D, ctx.skip = D, skip
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x_enc, packed_t, heads_w, saved = ctx.saved_tensors
        D, skip, Din = ctx.D, ctx.skip, x_enc.shape[1]
        g_w, g_b = get_C_function('mlp_backward')(x_enc, packed_t, heads_w, saved, grad_out.contiguous(), D, skip)
        grads, off = [], 0
        for i in range(D):
            K = Din if i == 0 else (Din + 256 if i == skip + 1 else 256)
            grads += [g_w[off:off + 256 * K].view(256, K), g_b[256 * i:256 * (i + 1)]]
            off += 256 * K
        lo = 0
        for n in (3, 4, 3):  # gaussian_warp, gaussian_rotation, gaussian_scaling rows of the stacked heads
            grads += [g_w[off + 256 * lo:off + 256 * (lo + n)].view(n, 256), g_b[256 * D + lo:256 * D + lo + n]]
            lo += n
        need = ctx.needs_input_grad[7:]
        return (None,) * 7 + tuple(g if n else None for g, n in zip(grads, need))


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
    @staticmethod
    def forward(ctx, points, sp_points, sp_t, sp_r, sp_s, d2, idx, temperature, centred):
        d_xyz, d_rot, d_scale, w = get_C_function('lbs_blend')(points, sp_points, sp_t, sp_r, sp_s, d2, idx,
                                                               temperature, centred)
        ctx.save_for_backward(points, sp_points, sp_t, sp_r, sp_s, d2, idx)
        ctx.temperature, ctx.centred = temperature, centred
        ctx.mark_non_differentiable(w)
        return d_xyz, d_rot, d_scale, w

    @staticmethod
    def backward(ctx, g_xyz, g_rot, g_scale, _):
        points, sp_points, sp_t, sp_r, sp_s, d2, idx = ctx.saved_tensors
        need = ctx.needs_input_grad
        g_points, g_d2, g_c, g_t, g_r, g_s = get_C_function('lbs_blend_backward')(
            points, sp_points, sp_t, sp_r, sp_s, d2, idx, g_xyz.contiguous(), g_rot.contiguous(),
            None if sp_s is None else g_scale.contiguous(), ctx.temperature, ctx.centred, need[0])
        pick = lambda g, n: g if n else None
        return (g_points, pick(g_c, need[1]), pick(g_t, need[2]), pick(g_r, need[3]), pick(g_s, need[4]),
                pick(g_d2, need[5]), None, None, None)


def superpoint_deform(points: Tensor, sp_points: Tensor, sp_t: Tensor, sp_r: Tensor, sp_s: Tensor, K: int = 4,
                      temperature: float = 1.0, centred: bool = False):
    """K-NN of Gaussians to control points, `softmax(-d^2 / temperature)` weights (LBS_method='dist', network.py:517) and
    the LBS warp (network.py:545-573). Returns (d_xyz, d_rot, d_scale, weights, indices). Differentiable with respect to
    points, sp_points (through the distances and, when centred, the pivot), sp_t, sp_r and sp_s; the returned weights
    are detached. The reference detaches `points` before this stage (network.py:577)."""
    d2, idx = _KnnTopk.apply(points.contiguous(), sp_points.contiguous(), K)
    d_xyz, d_rot, d_scale, w = _LbsBlend.apply(points.contiguous(), sp_points.contiguous(), sp_t.contiguous(),
                                               sp_r.contiguous(), None if sp_s is None else sp_s.contiguous(), d2, idx,
                                               temperature, centred)
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
