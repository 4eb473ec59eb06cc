"""Host side of the superpoint deformation branch: frequency encoders + fused MFMA MLP, K-NN of Gaussians to control
points, and LBS skinning -- the forward path of the reference's `SC_GS_DeformNetwork` (fast_2d_gs/network.py:1670-1776)
and `calc_LBS_weight` / `warp` (network.py:498-573) on the HIP operators."""
from __future__ import annotations

import math
from typing import List, Tuple

import torch
from torch import Tensor, nn

from fast_sp_gs_amd._C import get_C_function
from fast_sp_gs_amd.ops import FreqEncoder

__all__ = ['DeformNetwork', 'superpoint_deform']


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

    def pack(self):
        """Refresh the bf16 weight buffer (call after every optimiser step on these parameters)."""
        heads_w = torch.cat([self.gaussian_warp.weight, self.gaussian_rotation.weight, self.gaussian_scaling.weight], 0)
        heads_b = torch.cat([self.gaussian_warp.bias, self.gaussian_rotation.bias, self.gaussian_scaling.bias], 0)
        weights = [l.weight.detach().contiguous() for l in self.linear]
        packed = get_C_function('mlp_pack_weights')(weights, heads_w.detach().contiguous(), self.skip)
        bias = torch.cat([l.bias.detach() for l in self.linear] + [heads_b.detach()]).contiguous()
        self._packed = (packed, bias)
        return self._packed

    def encode(self, x: Tensor, t: Tensor) -> Tensor:
        t_emb = self.pos_enc_t(t.view(-1, 1)).expand(x.shape[0], self.pos_enc_t.output_dim)
        return torch.cat([self.pos_enc_p(x), t_emb], dim=-1).contiguous()

    @torch.no_grad()
    def forward(self, x: Tensor, t: Tensor):
        packed, bias = self._packed if self._packed is not None else self.pack()
        out = get_C_function('mlp_forward')(self.encode(x, t), packed, bias, self.D, self.skip, 10)
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


@torch.no_grad()
def superpoint_deform(points: Tensor, sp_points: Tensor, sp_t: Tensor, sp_r: Tensor, sp_s: Tensor, K: int = 4,
                      temperature: float = 1.0, centred: bool = False):
    """K-NN of Gaussians to control points, `softmax(-d^2 / temperature)` weights (LBS_method='dist', network.py:517) and
    the LBS warp (network.py:545-573). Returns (d_xyz, d_rot, d_scale, weights, indices)."""
    d2, idx = get_C_function('knn_topk')(points, sp_points, K)
    d_xyz, d_rot, d_scale, w = get_C_function('lbs_blend')(points, sp_points, sp_t.contiguous(), sp_r.contiguous(),
                                                           None if sp_s is None else sp_s.contiguous(), d2, idx,
                                                           temperature, centred)
    return d_xyz, d_rot, d_scale, w, idx
