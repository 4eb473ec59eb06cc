"""TEST INFRASTRUCTURE ONLY: CPU restatement of the deformation MLP's forward and backward in float64 torch.

The reference's network (fast_2d_gs/network.py:1670-1776) is D x (Linear(256) + ReLU) with the encoded input
re-concatenated in front of the hidden state after layer D // 2 (`skips`, :1695, :1766-1767) and linear heads on the
last hidden state; its backward is torch autograd. `mlp_forward` / `mlp_backward` below write both passes out by hand
(matrix products and masks only, no autograd), so that

  * with `round_bf16=False` the backward must equal torch.autograd of the same network in float64 to rounding -- that is
    what pins this file (tests/test_oracle_mlp.py: every weight, bias, head and the input gradient, four shapes, skip
    layer included), and
  * with `round_bf16=True` it restates the arithmetic of the HIP kernels, which keep operands in bf16 where the matrix
    cores take them: the encoded input, the hidden weights, the stored hidden states (`hidden`, handed in by the caller:
    their zeros are the ReLU mask), every dZ where it is stored, and g_out for the heads' gradients; sums stay float64
    (fp32 on the GPU). The GPU parity test calls it on the states the forward kernel stored.

Layout: weights[l] is [256, K_l] with K_0 = Din, K_{skip+1} = Din + 256 (input columns first), 256 otherwise;
head_w is the heads stacked along rows [n_out, 256].
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


def _bf16(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).to(torch.bfloat16).to(torch.float64)


def mlp_forward(x_enc, weights: Sequence, biases: Sequence, head_w, head_b, skip: int):
    """-> (out[B, n_out], hidden: list of the D post-ReLU states [B, 256]); float64, no rounding."""
    x0 = x_enc.double()
    h, hidden = x0, []
    for l, (W, b) in enumerate(zip(weights, biases)):
        inp = torch.cat([x0, h], -1) if l == skip + 1 else h
        h = torch.clamp_min(inp @ W.double().t() + b.double(), 0.0)
        hidden.append(h)
    return h @ head_w.double().t() + head_b.double(), hidden


def mlp_backward(x_enc, weights: Sequence, head_w, skip: int, g_out, hidden: Sequence, round_bf16: bool = False):
    """Chain rule through the network at the given post-ReLU states.
    -> dict: 'weights' / 'biases' (lists, layer order), 'head_w' [n_out,256], 'head_b' [n_out], 'x' [B,Din] (gradient of
    the encoded input through layer 0 and through the skip concatenation), 'dz' (list of the pre-activation gradients)."""
    r = _bf16 if round_bf16 else (lambda t: t.double())
    D, Din = len(weights), x_enc.shape[1]
    x0 = r(x_enc)
    H = [h.double() for h in hidden]  # stored states are bf16 values already when they come from the kernel
    g_out = g_out.double()
    out = {'head_w': r(g_out).t() @ H[D - 1], 'head_b': r(g_out).sum(0), 'weights': [None] * D, 'biases': [None] * D,
           'dz': [None] * D}
    # the chain starts from the unrounded product g_out . W_heads; every dZ is rounded where the kernel stores it
    dZ = r((g_out @ head_w.double()) * (H[D - 1] != 0))
    g_x = torch.zeros(x_enc.shape[0], Din, dtype=torch.float64)
    for l in range(D - 1, -1, -1):
        X = x0 if l == 0 else (torch.cat([x0, H[l - 1]], -1) if l == skip + 1 else H[l - 1])
        out['weights'][l] = dZ.t() @ X
        out['biases'][l] = dZ.sum(0)
        out['dz'][l] = dZ
        W = weights[l].double()
        if l == 0:
            g_x = g_x + dZ @ W
        else:
            if l == skip + 1:
                g_x = g_x + dZ @ W[:, :Din]
            dZ = r((dZ @ r(W[:, -256:])) * (H[l - 1] != 0))
    out['x'] = g_x
    return out
