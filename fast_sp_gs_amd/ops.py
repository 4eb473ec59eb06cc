"""Differentiable forms of the stand-alone operators: SH encoder, SH -> RGB, frequency encoder, nearest point.

Each is a `KernelPair` (autograd.py) over the extension's forward / backward operators; the callables keep the
reference's names and argument order so its call sites work unchanged: `sh_encode(dirs, degree)`,
`SH_to_RGB(sh, dirs, campos, degree, clamp)` (utils/ops_3d/spherical_harmonics.py:162-165, 238-240),
`freq_encode(x, degree, include_input, scale)` and the `FreqEncoder` module (fast_2d_gs/freq_encoder.py:38-60),
`cdist_top(x1, x2[, largest]) -> (distance, index)` (utils/cdist_top.py:76).
"""
from __future__ import annotations

import math

import torch
from torch import Tensor, nn

from fast_sp_gs_amd.autograd import KernelPair

__all__ = ['sh_encode', 'SH_to_RGB', 'freq_encode', 'FreqEncoder', 'cdist_top']


# ---- SH basis of unit directions: [B, D >= 3] -> [B, (degree + 1)^2] ---------------------------------------------------
def _sh_launch(fwd, needs, dirs, degree):
    rows, width = dirs.shape
    basis = dirs.new_empty(rows, (degree + 1) ** 2)
    fwd(dirs, basis, rows, width, degree)
    return basis, (dirs,), degree


def _sh_grads(bwd, needs, keep, degree, g_basis):
    dirs, = keep
    g_dirs = torch.zeros_like(dirs)  # the operator writes the first three columns only
    bwd(g_basis, dirs, dirs.shape[0], dirs.shape[1], degree, g_dirs)
    return g_dirs, None


_sh_pair = KernelPair('sh_encode_forward', 'sh_encode_backward', _sh_launch, _sh_grads, autocast_float32=True)


def sh_encode(dirs: Tensor, degree: int) -> Tensor:
    """Real SH basis up to `degree` of the directions in the last dimension; leading dimensions are kept."""
    lead = dirs.shape[:-1]
    return _sh_pair(dirs.reshape(-1, dirs.shape[-1]), degree).reshape(*lead, -1)


# ---- view-dependent colour: SH coefficients [P, F, 3] x direction (or position and camera centre) -> rgb [P, 3] ---------
def _rgb_launch(fwd, needs, sh, dirs, campos, degree, clamp):
    rgb = fwd(dirs, campos, sh, degree, clamp)
    return rgb, (sh, dirs, campos, rgb), (degree, clamp)


def _rgb_grads(bwd, needs, keep, remember, g_rgb):
    sh, dirs, campos, rgb = keep
    degree, clamp = remember
    want = lambda i, like: torch.zeros_like(like) if like is not None and needs[i] else None
    g_sh, g_dirs, g_campos = want(0, sh), want(1, dirs), want(2, campos)
    bwd(degree, clamp, dirs, campos, sh, rgb, g_rgb, g_dirs, g_campos, g_sh)
    return g_sh, g_dirs, g_campos, None, None


_rgb_pair = KernelPair('SH_to_RGB_forward', 'SH_to_RGB_backward', _rgb_launch, _rgb_grads)


def SH_to_RGB(sh: Tensor, dirs: Tensor, campos: Tensor = None, degree: int = 0, clamp: bool = True) -> Tensor:
    """rgb = max(0, sum_k basis_k(dir) sh_k + 0.5) (clamp optional); with `campos`, `dirs` are positions and the
    direction is normalize(position - campos)."""
    return _rgb_pair(sh, dirs, campos, degree, clamp)


# ---- frequency encoding: x -> [x | sin(2^0 s x), cos(2^0 s x), sin(2^1 s x), ...] --------------------------------------
def _freq_launch(fwd, needs, x, degree, include_input, scale):
    if not x.is_cuda:
        x = x.to('cuda')
    encoded = fwd(x, degree, include_input, scale)
    return encoded, (encoded,), (degree, include_input, scale)  # the backward reads sin / cos back from the output


def _freq_grads(bwd, needs, keep, remember, g_encoded):
    encoded, = keep
    return bwd(g_encoded, encoded, *remember), None, None, None


_freq_pair = KernelPair('freq_encode_forward', 'freq_encode_backward', _freq_launch, _freq_grads,
                        autocast_float32=True)


def freq_encode(inputs: Tensor, degree: int, include_input: bool = True, scale: float = 1.0) -> Tensor:
    return _freq_pair(inputs, degree, include_input, scale)


class FreqEncoder(nn.Module):
    """`degree` octaves of sin / cos per input coordinate, optionally preceded by the input itself; scale 'pi' = pi."""

    def __init__(self, input_dim: int = 3, degree: int = 4, include_input: bool = True, scale=1.):
        super().__init__()
        self.input_dim, self.degree, self.include_input = input_dim, degree, include_input
        self.scale = math.pi if scale == 'pi' else float(scale)
        self.output_dim = input_dim * (2 * degree + (1 if include_input else 0))

    def extra_repr(self) -> str:
        return f"{self.input_dim} -> {self.output_dim} (degree {self.degree}, include_input={self.include_input})"

    def forward(self, inputs: Tensor, **_unused) -> Tensor:
        return freq_encode(inputs, self.degree, self.include_input, self.scale)


# ---- nearest (or farthest) point of x2 for every point of x1 ------------------------------------------------------------
def _nearest_launch(fwd, needs, x1, x2, largest=False):
    distance, index = fwd(x1, x2, largest)
    return (distance, index), (x1, x2, distance, index), None


def _nearest_grads(bwd, needs, keep, _, g_distance, _g_index):
    g1, g2 = bwd(*keep, g_distance)
    return (g1, g2, None)[:len(needs)]


_nearest_pair = KernelPair('cdist_top', 'cdist_top_backward', _nearest_launch, _nearest_grads, non_differentiable=(1,))


def cdist_top(x1: Tensor, x2: Tensor, largest: bool = False):
    """(distance[..., N], index[..., N] int64) of the nearest -- `largest`: farthest -- row of x2 for every row of x1."""
    return _nearest_pair(x1, x2, largest)
