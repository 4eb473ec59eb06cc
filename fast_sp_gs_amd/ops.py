"""Autograd wrappers of the stand-alone operators, mirroring the reference's host code:
`sh_encode` / `SH_to_RGB` (utils/ops_3d/spherical_harmonics.py:128-165, 205-240), `freq_encode` / `FreqEncoder`
(fast_2d_gs/freq_encoder.py:12-60), `cdist_top` (utils/cdist_top.py:42-76)."""
from __future__ import annotations

import torch
from torch import Tensor, nn
from torch.autograd import Function
from torch.amp import custom_bwd, custom_fwd
from torch.autograd.function import once_differentiable

from fast_sp_gs_amd._C import get_C_function

__all__ = ['sh_encode', 'SH_to_RGB', 'freq_encode', 'FreqEncoder', 'cdist_top']


class _sh_encoder(Function):
    _forward = staticmethod(get_C_function('sh_encode_forward'))
    _backward = staticmethod(get_C_function('sh_encode_backward'))

    @staticmethod
    @custom_fwd(cast_inputs=torch.float32, device_type='cuda')  # float32 under autocast; otherwise the caller's dtype
    def forward(ctx, inputs, degree):
        inputs = inputs.contiguous()
        B, input_dim = inputs.shape
        outputs = torch.empty(B, (degree + 1) ** 2, dtype=inputs.dtype, device=inputs.device)
        _sh_encoder._forward(inputs, outputs, B, input_dim, degree)
        ctx.save_for_backward(inputs)
        ctx.dims = [B, input_dim, degree]
        return outputs

    @staticmethod
    @once_differentiable
    @custom_bwd(device_type='cuda')
    def backward(ctx, grad):
        inputs, = ctx.saved_tensors
        B, input_dim, degree = ctx.dims
        grad_inputs = torch.zeros_like(inputs)
        _sh_encoder._backward(grad.contiguous(), inputs, B, input_dim, degree, grad_inputs)
        return grad_inputs, None


def sh_encode(dirs: Tensor, degree: int) -> Tensor:
    shape = dirs.shape
    return _sh_encoder.apply(dirs.reshape(-1, shape[-1]), degree).reshape(*shape[:-1], -1)


class _SH_to_RGB(Function):
    _forward = staticmethod(get_C_function('SH_to_RGB_forward'))
    _backward = staticmethod(get_C_function('SH_to_RGB_backward'))

    @staticmethod
    def forward(ctx, sh, dirs, campos, degree, clamp):
        ctx._degree, ctx._clamp = degree, clamp
        dirs, sh = dirs.contiguous(), sh.contiguous()
        campos = None if campos is None else campos.contiguous()
        rgb = _SH_to_RGB._forward(dirs, campos, sh, degree, clamp)
        ctx.save_for_backward(sh, dirs, campos, rgb)
        return rgb

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_rgb):
        sh, dirs, campos, rgb = ctx.saved_tensors
        grad_sh = torch.zeros_like(sh) if ctx.needs_input_grad[0] else None
        grad_dirs = torch.zeros_like(dirs) if ctx.needs_input_grad[1] else None
        grad_campos = torch.zeros_like(campos) if campos is not None and ctx.needs_input_grad[2] else None
        _SH_to_RGB._backward(ctx._degree, ctx._clamp, dirs, campos, sh, rgb, grad_rgb.contiguous(), grad_dirs,
                             grad_campos, grad_sh)
        return grad_sh, grad_dirs, grad_campos, None, None


def SH_to_RGB(sh: Tensor, dirs: Tensor, campos: Tensor = None, degree: int = 0, clamp: bool = True) -> Tensor:
    return _SH_to_RGB.apply(sh, dirs, campos, degree, clamp)


class _freq_encoder(Function):
    _forward = staticmethod(get_C_function('freq_encode_forward'))
    _backward = staticmethod(get_C_function('freq_encode_backward'))

    @staticmethod
    @custom_fwd(cast_inputs=torch.float32, device_type='cuda')  # float32 under autocast; otherwise the caller's dtype
    def forward(ctx, inputs, degree, include_input, scale):
        if not inputs.is_cuda:
            inputs = inputs.cuda()
        inputs = inputs.contiguous()
        outputs = _freq_encoder._forward(inputs, degree, include_input, scale)
        ctx._info = [degree, include_input, scale]
        ctx.save_for_backward(outputs)
        return outputs

    @staticmethod
    @once_differentiable
    @custom_bwd(device_type='cuda')
    def backward(ctx, grad):
        outputs, = ctx.saved_tensors
        degree, include_input, scale = ctx._info
        return _freq_encoder._backward(grad.contiguous(), outputs, degree, include_input, scale), None, None, None


freq_encode = _freq_encoder.apply


class FreqEncoder(nn.Module):
    def __init__(self, input_dim=3, degree=4, include_input=True, scale=1.):
        super().__init__()
        self.input_dim = input_dim
        self.degree = degree
        self.output_dim = input_dim * (2 * degree + int(include_input))
        self.include_input = include_input
        self.scale = torch.pi if scale == 'pi' else float(scale)

    def extra_repr(self) -> str:
        return (f"input_dim={self.input_dim}, degree={self.degree}, output_dim={self.output_dim}, "
                f"include_input={self.include_input}")

    def forward(self, inputs, **kwargs):
        return freq_encode(inputs, self.degree, self.include_input, self.scale)


class _ChamferDistanceFunction(Function):
    _forward = staticmethod(get_C_function('cdist_top'))
    _backward = staticmethod(get_C_function('cdist_top_backward'))

    @staticmethod
    def forward(ctx, *inputs):
        if len(inputs) == 2:
            x1, x2 = inputs
            largest = False
        else:
            x1, x2, largest = inputs
        x1, x2 = x1.contiguous(), x2.contiguous()
        distance, index = _ChamferDistanceFunction._forward(x1, x2, largest)
        ctx.save_for_backward(x1, x2, distance, index)
        ctx.mark_non_differentiable(index)
        return distance, index

    @staticmethod
    def backward(ctx, *grad_outputs):
        points1, points2, distance, index = ctx.saved_tensors
        grad_1, grad_2 = _ChamferDistanceFunction._backward(points1, points2, distance, index,
                                                            grad_outputs[0].contiguous())
        return grad_1, grad_2, None


cdist_top = _ChamferDistanceFunction.apply
