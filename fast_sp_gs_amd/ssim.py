"""SSIM on the fused HIP kernel: the reference's `FusedSSIM` autograd function and `SSIM_Loss` module
(fast_2d_gs/losses/ssim.py:24-47, 70-95). The window is fixed at 11 taps, sigma 1.5, as in the kernel."""
import torch
from torch import Tensor, nn

from fast_sp_gs_amd._C import get_C_function

__all__ = ['FusedSSIM', 'ssim', 'SSIM_Loss']


class FusedSSIM(torch.autograd.Function):
    _forward_func = get_C_function('fusedssim')
    _backward_func = get_C_function('fusedssim_backward')
    C1 = 0.01 ** 2
    C2 = 0.03 ** 2

    @staticmethod
    def forward(ctx, img1, img2, window=None):
        ssim_map, d1, d2, d3 = FusedSSIM._forward_func(FusedSSIM.C1, FusedSSIM.C2, img1, img2, ctx.needs_input_grad[0])
        assert not ctx.needs_input_grad[1]
        ctx.save_for_backward(img1, img2, d1, d2, d3)
        return ssim_map

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outputs):
        img1, img2, d1, d2, d3 = ctx.saved_tensors
        grad_img1 = FusedSSIM._backward_func(FusedSSIM.C1, FusedSSIM.C2, img1, img2, grad_outputs[0].contiguous(), d1,
                                             d2, d3)
        return grad_img1, None, None


def ssim(img1: Tensor, img2: Tensor) -> Tensor:
    """SSIM map of [B,CH,H,W] (or [CH,H,W]) images; differentiable in img1."""
    if img1.ndim == 3:
        return FusedSSIM.apply(img1[None], img2[None], None)[0]
    return FusedSSIM.apply(img1, img2, None)


class SSIM_Loss(nn.Module):
    """1 - mean SSIM (reduction 'mean') or the per-image means (reduction 'none')."""

    def __init__(self, window_size=11, reduction='mean', **kwargs):
        super().__init__()
        if window_size != 11:
            raise ValueError('the fused SSIM kernel has a fixed 11-tap window')
        self.reduction = reduction

    def forward(self, img1: Tensor, img2: Tensor, mask: Tensor = None) -> Tensor:
        if img1.ndim == 3:
            img1 = img1.unsqueeze(0)
        if img2.ndim == 3:
            img2 = img2.unsqueeze(0)
        if img1.shape[-1] == 3:
            img1 = torch.permute(img1, (0, 3, 1, 2))  # -> [B, C, H, W]
        if img2.shape[-1] == 3:
            img2 = torch.permute(img2, (0, 3, 1, 2))
        m = ssim(img1, img2)
        if self.reduction == 'mean':
            return 1.0 - m.mean()
        return 1.0 - m.mean(dim=(1, 2, 3))
