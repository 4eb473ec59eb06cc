"""SSIM on the fused HIP kernel: the reference's `FusedSSIM` autograd function and `SSIM_Loss` module
(fast_2d_gs/losses/ssim.py:24-47, 70-95). The window is fixed at 11 taps, sigma 1.5, as in the kernel."""
import torch
from torch import Tensor, nn

from fast_sp_gs_amd._C import get_C_function

__all__ = ['FusedSSIM', 'ssim', 'SSIM_Loss', 'l1_dssim_loss']


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


class _L1DssimLoss(torch.autograd.Function):
    """(1 - lambda) * L1 + lambda * (1 - mean SSIM) on the fused kernels: the block sums are taken inside the SSIM
    kernel and the L1 term's sign is added inside its backward, so nothing image-sized is written but the gradient."""

    @staticmethod
    def forward(ctx, img, target, lambda_dssim):
        img, target = img.contiguous(), target.contiguous()
        loss, d1, d2, d3 = get_C_function('image_loss_forward')(FusedSSIM.C1, FusedSSIM.C2, lambda_dssim, img, target,
                                                                ctx.needs_input_grad[0])
        assert not ctx.needs_input_grad[1]
        ctx.lambda_dssim = lambda_dssim
        if ctx.needs_input_grad[0]:
            ctx.save_for_backward(img, target, d1, d2, d3)
        terms = loss[1:]
        ctx.mark_non_differentiable(terms)
        return loss[0], terms

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_loss, _):
        img, target, d1, d2, d3 = ctx.saved_tensors
        grad = get_C_function('image_loss_backward')(ctx.lambda_dssim, img, target, grad_loss.reshape(1).contiguous(),
                                                     d1, d2, d3)
        return grad, None, None


def l1_dssim_loss(img: Tensor, target: Tensor, lambda_dssim: float = 0.2, return_terms: bool = False):
    """The photometric loss of a training step, (1 - lambda) * mean|img - target| + lambda * (1 - mean SSIM), as one
    scalar (reference: the 'rgb' and 'ssim' terms summed at fast_2d_gs/gaussian_splatting.py:321 with their weights).
    [CH,H,W] or [B,CH,H,W]; differentiable in img. With `return_terms` also (L1 mean, SSIM mean), detached."""
    if img.ndim == 3:
        img, target = img[None], target[None]
    loss, terms = _L1DssimLoss.apply(img, target, float(lambda_dssim))
    return (loss, terms.detach()) if return_terms else loss


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
