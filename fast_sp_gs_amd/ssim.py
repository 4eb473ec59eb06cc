"""SSIM on the fused HIP kernel: the reference's `FusedSSIM` autograd function and `SSIM_Loss` module
(fast_2d_gs/losses/ssim.py:24-47, 70-95). The window is fixed at 11 taps, sigma 1.5, as in the kernel."""
import torch
from torch import Tensor, nn

from fast_sp_gs_amd._C import get_C_function
from fast_sp_gs_amd.autograd import KernelPair

__all__ = ['FusedSSIM', 'ssim', 'SSIM_Loss', 'l1_dssim_loss']


C1, C2 = 0.01 ** 2, 0.03 ** 2  # the usual SSIM stabilisers for images in [0, 1]


def _ssim_launch(fwd, needs, img, target, _window=None):
    if len(needs) > 1 and needs[1]:
        raise RuntimeError('fused SSIM is differentiable in its first image only')
    ssim_map, d_mu, d_var, d_cov = fwd(C1, C2, img, target, bool(needs[0]))
    return ssim_map, (img, target, d_mu, d_var, d_cov), None


def _ssim_grads(bwd, needs, keep, _, g_map):
    img, target, d_mu, d_var, d_cov = keep
    return (bwd(C1, C2, img, target, g_map, d_mu, d_var, d_cov), None, None)[:len(needs)]


_ssim_pair = KernelPair('fusedssim', 'fusedssim_backward', _ssim_launch, _ssim_grads)


class FusedSSIM:
    """The reference's autograd function of this name (losses/ssim.py:24-47) as a call-compatible shim:
    `FusedSSIM.apply(img1, img2, window)` -> SSIM map; the window argument is ignored (fixed 11 taps)."""
    C1, C2 = C1, C2
    apply = staticmethod(_ssim_pair)


def ssim(img1: Tensor, img2: Tensor) -> Tensor:
    """SSIM map of [B,CH,H,W] (or [CH,H,W]) images; differentiable in img1."""
    if img1.ndim == 3:
        return _ssim_pair(img1[None], img2[None])[0]
    return _ssim_pair(img1, img2)


class _L1DssimLoss(torch.autograd.Function):
    """(1 - lambda) * L1 + lambda * (1 - mean SSIM) on the fused kernels: the block sums are taken inside the SSIM
    kernel and the L1 term's sign is added inside its backward, so nothing image-sized is written but the gradient."""

    @staticmethod
    def forward(ctx, img, target, lambda_dssim):
        img, target = img.contiguous(), target.contiguous()
        loss, d1, d2, d3 = get_C_function('image_loss_forward')(C1, C2, lambda_dssim, img, target,
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

    @staticmethod
    def _as_batch(img: Tensor) -> Tensor:
        """[CH,H,W] / [H,W,3] / [B,H,W,3] / [B,CH,H,W] -> [B,CH,H,W] (a trailing dimension of 3 is taken as channels)."""
        img = img if img.ndim == 4 else img[None]
        return img.movedim(-1, 1) if img.shape[-1] == 3 else img

    def forward(self, img1: Tensor, img2: Tensor, mask: Tensor = None) -> Tensor:
        per_image = ssim(self._as_batch(img1), self._as_batch(img2)).flatten(1).mean(dim=1)
        return 1.0 - (per_image.mean() if self.reduction == 'mean' else per_image)
