"""GPU parity of the fused SSIM forward / backward with the CPU oracle (same float weights, same tap order), through the
operator boundary and through the autograd wrapper. SSIM maps agree to float rounding (FMA contraction on the GPU);
the partial-derivative maps and the image gradient are compared relative to their largest magnitude, since they
contain quotients by (A B^2) that reach 1e3 where both images are dark and flat."""
import numpy as np
import pytest
import torch

from util import abs_err, npy, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(2, 3, 45, 70), (1, 3, 800, 800), (1, 1, 7, 5), (3, 2, 32, 64)])
def test_fusedssim_parity(shape, device, oracle_mod):
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    B, CH, H, W = shape
    g = torch.Generator().manual_seed(1)
    img1, img2 = torch.rand(*shape, generator=g), torch.rand(*shape, generator=g)
    img2[..., : W // 2] = img1[..., : W // 2] * 0.9  # correlated half: SSIM near 1 there
    gmap = torch.randn(*shape, generator=g)
    print(f"[ssim] {shape}", flush=True)
    m, d1, d2, d3 = get_C_function('fusedssim')(0.01 ** 2, 0.03 ** 2, img1.to(device), img2.to(device), True)
    grad = get_C_function('fusedssim_backward')(0.01 ** 2, 0.03 ** 2, img1.to(device), img2.to(device),
                                                 gmap.to(device), d1, d2, d3)
    m_eval, e1, e2, e3 = get_C_function('fusedssim')(0.01 ** 2, 0.03 ** 2, img1.to(device), img2.to(device), False)
    torch.cuda.synchronize()
    a, b = npy(img1), npy(img2)
    rm, r1, r2, r3 = (np.zeros_like(a) for _ in range(4))
    assert O.call("fusedssim_forward_f32", B, CH, H, W, 0.01 ** 2, 0.03 ** 2, a, b, rm, r1, r2, r3) == 0
    rg = np.zeros_like(a)
    assert O.call("fusedssim_backward_f32", B, CH, H, W, a, b, npy(gmap), r1, r2, r3, rg) == 0
    assert abs_err(npy(m), rm) < 5e-6
    assert torch.equal(m, m_eval) and e1.numel() == 0 and e2.numel() == 0 and e3.numel() == 0
    for x, r, name in ((d1, r1, 'dm_dmu1'), (d2, r2, 'dm_dsigma1_sq'), (d3, r3, 'dm_dsigma12')):
        assert rel_err(npy(x), r) < 1e-4, name
    # the backward on the oracle's partials and on the GPU's own must both match
    assert rel_err(npy(grad), rg) < 1e-4
    grad2 = get_C_function('fusedssim_backward')(0.01 ** 2, 0.03 ** 2, img1.to(device), img2.to(device),
                                                  gmap.to(device), torch.from_numpy(r1).to(device),
                                                  torch.from_numpy(r2).to(device), torch.from_numpy(r3).to(device))
    assert rel_err(npy(grad2), rg) < 1e-5


def test_ssim_autograd_and_loss(device):
    from fast_sp_gs_amd.ssim import SSIM_Loss, ssim
    g = torch.Generator().manual_seed(2)
    img1 = torch.rand(3, 96, 80, generator=g).to(device).requires_grad_(True)
    img2 = torch.rand(3, 96, 80, generator=g).to(device)
    loss = SSIM_Loss()(img1, img2)
    loss.backward()
    assert img1.grad is not None and img1.grad.shape == img1.shape and float(img1.grad.abs().sum()) > 0
    assert abs(float(loss) - (1.0 - float(ssim(img1.detach(), img2).mean()))) < 1e-6
    assert float(ssim(img2, img2).min()) > 1.0 - 1e-5  # identical images
    # finite-difference check of the gradient along a random direction (float32: loose)
    d = torch.randn(3, 96, 80, generator=g).to(device)
    eps = 1e-2
    f = lambda x: float(SSIM_Loss()(x, img2).double())
    fd = (f(img1.detach() + eps * d) - f(img1.detach() - eps * d)) / (2 * eps)
    an = float((img1.grad * d).sum())
    assert abs(fd - an) < 2e-2 * max(abs(an), 1e-6) + 1e-6


def test_ssim_loss_channel_last_and_sliced_inputs(device):
    """The reference's loss call hands SSIM_Loss [H,W,3] renders and `targets['images'][..., :3]` of an RGBA batch
    (gaussian_splatting.py:295-297, 317-321): permuted / sliced views, not contiguous. The operator accepts any strides
    (structural_similarity.cu:341-357 checks the device only), forward and backward."""
    from fast_sp_gs_amd.ssim import SSIM_Loss
    g = torch.Generator().manual_seed(4)
    hwc = torch.rand(2, 40, 56, 3, generator=g).to(device).requires_grad_(True)
    rgba = torch.rand(2, 40, 56, 4, generator=g).to(device)
    target = rgba[..., :3]
    assert not target.is_contiguous()
    loss = SSIM_Loss()(hwc, target)
    loss.backward()
    chw = hwc.detach().permute(0, 3, 1, 2).contiguous().requires_grad_(True)
    ref = SSIM_Loss()(chw, target.permute(0, 3, 1, 2).contiguous())
    ref.backward()
    assert float(loss) == float(ref)
    assert hwc.grad.shape == hwc.shape and torch.equal(hwc.grad.permute(0, 3, 1, 2), chw.grad)
    # one [H,W,3] image
    one = SSIM_Loss()(hwc.detach()[0], target[0])
    assert abs(float(one) - float(SSIM_Loss()(chw.detach()[:1], target[:1].permute(0, 3, 1, 2).contiguous()))) < 1e-7


@pytest.mark.parametrize("shape,lam", [((1, 3, 800, 800), 0.2), ((2, 3, 45, 70), 0.35), ((1, 1, 7, 5), 1.0),
                                       ((3, 2, 32, 64), 0.0)])
def test_fused_image_loss(shape, lam, device, oracle_mod):
    """(1 - lambda) L1 + lambda (1 - mean SSIM) in the fused kernels against the CPU oracle's SSIM map and partials with
    the L1 term, the means and the chain rule taken in float64 numpy, and against the composition of the separate
    operators through torch autograd."""
    from fast_sp_gs_amd.ssim import l1_dssim_loss, ssim
    O = oracle_mod
    B, CH, H, W = shape
    g = torch.Generator().manual_seed(3)
    img1, img2 = torch.rand(*shape, generator=g), torch.rand(*shape, generator=g)
    img2[..., : W // 2] = img1[..., : W // 2] * 0.9
    img2[..., 0, :] = img1[..., 0, :]  # a row of equal pixels: the L1 term's gradient is exactly zero there
    x = img1.to(device).requires_grad_(True)
    print(f"[image loss] {shape} lambda={lam}", flush=True)
    loss, terms = l1_dssim_loss(x, img2.to(device), lam, return_terms=True)
    (3.0 * loss).backward()
    torch.cuda.synchronize()
    a, b = npy(img1), npy(img2)
    rm, r1, r2, r3 = (np.zeros_like(a) for _ in range(4))
    assert O.call("fusedssim_forward_f32", B, CH, H, W, 0.01 ** 2, 0.03 ** 2, a, b, rm, r1, r2, r3) == 0
    n = a.size
    l1, sm = np.abs(a.astype(np.float64) - b).mean(), rm.astype(np.float64).mean()
    want = (1 - lam) * l1 + lam * (1 - sm)
    assert abs(float(loss) - want) < 2e-6 * max(1.0, abs(want))
    assert abs(float(terms[0]) - l1) < 2e-6 and abs(float(terms[1]) - sm) < 2e-6
    rg = np.zeros_like(a)
    gmap = np.full_like(a, -3.0 * lam / n)
    assert O.call("fusedssim_backward_f32", B, CH, H, W, a, b, gmap, r1, r2, r3, rg) == 0
    rg = rg.astype(np.float64) + 3.0 * (1 - lam) / n * np.sign(a.astype(np.float64) - b)
    assert rel_err(npy(x.grad), rg.astype(np.float32)) < 1e-4
    # the separate operators through autograd
    y = img1.to(device).requires_grad_(True)
    t = img2.to(device)
    ref = (1 - lam) * (y - t).abs().mean() + lam * (1.0 - ssim(y, t).mean())
    (3.0 * ref).backward()
    assert abs(float(loss) - float(ref)) < 2e-6 * max(1.0, abs(float(ref)))
    assert rel_err(npy(x.grad), npy(y.grad)) < 1e-5
    # no gradient wanted: the same number
    assert float(l1_dssim_loss(img1.to(device), t, lam)) == float(loss)
