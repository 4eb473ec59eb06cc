"""One training step of the dynamic superpoint scene, assembled from the library's operators in the order the reference
runs them (fast_2d_gs/network.py:576-647 `sp_stage` + `forward`, :700-730 `render`, gaussian_splatting.py:295-321 loss,
train.py:343-374 loop): deformation network on the control points -> K-NN + neighbour weights + warp of the Gaussians ->
deformed parameters -> 2D-Gaussian render -> (1 - lambda) L1 + lambda (1 - SSIM) -> backward -> masked Adam on the
Gaussians, Adam on the network and the control points.

`DynamicStep` owns the state (parameters, the two optimisers); `forward_loss` is the differentiable part alone so that
tests can compare its gradients with other formulations.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from fast_sp_gs_amd.deform import DeformNetwork, deform_apply, superpoint_deform
from fast_sp_gs_amd.renderer import GS_2D_render
from fast_sp_gs_amd.sparse_gaussian_adam import SparseGaussianAdam
from fast_sp_gs_amd.ssim import l1_dssim_loss

__all__ = ['DynamicStep']

PARAM_NAMES = ('means3D', 'scales', 'rotations', 'opacities', 'shs')


class DynamicStep:
    def __init__(self, scene, cam, control_points: Tensor, target: Tensor, K: int = 4, temperature: float = 0.01,
                 local_frame: bool = True, warp_method: str = 'LBS', LBS_method: str = 'dist', lr: float = 1.6e-4,
                 net_lr: float = 1e-7, lambda_dssim: float = 0.2, background: Optional[Tensor] = None,
                 net: Optional[DeformNetwork] = None):
        dev = scene.means3D.device
        self.cam, self.target, self.K, self.temperature = cam, target, K, temperature
        self.warp_method, self.LBS_method, self.lambda_dssim = warp_method, LBS_method, lambda_dssim
        self.background = torch.ones(3, device=dev) if background is None else background
        self.ctrl = control_points.detach().clone().requires_grad_(True)
        self.net = (DeformNetwork(local_frame=local_frame) if net is None else net).to(dev)
        self.params = [getattr(scene, k).detach().clone().requires_grad_(True) for k in PARAM_NAMES]
        self.opt = SparseGaussianAdam([{'params': [p], 'name': k} for p, k in zip(self.params, PARAM_NAMES)], lr=lr,
                                      eps=1e-15)
        self.net_opt = torch.optim.Adam(list(self.net.parameters()) + [self.ctrl], lr=net_lr, fused=True)
        self.sh_degree = scene.sh_degree
        # the reference's training render passes `accum_max_count` on every step (network.py:706): per Gaussian, the
        # number of (pixel, blended entry) events at which it was the pixel's strongest contributor so far
        self.accum_max_count = torch.zeros(self.params[0].shape[0], dtype=torch.int32, device=dev)

    def forward_loss(self, t: Tensor):
        """-> (loss, render outputs). Differentiable in the Gaussians' parameters, the control points and the network."""
        means3D, scales, rotations, opacities, shs = self.params
        c_xyz, c_rot, c_scale, c_local = self.net(self.ctrl.detach(), t)
        d_xyz, d_rot, d_scale, _, _ = superpoint_deform(
            means3D.detach(), self.ctrl, c_xyz, c_rot, c_scale[:, :scales.shape[1]], sp_rot=c_local, K=self.K,
            temperature=self.temperature, warp_method=self.warp_method, LBS_method=self.LBS_method)
        xyz, sc, rot = deform_apply(means3D, d_xyz, scales, d_scale, rotations, d_rot)
        cam = self.cam
        out = GS_2D_render(xyz, sc, rot, opacities, (cam.W, cam.H), cam.Tw2v, cam.Tv2c, campos=cam.campos,
                           near=cam.near, far=cam.far, sh_degree=self.sh_degree, sh_features=shs,
                           background=self.background, accum_max_count=self.accum_max_count)
        return l1_dssim_loss(out['images'], self.target, self.lambda_dssim), out

    def step(self, t: Tensor):
        """One full iteration; returns (loss, visibility mask) as device tensors (nothing is copied to the host)."""
        loss, out = self.forward_loss(t)
        loss.backward()
        visible = out['radii'] > 0
        self.opt.set_before_step(visible, self.params[0].shape[0])
        self.opt.step()
        self.opt.zero_grad(set_to_none=True)
        self.net_opt.step()
        self.net_opt.zero_grad(set_to_none=True)
        return loss.detach(), visible
