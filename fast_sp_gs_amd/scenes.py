"""Seeded synthetic scenes and pinhole cameras for the benchmark configurations (host side, torch CPU generator).

Camera conventions follow the reference's OpenCV helpers, restated here because the benchmark must not depend on the
reference tree: `look_at` (utils/ops_3d/coord_trans_opencv.py:87-119), `perspective2` (:247-306, z in [0,1],
near/far = 0.1/1000 as datasets/base.py:214 passes), focal = W / (2 tan(FoV/2)) (coord_trans_common.py:87-89),
`camera_intrinsics` (coord_trans_opencv.py:131-200).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, Optional

import torch
from torch import Tensor


@dataclass
class Camera:
    W: int
    H: int
    Tw2v: Tensor  # [4,4] world -> view
    Tv2c: Tensor  # [4,4] view -> clip
    Tv2s: Tensor  # [3,3] view -> screen (intrinsics)
    campos: Tensor  # [3]
    near: float = 0.2
    far: float = 100.0

    def to(self, device):
        return Camera(self.W, self.H, self.Tw2v.to(device).contiguous(), self.Tv2c.to(device).contiguous(),
                      self.Tv2s.to(device).contiguous(), self.campos.to(device).contiguous(), self.near, self.far)


def _normalize(v: Tensor) -> Tensor:
    return v / v.norm().clamp_min(1e-12)


def look_at(eye: Tensor, at: Optional[Tensor] = None) -> Tensor:
    """World-to-view matrix of an OpenCV camera (x right, y down, z forward) at `eye` looking at `at`."""
    eye = eye.to(torch.float32)
    at = torch.zeros(3) if at is None else at.to(torch.float32)
    fwd = -_normalize(eye - at)
    y_axis = torch.tensor([0., -1., 0.])
    parallel = torch.linalg.cross(fwd, y_axis).norm() < 1e-6
    up = torch.tensor([0., 0., -1.]) if parallel else torch.tensor([0., 1., 0.])
    right = -_normalize(torch.linalg.cross(up, fwd))
    upv = torch.linalg.cross(fwd, right)
    R = torch.eye(4)
    T = torch.eye(4)
    R[0, :3], R[1, :3], R[2, :3] = right, upv, fwd
    T[:3, 3] = -eye
    return (R @ T).contiguous()


def pinhole(W: int, H: int, fov_deg: float, eye: Tensor, at: Optional[Tensor] = None, near_far=(0.1, 1000.0),
            near: float = 0.2, far: float = 100.0) -> Camera:
    f = W / (2.0 * math.tan(math.radians(fov_deg) * 0.5))
    n, fr = near_far
    Tv2c = torch.zeros(4, 4)
    Tv2c[0, 0] = 2.0 * f / W
    Tv2c[1, 1] = 2.0 * f / H
    Tv2c[0, 2] = (2.0 * (W / 2) - W) / W
    Tv2c[1, 2] = (2.0 * (H / 2) - H) / H
    Tv2c[2, 2] = fr / (fr - n)
    Tv2c[2, 3] = -(fr * n) / (fr - n)
    Tv2c[3, 2] = 1.0
    Tv2s = torch.tensor([[f, 0., W / 2], [0., f, H / 2], [0., 0., 1.]])
    Tw2v = look_at(eye, at)
    campos = torch.linalg.inv(Tw2v)[:3, 3].contiguous()
    return Camera(W, H, Tw2v, Tv2c, Tv2s, campos, near, far)


@dataclass
class SurfelScene:
    means3D: Tensor  # [P,3]
    scales: Tensor  # [P,2]
    rotations: Tensor  # [P,4] unit quaternions (x,y,z,w)
    opacities: Tensor  # [P,1]
    shs: Tensor  # [P,16,3]
    sh_degree: int = 3
    extra: Dict[str, Tensor] = field(default_factory=dict)

    @property
    def P(self) -> int:
        return self.means3D.shape[0]

    def to(self, device):
        return SurfelScene(*(t.to(device).contiguous() for t in
                             (self.means3D, self.scales, self.rotations, self.opacities, self.shs)),
                           self.sh_degree, {k: v.to(device) for k, v in self.extra.items()})


def _surfels(g: torch.Generator, P: int, centres: str, log_scale_mu: float, log_scale_sigma: float,
             opacity_mu: float, opacity_sigma: float, centre_scale: float = 1.0) -> SurfelScene:
    """Draw order: centres, log-scales, quaternions, opacity logits, SH DC, SH rest."""
    if centres == 'cube':  # U[-1,1]^3
        xyz = torch.rand(P, 3, generator=g) * 2 - 1
    elif centres == 'ball':  # uniform in the unit ball: direction = normalised N(0,1)^3, radius = U^(1/3)
        d = torch.randn(P, 3, generator=g)
        r = torch.rand(P, 1, generator=g).pow(1.0 / 3.0)
        xyz = d / d.norm(dim=-1, keepdim=True).clamp_min(1e-12) * r
    elif centres == 'normal':  # N(0, centre_scale^2) per axis
        xyz = torch.randn(P, 3, generator=g) * centre_scale
    else:
        raise ValueError(centres)
    scales = torch.exp(torch.randn(P, 2, generator=g) * log_scale_sigma + log_scale_mu)
    q = torch.randn(P, 4, generator=g)
    q = q / q.norm(dim=-1, keepdim=True).clamp_min(1e-12)
    opacity = torch.sigmoid(torch.randn(P, 1, generator=g) * opacity_sigma + opacity_mu)
    dc = torch.randn(P, 1, 3, generator=g) * 0.3
    rest = torch.randn(P, 15, 3, generator=g) * 0.05
    return SurfelScene(xyz.contiguous(), scales.contiguous(), q.contiguous(), opacity.contiguous(),
                       torch.cat([dc, rest], dim=1).contiguous(), 3)


def config0(P: int = 10_000, size: int = 256, seed: int = 0):
    """10k surfels in [-1,1]^3, 256x256, FoV 50 deg, radius 4, black background; dL/dimage ~ N(0,1)."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    scene = _surfels(g, P, 'cube', -4.6, 0.5, 0.0, 1.0)
    cam = pinhole(size, size, 50.0, torch.tensor([0., 0., 4.]))
    scene.extra['grad_image'] = torch.randn(3, size, size, generator=g)
    scene.extra['grad_extras'] = torch.cat([torch.randn(5, size, size, generator=g), torch.zeros(4, size, size)])
    scene.extra['grad_opacity'] = torch.zeros(size, size)
    return scene, cam


def config2(P: int = 300_000, size: int = 800, seed: int = 0):
    """300k surfels in the unit ball, 800x800, FoV 40 deg, radius 4 (white background is composited by the caller)."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    scene = _surfels(g, P, 'ball', -5.0, 0.6, 0.0, 1.5)
    cam = pinhole(size, size, 40.0, torch.tensor([0., 0., 4.]))
    scene.extra['grad_image'] = torch.randn(3, size, size, generator=g)
    scene.extra['grad_extras'] = torch.cat([torch.randn(5, size, size, generator=g), torch.zeros(4, size, size)])
    scene.extra['grad_opacity'] = torch.zeros(size, size)
    return scene, cam


def config4(P: int = 3_000_000, W: int = 1352, H: int = 1014, seed: int = 0, n_views: int = 4):
    """3M surfels ~ N(0, 2^2), 4 cameras on a 30 deg arc at radius 6, FoV 60 deg."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    scene = _surfels(g, P, 'normal', -5.5, 0.8, -0.5, 1.5, centre_scale=2.0)
    cams = []
    for i in range(n_views):
        th = math.radians(-15.0 + 30.0 * i / max(n_views - 1, 1))
        cams.append(pinhole(W, H, 60.0, torch.tensor([6.0 * math.sin(th), 0.0, 6.0 * math.cos(th)])))
    scene.extra['grad_image'] = torch.randn(3, H, W, generator=g)
    return scene, cams


def config1(seed: int = 1, n_dirs: int = 1_000_000, n_points: int = 200_000, n_ctrl: int = 512):
    """Stand-alone ops: unit directions + SH coefficients, K-NN clouds, SE(3) control transforms."""
    g = torch.Generator(device='cpu').manual_seed(seed)
    d = torch.randn(n_dirs, 3, generator=g)
    dirs = (d / d.norm(dim=-1, keepdim=True).clamp_min(1e-12)).contiguous()
    dc = torch.randn(n_dirs, 1, 3, generator=g) * 0.3
    rest = torch.randn(n_dirs, 15, 3, generator=g) * 0.05
    shs = torch.cat([dc, rest], dim=1).contiguous()
    points = (torch.rand(n_points, 3, generator=g) * 2 - 1).contiguous()
    ctrl = (torch.rand(n_ctrl, 3, generator=g) * 2 - 1).contiguous()
    axis_angle = torch.randn(n_ctrl, 3, generator=g) * 0.1
    trans = (torch.randn(n_ctrl, 3, generator=g) * 0.05).contiguous()
    ang = axis_angle.norm(dim=-1, keepdim=True).clamp_min(1e-12)
    quat = torch.cat([axis_angle / ang * torch.sin(ang / 2), torch.cos(ang / 2)], dim=-1)
    # the model stores rotations as residuals r with q = normalize(r + (0,0,0,1)) (network.py:547)
    sp_r = (quat - torch.tensor([0., 0., 0., 1.])).contiguous()
    sp_s = (torch.randn(n_ctrl, 2, generator=g) * 0.01).contiguous()
    return dict(dirs=dirs, shs=shs, points=points, ctrl=ctrl, sp_t=trans, sp_r=sp_r, sp_s=sp_s)
