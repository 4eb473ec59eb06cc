"""Host side of the 3D-Gaussian (EWA) render path on the HIP operators: the autograd wiring and entry points of the
reference's fast_2d_gs/renderer/gaussian_render.py (`_preprocess` :495-566, `preprocess` :569-, `GS_prepare` :742-772,
`_GS_render` :775-800, `_GS_render_fast` :803-837, `GS_render` :840-, `RasterizeGaussians` :226-274, `render` :277-359),
with covariances from scales + rotations or pre-computed (3D or 2D), gradients to the view matrix and the camera
position, and `_render_extra` / `render_extra` :925-962 for further feature tables of any width."""
from __future__ import annotations

from typing import NamedTuple, Optional, Tuple

import torch
from torch import Tensor

from fast_sp_gs_amd._C import get_C_function
from fast_sp_gs_amd.renderer.gs_2d_render import GS_prepare

_cull_masks = get_C_function('gs_cull_masks')

__all__ = ['RasterizeBuffer3D', 'preprocess', 'GS_render', 'GS_render_fast', 'RasterizeGaussians', 'render',
           'compute_cov3D', 'compute_cov2D', 'topk_weights', 'render_extra']


class RasterizeBuffer3D(NamedTuple):
    """gaussian_render.py:37-51"""
    W: int
    H: int
    P: int
    R: int
    tile_ranges: Tensor
    point_list: Tensor
    n_contribed: Tensor
    conic_opacity: Tensor
    means2D: Tensor
    opacity: Tensor


def topk_weights(topk: int, buffer: RasterizeBuffer3D) -> Tuple[Tensor, Tensor]:
    """Per-pixel top-k Gaussian indices and blend weights of a rendered view (reference: gaussian_render.py:362-367)."""
    return get_C_function('gaussian_topk_weights')(topk, buffer.W, buffer.H, buffer.P, buffer.R, buffer.means2D,
                                                   buffer.conic_opacity, buffer.tile_ranges, buffer.point_list)


class _render_extra(torch.autograd.Function):
    """renderer/gaussian_render.py:925-949 of the reference."""

    @staticmethod
    def forward(ctx, W, H, extras, means2D, conic_opacity, ranges, point_list, n_contrib, out_opacity):
        extras = extras.contiguous()
        out_pixels = get_C_function('gaussian_rasterize_extra_forward')(W, H, extras, means2D, conic_opacity, ranges,
                                                                        point_list, n_contrib)
        ctx.save_for_backward(out_opacity, extras, means2D, conic_opacity, ranges, point_list, n_contrib)
        return out_pixels

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out):
        out_opacity, extras, means2D, conic_opacity, ranges, point_list, n_contrib = ctx.saved_tensors
        H, W = out_opacity.shape
        grad_extra = torch.zeros_like(extras) if ctx.needs_input_grad[2] else None
        grad_means2D = torch.zeros_like(means2D) if ctx.needs_input_grad[3] else None
        grad_conic = torch.zeros_like(conic_opacity) if ctx.needs_input_grad[4] else None
        get_C_function('gaussian_rasterize_extra_backward')(
            W, H, extras, out_opacity, grad_out, means2D, conic_opacity, ranges, point_list, n_contrib, grad_extra,
            grad_means2D, grad_conic)
        return None, None, grad_extra, grad_means2D, grad_conic, None, None, None, None


def render_extra(buffer: RasterizeBuffer3D, *args: Tensor, detach=False):
    """Blends further per-Gaussian tables [P,E] with a rendered view's weights -> [H,W,E] each (reference:
    gaussian_render.py:952-962); `detach` keeps the gradient away from the geometry."""
    means2D, conic_opacity = buffer.means2D, buffer.conic_opacity
    if detach:
        means2D, conic_opacity = means2D.detach(), conic_opacity.detach()
    outputs = [_render_extra.apply(buffer.W, buffer.H, x, means2D, conic_opacity, buffer.tile_ranges, buffer.point_list,
                                   buffer.n_contribed, buffer.opacity) for x in args]
    return outputs[0] if len(args) == 1 else outputs


class _compute_cov3D(torch.autograd.Function):
    """renderer/gaussian_render.py:370-387 of the reference."""

    @staticmethod
    def forward(ctx, scaling, rotation):
        scaling, rotation = scaling.contiguous(), rotation.contiguous()
        ctx.save_for_backward(rotation, scaling)
        return get_C_function('gs_compute_cov3D_forward')(rotation, scaling)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_cov3D):
        rotation, scaling = ctx.saved_tensors
        grad_rotation, grad_scaling = get_C_function('gs_compute_cov3D_backward')(rotation, scaling, grad_cov3D)
        return grad_scaling, grad_rotation


def compute_cov3D(scaling: Tensor, rotation: Tensor) -> Tensor:
    """Upper triangle [N,6] of R(q) diag(s^2) R(q)^T (reference: renderer/gaussian_render.py:420-424)."""
    return _compute_cov3D.apply(scaling, rotation)


class _compute_cov2D(torch.autograd.Function):
    """renderer/gaussian_render.py:427-447 of the reference."""

    @staticmethod
    def forward(ctx, means, cov3D, Tw2v, fx, fy, tx, ty):
        means, cov3D, Tw2v = means.contiguous(), cov3D.contiguous(), Tw2v.contiguous()
        ctx.focal_fov = (fx, fy, tx, ty)
        ctx.save_for_backward(cov3D, means, Tw2v)
        return get_C_function('gs_compute_cov2D_forward')(cov3D, means, Tw2v, fx, fy, tx, ty)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_cov2D):
        cov3D, means, Tw2v = ctx.saved_tensors
        grad_Tw2v = torch.zeros_like(Tw2v) if ctx.needs_input_grad[2] else None
        grad_cov3D, grad_mean = get_C_function('gs_compute_cov2D_backward')(cov3D, means, Tw2v, *ctx.focal_fov,
                                                                           grad_cov2D, grad_Tw2v)
        return grad_mean, grad_cov3D, grad_Tw2v, None, None, None, None


def compute_cov2D(means: Tensor, cov3D: Tensor, Tw2v: Tensor, focal_x: float, focal_y: float, tan_fovx: float,
                  tan_fovy: float) -> Tensor:
    """(a, b, c) [N,3] of J W cov3D W^T J^T + 0.3 I (reference: renderer/gaussian_render.py:450-493)."""
    return _compute_cov2D.apply(means, cov3D, Tw2v, focal_x, focal_y, tan_fovx, tan_fovy)


class _preprocess(torch.autograd.Function):
    _forward = get_C_function('gs_preprocess_forward')
    _backward = get_C_function('gs_preprocess_backward')

    @staticmethod
    def forward(ctx, means3D, scales, rotations, opacities, sh_or_colors, sh_rest, Tw2v, Tv2c, campos, tanFoV, W, H,
                sh_degree, is_opengl, cov3D, cov2D, means2D, culling):
        tan = (float(tanFoV[0]), float(tanFoV[1]))
        ctx._args = (W, H, sh_degree, is_opengl, tan, cov3D is not None)
        c = lambda t: None if t is None else t.contiguous()
        means2D, depths, colors, radii, tiles_touched, cov3D, conic_opacity = _preprocess._forward(
            W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, sh_or_colors, sh_rest, Tw2v, Tv2c,
            campos, tan, c(cov3D), c(cov2D), means2D, culling)
        ctx.save_for_backward(means3D, scales, rotations, opacities, sh_or_colors, sh_rest, Tw2v, Tv2c, campos, cov3D,
                              c(cov2D), radii, colors)
        ctx.mark_non_differentiable(radii, tiles_touched)
        return means2D, depths, colors, radii, tiles_touched, conic_opacity

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, g_means2D, g_depths, g_colors, _g_radii, _g_tiles, g_conic):
        (means3D, scales, rotations, opacities, sh_or_colors, sh_rest, Tw2v, Tv2c, campos, cov3D, cov2D, radii,
         colors) = ctx.saved_tensors
        W, H, sh_degree, is_opengl, tan, has_cov3D = ctx._args
        P = means3D.shape[0]
        zeros = lambda *shape: torch.zeros(shape, dtype=torch.float32, device=means3D.device)
        g_means2D = zeros(P, 2) if g_means2D is None else g_means2D.contiguous().clone()
        g_conic = zeros(P, 4) if g_conic is None else g_conic.contiguous()
        g_colors = zeros(P, 3) if g_colors is None else g_colors.contiguous()
        # every row of these is assigned by the kernel
        grad_means3D, grad_opacities = torch.empty_like(means3D), torch.empty_like(opacities)
        grad_scales = grad_rotations = grad_cov = None
        # which covariance was given decides where its gradient goes (gaussian_render.py:532-541 of the reference)
        if cov2D is not None:
            grad_cov = torch.empty_like(cov2D) if ctx.needs_input_grad[15] else None
        elif has_cov3D:
            grad_cov = torch.empty_like(cov3D) if ctx.needs_input_grad[14] else None
        else:
            grad_scales = torch.empty_like(scales) if ctx.needs_input_grad[1] else None
            grad_rotations = torch.empty_like(rotations) if ctx.needs_input_grad[2] else None
        grad_shs = torch.empty_like(sh_or_colors) if sh_degree >= 0 and ctx.needs_input_grad[4] else None
        grad_sh_rest = torch.empty_like(sh_rest) if (sh_degree >= 0 and sh_rest is not None and
                                                     ctx.needs_input_grad[5]) else None
        grad_Tw2v = torch.zeros_like(Tw2v) if ctx.needs_input_grad[6] else None  # these two are accumulated into
        grad_campos = torch.zeros_like(campos) if ctx.needs_input_grad[8] else None
        _preprocess._backward(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, sh_or_colors, sh_rest,
                              Tw2v, Tv2c, campos, tan, cov3D, cov2D, radii, colors, g_means2D, None, g_colors, g_conic,
                              grad_means3D, grad_scales, grad_rotations, grad_opacities, grad_shs, grad_sh_rest,
                              grad_cov, grad_Tw2v, grad_campos)
        grad_inputs = [grad_means3D, grad_scales, grad_rotations, grad_opacities, grad_shs, grad_sh_rest,
                       grad_Tw2v, None, grad_campos] + [None] * 9
        if cov2D is not None:
            grad_inputs[15] = grad_cov
        elif has_cov3D:
            grad_inputs[14] = grad_cov
        if sh_degree < 0:
            grad_inputs[4] = g_colors if ctx.needs_input_grad[4] else None  # pre-computed colours pass through
        # the dummy screen-space leaf receives the (rewritten) screen-space gradient: it is what densification reads
        grad_inputs[-2] = g_means2D if ctx.needs_input_grad[-2] else None
        return tuple(grad_inputs)


def preprocess(means3D: Tensor, scales: Tensor, rotations: Tensor, opacities: Tensor, sh_or_colors: Tensor,
               sh_rest: Optional[Tensor], Tw2v: Tensor, Tv2c: Tensor, campos: Tensor, tanFoV: Tensor, W: int, H: int,
               sh_degree=0, is_opengl=True, cov3D: Tensor = None, cov2D: Tensor = None, means2D: Tensor = None,
               culling: Tensor = None):
    """-> (means2D, depths, colors, radii, tiles_touched, conic_opacity); gaussian_render.py:569-626."""
    return _preprocess.apply(means3D, scales, rotations, opacities, sh_or_colors, sh_rest, Tw2v, Tv2c, campos, tanFoV,
                             W, H, sh_degree, is_opengl, cov3D, cov2D, means2D, culling)


# How the blend backward of `RasterizeGaussians` sums a Gaussian's gradient over its tiles: False = device-scope atomics
# into zero-filled tensors as the reference does (the faster way on this path: 2 058 against 1 839 frames/s at 300k
# Gaussians, 800x800, because a Gaussian's record is small and the records' fill and second pass cost more than its few
# atomics); True = per-instance records added in a fixed order, so that the sums do not vary from run to run.
DETERMINISTIC_SUMS = False
# `RasterizeGaussians` bins without the (Gaussian, tile) instances that no pixel of their tile can blend (the ellipse on
# which alpha reaches 1/255 against each tile of the 3-sigma rectangle): same images and gradients from shorter lists;
# the lists and n_contrib in RasterizeBuffer3D are the shorter ones. False: the reference's lists.
CULL_LISTS = True


class _GS_render(torch.autograd.Function):
    _forward = get_C_function('gaussian_rasterize_forward')
    _backward = get_C_function('gaussian_rasterize_backward')

    @staticmethod
    def forward(ctx, W, H, mean2D, colors, conic_opacity, tile_range, point_list, extras, accum_max_count,
                accum_weights_p, accum_weights_count, point_offsets=None, radii=None, keep_masks=None):
        images, out_opacity, out_extras, n_contrib = _GS_render._forward(
            W, H, mean2D, conic_opacity, colors, extras, point_list, tile_range, accum_max_count, accum_weights_p,
            accum_weights_count, None)
        ctx.save_for_backward(mean2D, colors, conic_opacity, extras, tile_range, point_list, out_opacity, n_contrib,
                              point_offsets, radii, keep_masks)
        ctx.mark_non_differentiable(n_contrib)
        return images, out_opacity, out_extras, n_contrib

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_images, grad_alpha, grad_out_extra, _):
        (mean2D, colors, conic_opacity, extras, tile_range, point_list, out_opacity, n_contrib, point_offsets,
         radii, keep_masks) = ctx.saved_tensors
        zeros_like = lambda t: torch.zeros_like(t)
        grad_images = zeros_like(out_opacity).expand(3, -1, -1).contiguous() if grad_images is None else grad_images
        grad_alpha = zeros_like(out_opacity) if grad_alpha is None else grad_alpha
        if extras is not None and grad_out_extra is None:
            grad_out_extra = torch.zeros((extras.shape[1],) + tuple(out_opacity.shape), dtype=torch.float32,
                                         device=out_opacity.device)
        grad_colors, grad_extra, grad_means2D, grad_conic_opacity = _GS_render._backward(
            mean2D, conic_opacity, colors, extras, out_opacity, grad_images.contiguous(), grad_alpha.contiguous(),
            None if grad_out_extra is None else grad_out_extra.contiguous(), tile_range, point_list, n_contrib,
            point_offsets, radii, culled=keep_masks)
        return (None, None, grad_means2D, grad_colors, grad_conic_opacity, None, None, grad_extra, None, None, None,
                None, None, None)


class _GS_render_fast(torch.autograd.Function):
    """The reference's bucketed variant (gaussian_render.py:803-837): the forward also stores the running state before
    every 32nd list entry, the backward is `gaussian_rasterize_fast_backward` on those snapshots."""
    _forward = get_C_function('gaussian_rasterize_forward')
    _backward = get_C_function('gaussian_rasterize_fast_backward')

    @staticmethod
    def forward(ctx, W, H, mean2D, colors, conic_opacity, tile_range, point_list, extras, accum_max_count,
                accum_weights_p, accum_weights_count, point_offsets=None, radii=None, keep_masks=None):
        per_tile_bucket_offset = (tile_range[..., 1] - tile_range[..., 0] + 31) // 32
        per_tile_bucket_offset = torch.cumsum(per_tile_bucket_offset, dim=-1).contiguous()
        (images, out_opacity, out_extras, n_contrib, max_contrib, bucket_to_tile, sampled_T,
         sampled_ar) = _GS_render_fast._forward(W, H, mean2D, conic_opacity, colors, extras, point_list, tile_range,
                                                accum_max_count, accum_weights_p, accum_weights_count,
                                                per_tile_bucket_offset)
        ctx.save_for_backward(mean2D, colors, conic_opacity, extras, tile_range, point_list, images, out_opacity,
                              out_extras, n_contrib, per_tile_bucket_offset, max_contrib, bucket_to_tile, sampled_T,
                              sampled_ar, point_offsets, radii, keep_masks)
        ctx.mark_non_differentiable(n_contrib)
        return images, out_opacity, out_extras, n_contrib

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_images, grad_alpha, grad_out_extra, _):
        (mean2D, colors, conic_opacity, extras, tile_range, point_list, images, out_opacity, out_extras, n_contrib,
         per_tile_bucket_offset, max_contrib, bucket_to_tile, sampled_T, sampled_ar, point_offsets,
         radii, keep_masks) = ctx.saved_tensors
        grad_images = torch.zeros_like(images) if grad_images is None else grad_images
        grad_alpha = torch.zeros_like(out_opacity) if grad_alpha is None else grad_alpha
        if extras is not None and grad_out_extra is None:
            grad_out_extra = torch.zeros_like(out_extras)
        grad_colors, grad_extra, grad_means2D, grad_conic_opacity = _GS_render_fast._backward(
            mean2D, conic_opacity, colors, extras, images, out_extras, out_opacity, grad_images.contiguous(),
            grad_alpha.contiguous(), None if grad_out_extra is None else grad_out_extra.contiguous(), tile_range,
            point_list, n_contrib, max_contrib, per_tile_bucket_offset, bucket_to_tile, sampled_T, sampled_ar,
            point_offsets, radii, culled=keep_masks)
        return (None, None, grad_means2D, grad_colors, grad_conic_opacity, None, None, grad_extra, None, None, None,
                None, None, None)


def GS_render_fast(W: int, H: int, mean2D: Tensor, colors: Tensor, conic_opacity: Tensor, tile_range: Tensor,
                   point_list: Tensor, extra: Tensor = None, accum_max_count=None, accum_weights_p=None,
                   accum_weights_count=None, point_offsets: Tensor = None, radii: Tensor = None,
                   keep_masks: Tensor = None):
    """`GS_render` through the bucketed forward / per-Gaussian backward pair (gaussian_render.py:803-837).
    `point_offsets` / `radii` / `keep_masks` as for `GS_render`."""
    return _GS_render_fast.apply(W, H, mean2D, colors, conic_opacity, tile_range, point_list, extra, accum_max_count,
                                 accum_weights_p, accum_weights_count, point_offsets, radii, keep_masks)


def GS_render(W: int, H: int, mean2D: Tensor, colors: Tensor, conic_opacity: Tensor, tile_range: Tensor,
              point_list: Tensor, extra: Tensor = None, accum_max_count=None, accum_weights_p=None,
              accum_weights_count=None, point_offsets: Tensor = None, radii: Tensor = None,
              keep_masks: Tensor = None):
    """-> (images[3,H,W], opacity[H,W], extras[E,H,W]|None, n_contrib[H,W]); gaussian_render.py:839-845. With the
    binning's scan offsets (`GS_prepare(..., return_offsets=True)`) and the radii the backward sums the per-Gaussian
    gradients in a fixed order without atomics; `keep_masks` must come along when the lists were built by
    `GS_prepare(..., cull=True)`."""
    return _GS_render.apply(W, H, mean2D, colors, conic_opacity, tile_range, point_list, extra, accum_max_count,
                            accum_weights_p, accum_weights_count, point_offsets, radii, keep_masks)


def RasterizeGaussians(means3D: Tensor, means2D: Optional[Tensor], colors: Tensor, sh_rest: Optional[Tensor],
                       opacities: Tensor, scales: Optional[Tensor], rotations: Optional[Tensor],
                       cov3Ds_precomp: Optional[Tensor], cov2Ds_precomp: Optional[Tensor], extras: Optional[Tensor],
                       image_size: Tuple[int, int], sh_degree: int, Tw2v: Tensor, Tv2c: Tensor, cam_pos: Tensor,
                       tanFoV: Tensor, is_opengl: bool, culling: Optional[Tensor], accum_max_count: Optional[Tensor],
                       accum_weights_p: Optional[Tensor], accum_weights_count: Optional[Tensor], *other_extras: Tensor):
    """gaussian_render.py:226-274: preprocess -> binning -> blend."""
    W, H = image_size
    means2D, depths, colors, radii, tiles_touched, conic_opacity = preprocess(
        means3D, scales, rotations, opacities, colors, sh_rest, Tw2v, Tv2c, cam_pos, tanFoV, W, H, sh_degree,
        is_opengl, cov3Ds_precomp, cov2Ds_precomp, means2D, culling)
    keep = _cull_masks(W, H, means2D.detach(), conic_opacity.detach(), radii) if CULL_LISTS else None
    tile_ranges, point_list, point_offsets = GS_prepare(W, H, means2D.detach(), depths.detach(), radii, tiles_touched,
                                                        False, return_offsets=True, cull=keep is not None,
                                                        keep_masks=keep)[:3]
    ordered = DETERMINISTIC_SUMS
    out_pixels, out_opacities, out_extras, n_contrib = GS_render(
        W, H, means2D, colors, conic_opacity, tile_ranges, point_list, extras, accum_max_count, accum_weights_p,
        accum_weights_count, point_offsets if ordered else None, radii if ordered else None,
        keep if ordered else None)
    buffer = RasterizeBuffer3D(W, H, len(opacities), point_list.shape[0], tile_ranges, point_list, n_contrib,
                               conic_opacity, means2D, out_opacities)
    out_other_extras = [_render_extra.apply(W, H, extras_, means2D, conic_opacity, tile_ranges, point_list, n_contrib,
                                            out_opacities) for extras_ in other_extras]
    return (out_pixels, out_opacities, out_extras, radii, buffer, *out_other_extras)


def render(Tw2v: Tensor, Tv2c: Tensor, size: Tuple[int, int], points: Tensor, opacity: Tensor, scales: Tensor = None,
           rotations: Tensor = None, campos: Tensor = None, FoV: Tensor = None, focals: Tensor = None,
           cov3Ds: Tensor = None, cov2Ds: Tensor = None, sh_features: Tensor = None, sh_features_rest: Tensor = None,
           colors: Tensor = None, sh_degree=0, is_opengl=False, culling: Tensor = None,
           accum_max_count: Tensor = None, accum_weights_p: Tensor = None, accum_weights_count: Tensor = None,
           **kwargs):
    """Same inputs, outputs and dict keys as the reference's `render` (gaussian_render.py:277-359)."""
    means2D = torch.zeros_like(points[:, :2]).contiguous().requires_grad_()
    if campos is None:
        campos = Tw2v.inverse()[:3, 3].contiguous()
    if FoV is None:
        tanFoV = 0.5 * torch.as_tensor(size, device=Tw2v.device) / focals
    else:
        tanFoV = torch.tan(torch.as_tensor(FoV) * 0.5)
    extras, extra_key = None, None
    for k, v in list(kwargs.items()):
        if isinstance(v, Tensor) and v.shape[-1] <= 4:
            extras, extra_key = v, k
            kwargs.pop(k)
            break
    c = lambda t: None if t is None else t.contiguous()
    others = {k: v for k, v in kwargs.items() if isinstance(v, Tensor)}
    image, out_opacity, out_extra, radii, buffer, *out_others = RasterizeGaussians(
        points.contiguous(), means2D, c(sh_features) if colors is None else colors.contiguous(), c(sh_features_rest),
        opacity.contiguous(), c(scales), c(rotations), c(cov3Ds), c(cov2Ds), c(extras), size,
        sh_degree if colors is None else -1, Tw2v.view(4, 4).contiguous(), Tv2c.view(4, 4).contiguous(),
        campos.view(3).contiguous(), tanFoV.view(2), is_opengl, culling, accum_max_count, accum_weights_p,
        accum_weights_count, *others.values())
    out = {'images': image, 'opacity': out_opacity, 'viewspace_points': means2D, 'visibility_filter': radii > 0,
           'radii': radii, 'buffer': buffer}
    out.update(zip(others.keys(), out_others))  # each [H,W,E], pixel-major as in the reference
    if extra_key is not None:
        out[extra_key] = out_extra
    return out
