"""Host side of the 2DGS surfel renderer: the autograd wiring and the PyTorch epilogue of the reference's
`fast_2d_gs/renderer/gs_2d_render.py` (`_GS_2D_Render` :473-547, `GS_2D_render` :550-633, `depth_to_normal` :438-470),
calling the HIP operators through the operator boundary by name, exactly as the reference's wrappers do.
"""
from __future__ import annotations

from typing import NamedTuple, Tuple, Union

import torch
from torch import Tensor

from fast_sp_gs_amd._C import get_C_function

__all__ = ['GS_2D_render', 'RasterizeBuffer', 'GS_2D_topk_weights', 'GS_prepare', 'render_step']

GS_prepare = get_C_function('GS_prepare')
# `_GS_2D_Render` bins with the blend kernels' own bound applied per (surfel, tile) instance: instances that no pixel of
# their tile can blend are left out of the lists (same images and gradients from shorter lists; the lists and n_contrib
# handed back in RasterizeBuffer are the shorter ones). False: the reference's lists, every tile of a surfel's rectangle.
CULL_LISTS = True


class RasterizeBuffer(NamedTuple):
    W: int
    H: int
    P: int
    R: int
    near: float
    far: float
    tile_ranges: Tensor
    point_list: Tensor
    n_contribed: Tensor
    means2D: Tensor
    normal_opacity: Tensor
    trans_mat: Tensor


def depths_to_points(Tw2v: Tensor, Tv2c: Tensor, size, depthmap: Tensor) -> Tensor:
    c2w = Tw2v.inverse()
    W, H = size
    ndc2pix = torch.tensor([[W / 2, 0, 0, W / 2], [0, H / 2, 0, H / 2], [0, 0, 0, 1]],
                           dtype=torch.float32, device=Tw2v.device).T
    projection_matrix = c2w.T @ (Tv2c @ Tw2v).T
    intrins = (projection_matrix @ ndc2pix)[:3, :3].T
    grid_x, grid_y = torch.meshgrid(torch.arange(W, device=c2w.device).float(),
                                    torch.arange(H, device=c2w.device).float(), indexing='xy')
    points = torch.stack([grid_x, grid_y, torch.ones_like(grid_x)], dim=-1).reshape(-1, 3)
    rays_d = points @ intrins.inverse().T @ c2w[:3, :3].T
    rays_o = c2w[:3, 3]
    return depthmap.reshape(-1, 1) * rays_d + rays_o


def depth_to_normal(Tw2v: Tensor, Tv2c: Tensor, size, depth: Tensor) -> Tensor:
    points = depths_to_points(Tw2v, Tv2c, size, depth).reshape(*depth.shape[1:], 3)
    output = torch.zeros_like(points)
    dx = points[2:, 1:-1] - points[:-2, 1:-1]
    dy = points[1:-1, 2:] - points[1:-1, :-2]
    output[1:-1, 1:-1, :] = torch.nn.functional.normalize(torch.cross(dx, dy, dim=-1), dim=-1)
    return output


class _GS_2D_Render(torch.autograd.Function):
    _preprocess_forward = get_C_function('gs_2d_preprocess_forward')
    _preprocess_backward = get_C_function('gs_2d_preprocess_backward')
    _render_forward = get_C_function('GS_2D_render_forward')
    _render_backward = get_C_function('GS_2D_render_backward')

    @staticmethod
    def forward(ctx, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, campos, size,
                sh_degree, is_opengl, near_n, far_n, only_image, trans_precomp, means2D, transe_mat_t2, culling,
                accum_max_count, accum_weights_p, accum_weights_count):
        W, H = size
        # the preprocess kernel also writes the blend kernels' packed per-surfel record (no second pass, no launch)
        cull = bool(CULL_LISTS)
        (means2D, colors, trans_mat, normal_opacity, depths, radii, tiles_touched, records,
         *keep) = _GS_2D_Render._preprocess_forward(
            W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c,
            campos, trans_precomp, means2D, culling, return_records=True, return_masks=cull)
        keep = keep[0] if cull else None
        tile_range, point_list, point_offsets = GS_prepare(
            W, H, means2D, depths, radii, tiles_touched, False, return_offsets=True, records=records, cull=cull,
            keep_masks=keep)[:3]
        pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib = _GS_2D_Render._render_forward(
            W, H, means2D, colors, normal_opacity, trans_mat, point_list, tile_range, near_n, far_n, only_image,
            transe_mat_t2, accum_max_count, accum_weights_p, accum_weights_count, records)
        ctx._info = (W, H, sh_degree, is_opengl, near_n, far_n)
        ctx._keep_masks = keep
        ctx.save_for_backward(means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, campos,
                              means2D, trans_mat, transe_mat_t2, radii, colors, normal_opacity, tile_range,
                              point_list, pixel_extras, pixel_opacity, pixel_flow, n_contrib, point_offsets, records)
        buffer = RasterizeBuffer(int(W), int(H), means3D.shape[0], point_list.shape[0], near_n, far_n, tile_range,
                                 point_list, n_contrib, means2D, normal_opacity, trans_mat)
        ctx.mark_non_differentiable(n_contrib, radii)
        return pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib, radii, buffer

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outputs):
        (means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, campos, means2D, trans_mat,
         transe_mat_t2, radii, colors, normal_opacity, tile_range, point_list, pixel_extras, pixel_opacity, pixel_flow,
         n_contrib, point_offsets, records) = ctx.saved_tensors
        W, H, sh_degree, is_opengl, near_n, far_n = ctx._info
        grad_images, grad_opacity, grad_others, grad_flows = grad_outputs[:4]
        if grad_images is None:
            grad_images = torch.zeros((3, H, W), dtype=torch.float32, device=means3D.device)
        if grad_opacity is None:
            grad_opacity = torch.zeros((H, W), dtype=torch.float32, device=means3D.device)
        grad_colors, grad_means2D, grad_trans, grad_normal_opacity = _GS_2D_Render._render_backward(
            means2D, normal_opacity, colors, trans_mat, transe_mat_t2, pixel_opacity, pixel_extras, pixel_flow,
            grad_images, grad_opacity, grad_others, grad_flows, tile_range, point_list, n_contrib, near_n, far_n,
            point_offsets, radii, records, culled=ctx._keep_masks)
        # the preprocess backward writes every row of its outputs (zeros for surfels that were not rendered), so they
        # are allocated uninitialised; pre-computed colours (sh_degree < 0) receive no gradient, as in the reference
        new = torch.empty_like
        grad_inputs = [
            new(means3D), new(scales), new(rotations), new(opacities),
            (new(shs_or_colors) if sh_degree >= 0 else torch.zeros_like(shs_or_colors))
            if ctx.needs_input_grad[4] else None,
            new(shs_rest) if shs_rest is not None and ctx.needs_input_grad[5] else None,
            None, None, None, None, None, None, None, None, None, None, grad_means2D, None, None, None, None, None,
        ]
        _GS_2D_Render._preprocess_backward(
            W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c,
            campos, trans_mat, radii, colors, normal_opacity, grad_means2D, grad_trans, None, grad_colors,
            grad_normal_opacity, grad_inputs[0], grad_inputs[1], grad_inputs[2], grad_inputs[3], grad_inputs[4],
            grad_inputs[5], grad_inputs[6], grad_inputs[8])
        return tuple(grad_inputs)


class _GS_2D_Epilogue(torch.autograd.Function):
    """normals to world space, nan_to_num of the depth maps, surf_depth, depth_to_normal * opacity.detach() and the
    optional background composite (gs_2d_render.py:608-617, network.py:725-726) through the fused kernels."""
    _forward = get_C_function('gs_2d_epilogue_forward')
    _backward = get_C_function('gs_2d_epilogue_backward')

    @staticmethod
    def forward(ctx, extras, opacity, images, background, Tw2v, Tv2c, depth_ratio, W, H):
        extras, opacity = extras.contiguous(), opacity.contiguous()
        bg = None if background is None else background.detach().reshape(3).contiguous()
        normals, depths, surf_depth, surf_normal, comp = _GS_2D_Epilogue._forward(
            W, H, depth_ratio, Tw2v, Tv2c, extras, opacity, None if images is None else images.contiguous(), bg)
        ctx.save_for_backward(extras, opacity, Tw2v, Tv2c, bg)
        ctx._info = (W, H, depth_ratio)
        ctx.set_materialize_grads(False)
        return normals, depths, surf_depth, surf_normal, comp

    @staticmethod
    def backward(ctx, g_normals, g_depths, g_surf_depth, g_surf_normal, g_comp):
        extras, opacity, Tw2v, Tv2c, bg = ctx.saved_tensors
        W, H, depth_ratio = ctx._info
        c = lambda t: None if t is None else t.contiguous()
        g_extras, g_opacity = _GS_2D_Epilogue._backward(W, H, depth_ratio, Tw2v, Tv2c, extras, opacity, bg,
                                                        c(g_normals), c(g_depths), c(g_surf_depth), c(g_surf_normal),
                                                        None, c(g_comp))
        return g_extras, g_opacity, g_comp, None, None, None, None, None, None


def GS_2D_render(points: Tensor, scales: Tensor, rotations: Tensor, opacity: Tensor,
                 size: Union[Tuple[int, int], Tensor], Tw2v: Tensor, Tv2c: Tensor, campos: Tensor = None,
                 focals: Tensor = None, FoV: Tensor = None, is_opengl=False, near=0.2, far=100, sh_degree=0,
                 colors: Tensor = None, sh_features: Tensor = None, sh_features_rest: Tensor = None, depth_ratio=1.,
                 culling: Tensor = None, trans_mat_t2: Tensor = None, accum_max_count: Tensor = None,
                 accum_weights_p: Tensor = None, accum_weights_count: Tensor = None, background: Tensor = None,
                 **kwargs):
    """Same inputs, outputs and dict keys as the reference's GS_2D_render (gs_2d_render.py:550-633). The per-pixel tail
    (:608-617) runs as one fused kernel each way. `background` ([3], optional, not in the reference's signature) also
    folds the caller's composite `images + (1 - opacity) * background` (network.py:725-726) into that kernel."""
    means2D = points.new_zeros(points.shape[0], 2, requires_grad=True)
    W, H = size
    if campos is None:
        campos = Tw2v.inverse()[:3, 3].contiguous()
    images, opacities, out_extras, flow, n_contrib, radii, buffer = _GS_2D_Render.apply(
        points, scales, rotations, opacity, sh_features if colors is None else colors, sh_features_rest,
        Tw2v.contiguous(), Tv2c.contiguous(), campos.contiguous(), size, sh_degree if colors is None else -1,
        is_opengl, near, far, False, None, means2D, trans_mat_t2, culling, accum_max_count, accum_weights_p,
        accum_weights_count)
    distortion = out_extras[5:6]
    if Tw2v.requires_grad or Tv2c.requires_grad:
        # camera optimisation: the fused epilogue produces no camera gradients, take the reference's torch ops
        if background is not None:
            images = images + (1.0 - opacities) * background.view(3, 1, 1)
        depths, normals, median_depths, _, _ = out_extras.split([1, 3, 1, 1, 3], dim=0)
        normals = (normals.permute(1, 2, 0) @ Tw2v[:3, :3]).permute(2, 0, 1)
        median_depths = torch.nan_to_num(median_depths, 0, 0)
        depths = torch.nan_to_num(depths, 0, 0)
        surf_depth = depths * (1 - depth_ratio) + depth_ratio * median_depths
        surf_normal = depth_to_normal(Tw2v, Tv2c, (W, H), surf_depth).permute(2, 0, 1)
        surf_normal = surf_normal * opacities.detach()
    else:
        normals, median_depths, surf_depth, surf_normal, composited = _GS_2D_Epilogue.apply(
            out_extras, opacities, images if background is not None else None, background, Tw2v.contiguous(),
            Tv2c.contiguous(), float(depth_ratio), W, H)
        if background is not None:
            images = composited
    outputs = {
        'images': images, 'depths': median_depths, 'normals': normals, 'opacity': opacities,
        'distortion': distortion, 'surf_depth': surf_depth, 'surf_normal': surf_normal, 'radii': radii,
        'viewspace_points': means2D, 'visibility_filter': radii > 0, 'buffer': buffer,
    }
    if flow is not None:
        outputs['flow'] = flow
    return outputs


def GS_2D_topk_weights(topk: int, buffer: RasterizeBuffer) -> Tuple[Tensor, Tensor]:
    fn = get_C_function('gs_2d_topk_weights')
    if fn is None:
        raise RuntimeError('gs_2d_topk_weights is not built into this library')
    return fn(topk, buffer.W, buffer.H, buffer.near, buffer.far, buffer.means2D, buffer.normal_opacity,
              buffer.trans_mat, buffer.tile_ranges, buffer.point_list)


def render_step(scene, cam, grad_image: Tensor, grad_extras: Tensor = None, grad_opacity: Tensor = None,
                ordered_sums: bool = True, packed: bool = True, background: Tensor = None, depth_ratio: float = 1.0,
                cull: bool = False):
    """One forward + backward pass of the hot path on raw operators (no autograd graph): preprocess -> binning ->
    blend -> blend backward -> preprocess backward, in the order `_GS_2D_Render` runs them. Returns a dict with every
    intermediate so callers (benchmark, parity tests) can inspect or time the stages.

    With `background` ([3]) the per-pixel epilogue of `GS_2D_render` runs between the two blend passes as it does in
    training: forward -> normals / depths / surf_depth / surf_normal / composited image; then `grad_image` is the
    gradient of the COMPOSITED image and the first six channels of `grad_extras` are read as the gradients of
    (surf_depth, normals x 3, depths, distortion); the epilogue backward turns them into the blend's dL/dextras and
    the composite's dL/dopacity (added to `grad_opacity`).

    `cull` (needs `packed`): bin as `_GS_2D_Render` does by default, leaving out the (surfel, tile) instances that no
    pixel of their tile can blend; every image and gradient is the same, `ranges` / `point_list` / `n_contrib` are those
    of the shorter lists."""
    f = get_C_function
    if cull and not packed:
        raise ValueError('cull needs the packed records')
    W, H = cam.W, cam.H
    dev = scene.means3D.device
    # with `packed` the preprocess kernel also writes the blend kernels' packed per-surfel record
    m2, colors, tm, no, depths, radii, tt, *rec = f('gs_2d_preprocess_forward')(
        W, H, scene.sh_degree, False, scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs, None,
        cam.Tw2v, cam.Tv2c, cam.campos, None, None, None, return_records=packed, return_masks=cull)
    keep = rec[-1] if cull else None
    rec = rec[0] if packed else None
    ranges, point_list, offsets = f('GS_prepare')(W, H, m2, depths, radii, tt, False, return_offsets=True,
                                                  records=rec, cull=cull, keep_masks=keep)[:3]
    oc, oo, oe, of, nc = f('GS_2D_render_forward')(W, H, m2, colors, no, tm, point_list, ranges, cam.near, cam.far,
                                                   False, None, None, None, None, rec)
    epilogue = {}
    if background is not None:
        normals, med, surf_depth, surf_normal, comp = f('gs_2d_epilogue_forward')(
            W, H, depth_ratio, cam.Tw2v, cam.Tv2c, oe, oo, oc, background)
        ge = grad_extras
        g_ex, g_op = f('gs_2d_epilogue_backward')(
            W, H, depth_ratio, cam.Tw2v, cam.Tv2c, oe, oo, background,
            None if ge is None else ge[1:4], None if ge is None else ge[4:5], None if ge is None else ge[0:1],
            None, None if ge is None else ge[5:6], grad_image)
        grad_extras = g_ex
        grad_opacity = g_op if grad_opacity is None else grad_opacity + g_op
        epilogue = dict(normals=normals, median_depths=med, surf_depth=surf_depth, surf_normal=surf_normal,
                        composited=comp)
    if grad_extras is None:
        grad_extras = torch.zeros((9, H, W), dtype=torch.float32, device=dev)
    if grad_opacity is None:
        grad_opacity = torch.zeros((H, W), dtype=torch.float32, device=dev)
    gc, gm2, gt, gno = f('GS_2D_render_backward')(m2, no, colors, tm, None, oo, oe, None, grad_image, grad_opacity,
                                                  grad_extras, None, ranges, point_list, nc, cam.near, cam.far,
                                                  offsets if ordered_sums else None, radii, rec, culled=keep)
    g_means3D, g_scales = torch.empty_like(scene.means3D), torch.empty_like(scene.scales)
    g_rot, g_opac, g_shs = torch.empty_like(scene.rotations), torch.empty_like(scene.opacities), torch.empty_like(scene.shs)
    f('gs_2d_preprocess_backward')(W, H, scene.sh_degree, False, scene.means3D, scene.scales, scene.rotations,
                                   scene.opacities, scene.shs, None, cam.Tw2v, cam.Tv2c, cam.campos, tm, radii, colors,
                                   no, gm2, gt, None, gc, gno, g_means3D, g_scales, g_rot, g_opac, g_shs, None)
    return dict(means2D=m2, colors=colors, trans_mat=tm, normal_opacity=no, depths=depths, radii=radii,
                tiles_touched=tt, ranges=ranges, point_list=point_list, image=oc, opacity=oo, extras=oe,
                n_contrib=nc, g_colors=gc, g_means2D=gm2, g_trans=gt, g_normal_opacity=gno, g_means3D=g_means3D,
                g_scales=g_scales, g_rot=g_rot, g_opac=g_opac, g_shs=g_shs, **epilogue)
