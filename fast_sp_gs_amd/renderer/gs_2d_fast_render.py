"""Host side of the "fast" 2DGS surfel renderer: the autograd wiring and the PyTorch epilogue of the reference's
`fast_2d_gs/renderer/gs_2d_fast_render.py` (`_fast_preprocess` :23-72, `_fast_rasterize` :345-383, `_fast_rasterize_v2`
:386-431, `_Fast_Render` :592-667, `GS_2D_fast_render` :670-754, `_fast_compute_trans_mat` :757-789), calling the HIP
operators through the operator boundary by name.
"""
from __future__ import annotations

import torch
from torch import Tensor

from fast_sp_gs_amd._C import get_C_function
from .gs_2d_render import depth_to_normal

__all__ = ['GS_2D_fast_render', 'GS_2D_fast_preprocess', 'GS_2D_fast_rasterize', 'GS_2D_fast_rasterize_v2',
           'fast_compuate_transmat', 'fast_render_step']


def _grad_buffers(means3D, scales, rotations, opacities, shs_or_colors, shs_rest, sh_degree, want_shs, want_rest):
    """Outputs of gs_2d_fast_preprocess_backward. The kernel writes every row of the geometry gradients (zeros for
    surfels that were not rendered) and, when every stored coefficient is active, of the SH gradient, so those are
    allocated uninitialised; anything else starts from zeros, as the reference's wrapper has it."""
    full_sh = (sh_degree >= 0 and shs_rest is None and shs_or_colors is not None
               and shs_or_colors.shape[1] == (sh_degree + 1) ** 2)
    g_shs = None
    if want_shs and shs_or_colors is not None:
        g_shs = torch.empty_like(shs_or_colors) if full_sh else torch.zeros_like(shs_or_colors)
    g_rest = torch.zeros_like(shs_rest) if shs_rest is not None and want_rest else None
    return (torch.empty_like(means3D), torch.empty_like(scales), torch.empty_like(rotations),
            torch.empty_like(opacities), g_shs, g_rest)


class _fast_preprocess(torch.autograd.Function):
    _forward_func = get_C_function('gs_2d_fast_preprocess_forward')
    _backward_func = get_C_function('gs_2d_fast_preprocess_backward')

    @staticmethod
    def forward(ctx, W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v,
                Tv2c, Tv2s, campos, trans_precomp, means2D, culling):
        (means2D, colors, trans_mat, inverse_m, normal_opacity, depths, radii, tile_range,
         point_list) = _fast_preprocess._forward_func(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities,
                                                      shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s, campos, trans_precomp,
                                                      means2D, culling, False)
        ctx.save_for_backward(means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s, campos,
                              means2D, colors, trans_mat, radii, normal_opacity)
        ctx._info = (W, H, sh_degree, is_opengl)
        ctx.mark_non_differentiable(radii, tile_range, point_list)
        return colors, means2D, trans_mat, inverse_m, normal_opacity, depths, radii, tile_range, point_list

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outputs):
        (means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s, campos, means2D, colors,
         trans_mat, radii, normal_opacity) = ctx.saved_tensors
        W, H, sh_degree, is_opengl = ctx._info
        grad_colors, grad_means2D, grad_mat, grad_inverse_m, grad_normal_opacity, grad_depth = grad_outputs[:6]
        z = lambda g, like: torch.zeros_like(like) if g is None else g.contiguous()
        grad_colors, grad_means2D = z(grad_colors, colors), z(grad_means2D, means2D).clone()
        grad_mat, grad_inverse_m = z(grad_mat, trans_mat), z(grad_inverse_m, trans_mat)
        grad_normal_opacity = z(grad_normal_opacity, normal_opacity)
        grad_inputs = [
            None, None, None, None,
            *_grad_buffers(means3D, scales, rotations, opacities, shs_or_colors, shs_rest, sh_degree,
                           ctx.needs_input_grad[8], ctx.needs_input_grad[9]),
            None, None, None, None, None, None, None,
        ]
        _fast_preprocess._backward_func(
            W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2s,
            campos, trans_mat, radii, colors, normal_opacity, grad_means2D, grad_mat, grad_inverse_m, grad_depth,
            grad_colors, grad_normal_opacity, grad_inputs[4], grad_inputs[5], grad_inputs[6], grad_inputs[7],
            grad_inputs[8], grad_inputs[9], grad_inputs[10], grad_inputs[11])
        if sh_degree < 0 and grad_inputs[8] is not None:
            grad_inputs[8] = grad_colors  # precomputed colours pass their gradient straight through
        grad_inputs[15] = grad_means2D if ctx.needs_input_grad[15] else None  # densification proxy
        return tuple(grad_inputs)


def GS_2D_fast_preprocess(W: int, H: int, sh_degree: int, is_opengl: bool, means3D: Tensor, scales: Tensor,
                          rotations: Tensor, opacities: Tensor, shs_or_colors: Tensor, shs_features_rest, Tw2v: Tensor,
                          Tv2c: Tensor, Tv2s: Tensor, campos: Tensor, trans_precomp: Tensor = None,
                          means2D: Tensor = None, culling: Tensor = None):
    return _fast_preprocess.apply(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors,
                                  shs_features_rest, Tw2v, Tv2c, Tv2s, campos, trans_precomp, means2D, culling)


class _fast_rasterize(torch.autograd.Function):
    """Blend with the per-pixel backward (no snapshots)."""
    _forward_func = get_C_function('GS_2D_fast_render_forward')
    _backward_func = get_C_function('GS_2D_fast_render_backward')
    _per_splat = False

    @classmethod
    def _bucket_offset(cls, tile_range):
        if not cls._per_splat:
            return None
        per_tile = (tile_range[..., 1] - tile_range[..., 0] + 31) // 32
        return torch.cumsum(per_tile, dim=-1).contiguous()

    @classmethod
    def _forward(cls, ctx, W, H, means2D, colors, normal_opacity, trans_mat, inverse_m, tile_range, point_list, near_n,
                 far_n, only_image, trans_mat_t2, accum_max_count, accum_weights_p, accum_weights_count):
        offset = cls._bucket_offset(tile_range)
        outs = cls._forward_func(W, H, near_n, far_n, only_image, means2D, colors, normal_opacity, trans_mat, inverse_m,
                                 point_list, tile_range, trans_mat_t2, accum_max_count, accum_weights_p,
                                 accum_weights_count, offset)
        pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib = outs[:5]
        ctx._info = (near_n, far_n)
        ctx._snap = (offset, *outs[5:]) if offset is not None and len(outs) > 5 else None
        ctx.save_for_backward(means2D, normal_opacity, trans_mat, inverse_m, colors, pixel_colors, pixel_extras,
                              pixel_opacity, tile_range, point_list, n_contrib, trans_mat_t2, pixel_flow)
        ctx.mark_non_differentiable(n_contrib)
        return pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib

    @classmethod
    def _backward(cls, ctx, grad_outputs):
        (means2D, normal_opacity, trans_mat, inverse_m, colors, pixel_colors, pixel_extras, pixel_opacity, tile_range,
         point_list, n_contrib, trans_mat_t2, pixel_flow) = ctx.saved_tensors
        grad_images, grad_opacity, grad_others, grad_flow, _ = grad_outputs
        if pixel_flow is None or grad_others is None:
            grad_flow = None
        if grad_images is None:
            grad_images = torch.zeros_like(pixel_colors)
        if grad_opacity is None:
            grad_opacity = torch.zeros_like(pixel_opacity)
        if ctx._snap is not None:
            offset, max_contrib, bucket_to_tile, sampled_T, sampled_acc, sampled_aux = ctx._snap
            snap = (offset, bucket_to_tile, max_contrib, sampled_T, sampled_acc, sampled_aux)
        else:
            snap = (None,) * 6
        grad_colors, grad_means2D, grad_trans, grad_inv_m, grad_normal_opacity = cls._backward_func(
            means2D, normal_opacity, colors, trans_mat, inverse_m, trans_mat_t2, pixel_colors, pixel_opacity,
            pixel_extras, pixel_flow, grad_images, grad_opacity, grad_others, grad_flow, tile_range, point_list,
            n_contrib, *ctx._info, *snap)
        grad_inputs = [None] * 16
        grad_inputs[2] = grad_means2D
        grad_inputs[3] = grad_colors
        grad_inputs[4] = grad_normal_opacity
        grad_inputs[5] = grad_trans
        grad_inputs[6] = grad_inv_m
        return tuple(grad_inputs)

    @staticmethod
    def forward(ctx, *inputs):
        return _fast_rasterize._forward(ctx, *inputs)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outputs):
        return _fast_rasterize._backward(ctx, grad_outputs)


class _fast_rasterize_v2(_fast_rasterize):
    """Blend whose forward also records the per-bucket snapshots and whose backward uses the per-splat channel set."""
    _per_splat = True

    @staticmethod
    def forward(ctx, *inputs):
        return _fast_rasterize_v2._forward(ctx, *inputs)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outputs):
        return _fast_rasterize_v2._backward(ctx, grad_outputs)


def GS_2D_fast_rasterize(W: int, H: int, mean2D: Tensor, colors: Tensor, normal_opacity: Tensor, trans_mat: Tensor,
                         inverse_m: Tensor, tile_range: Tensor, point_list: Tensor, near_n=0.2, far_n=100.,
                         only_image=False, accum_max_count=None, accum_weights_p=None, accum_weights_count=None):
    images, opacities, extras, _, n_contrib = _fast_rasterize.apply(
        W, H, mean2D, colors, normal_opacity, trans_mat, inverse_m, tile_range, point_list, near_n, far_n, only_image,
        None, accum_max_count, accum_weights_p, accum_weights_count)
    return images, opacities, extras, n_contrib


def GS_2D_fast_rasterize_v2(W: int, H: int, mean2D: Tensor, colors: Tensor, normal_opacity: Tensor, trans_mat: Tensor,
                            inverse_m: Tensor, tile_range: Tensor, point_list: Tensor, near_n=0.2, far_n=100.,
                            only_image=False, accum_max_count=None, accum_weights_p=None, accum_weights_count=None):
    images, opacities, extras, _, n_contrib = _fast_rasterize_v2.apply(
        W, H, mean2D, colors, normal_opacity, trans_mat, inverse_m, tile_range, point_list, near_n, far_n, only_image,
        None, accum_max_count, accum_weights_p, accum_weights_count)
    return images, opacities, extras, n_contrib


class _Fast_Render(torch.autograd.Function):
    _preprocess_forward = get_C_function('gs_2d_fast_preprocess_forward')
    _preprocess_backward = get_C_function('gs_2d_fast_preprocess_backward')
    _render_forward = get_C_function('GS_2D_fast_render_forward')
    _render_backward = get_C_function('GS_2D_fast_render_backward')

    @staticmethod
    def forward(ctx, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s, campos, size,
                sh_degree, is_opengl, near_n, far_n, only_image, trans_precomp, means2D, trans_mat_t2, culling,
                accum_max_count, accum_weights_p, accum_weights_count):
        W, H = size
        (means2D, colors, trans_mat, inverse_m, normal_opacity, depths, radii, tile_range, point_list,
         point_offsets, keep_masks) = _Fast_Render._preprocess_forward(
            W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s,
            campos, trans_precomp, means2D, culling, False, return_offsets=True, return_masks=True)
        pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib = _Fast_Render._render_forward(
            W, H, near_n, far_n, only_image, means2D, colors, normal_opacity, trans_mat, inverse_m, point_list,
            tile_range, trans_mat_t2, accum_max_count, accum_weights_p, accum_weights_count, None)
        ctx._info = (W, H, sh_degree, is_opengl, near_n, far_n)
        ctx.save_for_backward(means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s, campos,
                              means2D, trans_mat, inverse_m, radii, colors, normal_opacity, tile_range, point_list,
                              pixel_colors, pixel_extras, pixel_opacity, n_contrib, trans_mat_t2, pixel_flow,
                              point_offsets, keep_masks)
        ctx.mark_non_differentiable(n_contrib, radii)
        return pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib, radii

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outputs):
        (means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2c, Tv2s, campos, means2D, trans_mat,
         inverse_m, radii, colors, normal_opacity, tile_range, point_list, pixel_colors, pixel_extras, pixel_opacity,
         n_contrib, trans_mat_t2, pixel_flow, point_offsets, keep_masks) = ctx.saved_tensors
        W, H, sh_degree, is_opengl, near_n, far_n = ctx._info
        grad_images, grad_opacity, grad_others, grad_flow = grad_outputs[:4]
        if pixel_flow is None or grad_others is None:
            grad_flow = None
        if grad_images is None:
            grad_images = torch.zeros_like(pixel_colors)
        if grad_opacity is None:
            grad_opacity = torch.zeros_like(pixel_opacity)
        grad_colors, grad_means2D, grad_trans, grad_inv_m, grad_normal_opacity = _Fast_Render._render_backward(
            means2D, normal_opacity, colors, trans_mat, inverse_m, trans_mat_t2, pixel_colors, pixel_opacity,
            pixel_extras, pixel_flow, grad_images, grad_opacity, grad_others, grad_flow, tile_range, point_list,
            n_contrib, near_n, far_n, None, None, None, None, None, None, point_offsets, radii,
            keep_masks=keep_masks)
        grad_inputs = [
            *_grad_buffers(means3D, scales, rotations, opacities, shs_or_colors, shs_rest, sh_degree,
                           ctx.needs_input_grad[4], ctx.needs_input_grad[5]),
            None, None, None, None,
            None, None, None, None, None, None,
            None, grad_means2D, None,
            None, None, None, None,
        ]
        _Fast_Render._preprocess_backward(
            W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs_or_colors, shs_rest, Tw2v, Tv2s,
            campos, trans_mat, radii, colors, normal_opacity, grad_means2D, grad_trans, grad_inv_m, None, grad_colors,
            grad_normal_opacity, grad_inputs[0], grad_inputs[1], grad_inputs[2], grad_inputs[3], grad_inputs[4],
            grad_inputs[5], grad_inputs[6], grad_inputs[9])
        if sh_degree < 0 and grad_inputs[4] is not None:
            grad_inputs[4] = grad_colors
        return tuple(grad_inputs)


def GS_2D_fast_render(points: Tensor, scales: Tensor, rotations: Tensor, opacity: Tensor, size, Tw2v: Tensor,
                      Tv2c: Tensor, Tv2s: Tensor, campos: Tensor = None, focals: Tensor = None, FoV: Tensor = None,
                      is_opengl=False, near=0.2, far=100, sh_degree=0, colors: Tensor = None,
                      sh_features: Tensor = None, sh_features_rest: Tensor = None, depth_ratio=1.,
                      culling: Tensor = None, accum_max_count: Tensor = None, accum_weights_p: Tensor = None,
                      accum_weights_count: Tensor = None, trans_mat_t2: Tensor = None, **kwargs):
    means2D = points.new_zeros(points.shape[0], 2, requires_grad=True)
    W, H = size
    if campos is None:
        campos = Tw2v.inverse()[:3, 3].contiguous()
    images, opacities, out_extras, flows, n_contrib, radii = _Fast_Render.apply(
        points, scales, rotations, opacity, sh_features if colors is None else colors, sh_features_rest,
        Tw2v.contiguous(), Tv2c.contiguous(), Tv2s.contiguous(), campos.contiguous(), size,
        sh_degree if colors is None else -1, is_opengl, near, far, False, None, means2D, trans_mat_t2, culling,
        accum_max_count, accum_weights_p, accum_weights_count)
    depths, normals, median_depths, distortion, _ = out_extras.split([1, 3, 1, 1, 2], dim=0)
    normals = (normals.permute(1, 2, 0) @ Tw2v[:3, :3]).permute(2, 0, 1)
    median_depths = torch.nan_to_num(median_depths, 0, 0)
    depths = torch.nan_to_num(depths, 0, 0)
    surf_depth = depths * (1 - depth_ratio) + depth_ratio * median_depths
    surf_normal = depth_to_normal(Tw2v, Tv2c, (W, H), surf_depth).permute(2, 0, 1)
    surf_normal = surf_normal * opacities.detach()
    return {
        'images': images, 'normals': normals, 'opacity': opacities, 'distortion': distortion,
        'surf_depth': surf_depth, 'surf_normal': surf_normal, 'radii': radii, 'viewspace_points': means2D,
        'visibility_filter': radii > 0, 'flows': flows,
    }


class _fast_compute_trans_mat(torch.autograd.Function):
    _forward_func = get_C_function('gs_2d_fast_compute_transmat_forward')
    _backward_func = get_C_function('gs_2d_fast_compute_trans_mat_backward')

    @staticmethod
    def forward(ctx, means3D, scales, rotations, Tw2v, Tv2s):
        matrix, normals = _fast_compute_trans_mat._forward_func(means3D, scales, rotations, Tw2v, Tv2s)
        ctx.save_for_backward(means3D, scales, rotations, Tw2v, Tv2s)
        return matrix, normals

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_matrix, grad_normals):
        means3D, scales, rotations, Tw2v, Tv2s = ctx.saved_tensors
        g3, gs, gr = _fast_compute_trans_mat._backward_func(means3D, scales, rotations, Tw2v, Tv2s,
                                                            grad_matrix.contiguous(), grad_normals.contiguous())
        return g3, gs, gr, None, None


def fast_compuate_transmat(means3D: Tensor, scales: Tensor, rotations: Tensor, Tw2v: Tensor, Tv2s: Tensor):
    """Name kept as spelled in the reference (gs_2d_fast_render.py:779)."""
    return _fast_compute_trans_mat.apply(means3D, scales, rotations, Tw2v, Tv2s)


def fast_render_step(scene, cam, grad_image: Tensor, grad_extras: Tensor = None, grad_opacity: Tensor = None,
                     per_splat: bool = False, ordered_sums: bool = True, per_splat_kernel: bool = False,
                     reuse_masks: bool = True):
    """One forward + backward pass of the fast path through the raw operators, returning every intermediate. With
    `ordered_sums` the blend backward adds per-instance records in a fixed order instead of using atomics. With
    `per_splat_kernel` (needs `per_splat`) the backward is the reference's per-splat decomposition, started from the
    forward's snapshots, instead of the back-to-front kernel with the per-splat channel set. `reuse_masks`: the ordered
    sum reads the corner test's verdicts the preprocess left instead of repeating the test (same sums)."""
    pre_f = get_C_function('gs_2d_fast_preprocess_forward')
    pre_b = get_C_function('gs_2d_fast_preprocess_backward')
    ren_f = get_C_function('GS_2D_fast_render_forward')
    ren_b = get_C_function('GS_2D_fast_render_backward')
    W, H = cam.W, cam.H
    (means2D, colors, trans_mat, inverse_m, normal_opacity, depths, radii, ranges, point_list, keys,
     tiles_touched, point_offsets, keep_masks) = pre_f(W, H, scene.sh_degree, False, scene.means3D, scene.scales,
                                                       scene.rotations, scene.opacities, scene.shs, None, cam.Tw2v,
                                                       cam.Tv2c, cam.Tv2s, cam.campos, None, None, None, False, True,
                                                       True, True)
    offset = None
    if per_splat:
        offset = torch.cumsum((ranges[:, 1] - ranges[:, 0] + 31) // 32, dim=0).contiguous()
    outs = ren_f(W, H, cam.near, cam.far, False, means2D, colors, normal_opacity, trans_mat, inverse_m, point_list,
                 ranges, None, None, None, None, offset)
    image, opacity, extras, _, n_contrib = outs[:5]
    if grad_opacity is None:
        grad_opacity = torch.zeros_like(opacity)
    g_colors, g_means2D, g_trans, g_inv, g_no = ren_b(
        means2D, normal_opacity, colors, trans_mat, inverse_m, None, image, opacity, extras, None, grad_image,
        grad_opacity, grad_extras, None, ranges, point_list, n_contrib, cam.near, cam.far, offset,
        *((outs[6], outs[5], outs[7], outs[8], outs[9]) if per_splat and per_splat_kernel else (None,) * 5),
        point_offsets if ordered_sums else None, radii if ordered_sums else None,
        per_splat_kernel=bool(per_splat and per_splat_kernel), keep_masks=keep_masks if reuse_masks else None)
    g_means2D_in = g_means2D.clone()
    # the preprocess backward writes every row of its outputs (zeros for surfels that were not rendered)
    g = dict(means3D=torch.empty_like(scene.means3D), scales=torch.empty_like(scene.scales),
             rotations=torch.empty_like(scene.rotations), opacities=torch.empty_like(scene.opacities),
             shs=torch.empty_like(scene.shs))
    pre_b(W, H, scene.sh_degree, False, scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs, None,
          cam.Tw2v, cam.Tv2s, cam.campos, trans_mat, radii, colors, normal_opacity, g_means2D, g_trans, g_inv, None,
          g_colors, g_no, g['means3D'], g['scales'], g['rotations'], g['opacities'], g['shs'], None)
    out = dict(means2D=means2D, colors=colors, trans_mat=trans_mat, inverse_m=inverse_m,
               normal_opacity=normal_opacity, depths=depths, radii=radii, tiles_touched=tiles_touched, ranges=ranges,
               point_list=point_list, keys=keys, keep_masks=keep_masks, image=image, opacity=opacity, extras=extras, n_contrib=n_contrib,
               g_colors=g_colors, g_means2D_blend=g_means2D_in, g_trans=g_trans, g_inv=g_inv, g_normal_opacity=g_no,
               g_means2D_proxy=g_means2D, g_means3D=g['means3D'], g_scales=g['scales'], g_rotations=g['rotations'],
               g_opacities=g['opacities'], g_shs=g['shs'])
    if per_splat:
        out.update(bucket_offset=offset, max_contrib=outs[5], bucket_to_tile=outs[6], sampled_T=outs[7],
                   sampled_acc=outs[8], sampled_aux=outs[9])
    return out
