"""Python-facing operators with the reference's names and positional signatures (the pybind `m.def` list of
`fast_2d_gs/_C/src/**`), each a thin marshalling layer over one C-ABI entry point of libfsgs_hip.so.

torch is used only to allocate device memory and to name the current stream. Argument checks mirror the reference's
CHECK_INPUT / CHECK_SHAPE macros and raise RuntimeError like TORCH_CHECK does.
"""
from __future__ import annotations

import ctypes
import threading
from typing import List, Optional, Sequence, Tuple

import torch
from torch import Tensor

from .. import lib as L

__all__ = [
    'gs_2d_preprocess_forward', 'gs_2d_preprocess_backward', 'gs_2d_compute_transmat_forward',
    'gs_2d_compute_trans_mat_backward', 'GS_prepare', 'GS_2D_render_forward', 'GS_2D_render_backward',
    'SH_to_RGB_forward', 'SH_to_RGB_backward', 'sh_encode_forward', 'sh_encode_backward', 'freq_encode_forward',
    'freq_encode_backward', 'cdist_top', 'cdist_top_backward', 'AdamMasksedUpdated', 'knn_topk', 'lbs_blend',
    'knn_topk_backward', 'lbs_blend_backward',
    'gs_2d_topk_weights', 'mlp_pack_weights', 'mlp_forward', 'mlp_pack_transposed', 'mlp_backward', 'gs_2d_pack_records', 'gs_cull_masks', 'gs_2d_fast_preprocess_forward',
    'gs_2d_fast_preprocess_backward', 'gs_2d_fast_compute_transmat_forward', 'gs_2d_fast_compute_trans_mat_backward',
    'GS_2D_fast_render_forward', 'GS_2D_fast_render_backward', 'fusedssim', 'fusedssim_backward',
    'gs_2d_epilogue_forward', 'gs_2d_epilogue_backward', 'simple_knn', 'gs_preprocess_forward',
    'gs_preprocess_backward', 'gaussian_rasterize_forward', 'gaussian_rasterize_backward', 'gaussian_rasterize_fast_backward',
    'select_indices',
    'gather_rows', 'densify_masks', 'prune_mask', 'split_children', 'densification_stats',
    'gs_compute_cov3D_forward', 'gs_compute_cov3D_backward', 'gs_compute_cov2D_forward', 'gs_compute_cov2D_backward',
    'gaussian_topk_weights', 'gaussian_rasterize_extra_forward', 'gaussian_rasterize_extra_backward',
    'gaussian_rasterize_extra_backward_v2', 'AdamMasksedUpdatedMulti', 'mlp_pack_all',
    'image_loss_forward', 'image_loss_backward', 'deform_apply_forward', 'deform_apply_backward',
]

_TILE = 16

# When set to a list, every operator appends (name, start_event, end_event) recorded on the current stream tightly
# around its C-ABI call (allocation and zero-fill of outputs stay outside), so callers can time the kernels themselves.
STAGE_EVENTS = None
# Optional set of operator names: when set, only these are timed. An event is a packet of its own in the device queue
# and costs a few microseconds between two kernels, so a caller that times a whole region brackets only what it needs.
STAGE_FILTER = None
# Events to use for that (already created and recorded once by the caller): creating timing events is not free -- the
# runtime grows its event pool in bursts of tens of milliseconds -- so a caller that times a region fills this first.
EVENT_POOL: list = []


def _event():
    return EVENT_POOL.pop() if EVENT_POOL else torch.cuda.Event(enable_timing=True)


class _timed:
    __slots__ = ('name', 'start')

    def __init__(self, name):
        self.name = name

    def __enter__(self):
        self.start = None
        if STAGE_EVENTS is not None and (STAGE_FILTER is None or self.name in STAGE_FILTER):
            self.start = _event()
            self.start.record()

    def __exit__(self, *exc):
        if self.start is not None and STAGE_EVENTS is not None:
            end = _event()
            end.record()
            STAGE_EVENTS.append((self.name, self.start, end))
        return False


def _lib():
    return L.load()


def _cuda_f32(what, **tensors):
    """CHECK_CUDA only (common.hpp:25-27): device fp32 tensors of any stride; returns them made contiguous, which is what
    the reference's hosts that call `.contiguous()` themselves do (structural_similarity.cu:341-357)."""
    out = []
    for k, t in tensors.items():
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(f"{what}: {k} must be a Tensor")
        if not t.is_cuda:
            raise RuntimeError(f"{what}: {k} must be a CUDA tensor")
        L.require_dtype(what, k, t, torch.float32)
        out.append(t.contiguous())
    return out


def _f32(what, **tensors):
    L.require_cuda(what, **tensors)
    for k, t in tensors.items():
        if t is not None:
            L.require_dtype(what, k, t, torch.float32)


_DTYPE_CODES = {torch.float32: 0, torch.float64: 1, torch.float16: 2}  # FSGS_DTYPE_* of the `_typed` entry points


def _same_float(what, allowed, **tensors):
    """The selector of the tensors' common element type; all of them must be on the GPU, contiguous, of one of the
    `allowed` floating types (the ones the reference dispatches this operator on) and agree with each other."""
    L.require_cuda(what, **tensors)
    first = next(iter(tensors.values()))
    if first.dtype not in allowed:
        raise RuntimeError(f'{what}: element type {first.dtype} is not supported (expected one of '
                           f'{", ".join(str(d) for d in allowed)})')
    for k, t in tensors.items():
        L.require_dtype(what, k, t, first.dtype)
    return _DTYPE_CODES[first.dtype]


_FLOAT_DOUBLE = (torch.float32, torch.float64)
_FLOAT_DOUBLE_HALF = (torch.float32, torch.float64, torch.float16)

_PINNED = threading.local()


def _pinned_count() -> Tensor:
    """A page-locked int64 the binning's instance count is copied into, one per host thread (a binning call waits for
    its count before it returns, so a thread never has two in flight): a device-to-host copy into pinned memory is a
    direct transfer, into pageable memory it is staged by the runtime (about 25 us more per call)."""
    if getattr(_PINNED, 'count', None) is None:
        _PINNED.count = torch.zeros(1, dtype=torch.int64, pin_memory=True)
    return _PINNED.count


def _workspace(nbytes: int, device) -> Tensor:
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


# --------------------------------------------------------------------------------------------------------------------
def gs_2d_preprocess_forward(W: int, H: int, sh_degree: int, is_opengl: bool, means3D: Tensor, scales: Tensor,
                             rotations: Tensor, opacities: Tensor, shs: Tensor, sh_rest: Optional[Tensor],
                             Tw2v: Tensor, Tv2c: Tensor, cam_pos: Tensor, trans_precomp: Optional[Tensor] = None,
                             means2D: Optional[Tensor] = None, culling: Optional[Tensor] = None,
                             return_records: bool = False, return_masks: bool = False) -> List[Tensor]:
    """gs_2d_preprocess.cu:331-421 -> [means2D, colors, trans_mat, normal_opacity, depths, radii, tiles_touched]
    (+ records[P,20], the packed per-surfel record of gs_2d_pack_records written by the same kernel, on request;
    + keep_masks[P] int32, the per-surfel tile masks of the culled binning, GS_prepare(..., cull=True), on request)."""
    what = 'gs_2d_preprocess_forward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, opacities=opacities, shs=shs, Tw2v=Tw2v,
         Tv2c=Tv2c, cam_pos=cam_pos)
    if means3D.ndim != 2 or means3D.shape[-1] != 3:
        raise RuntimeError('Error shape for means3D')
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.numel() > 0
    M = 0
    if has_rest:
        _f32(what, sh_rest=sh_rest)
        if not (sh_rest.ndim == 3 and sh_rest.shape[0] == P and sh_rest.shape[1] >= (1 + sh_degree) ** 2 - 1
                and sh_rest.shape[2] == 3):
            raise RuntimeError('Error shape for sh features')
        M = sh_rest.shape[1]
    elif sh_degree >= 0:
        if not (shs.ndim == 3 and shs.shape[0] == P and shs.shape[1] >= (1 + sh_degree) ** 2 and shs.shape[2] == 3):
            raise RuntimeError('Error shape for sh features')
        M = shs.shape[1]
    if means2D is not None:
        _f32(what, means2D=means2D)
        L.require_shape(what, 'means2D', means2D, P, 2)
    if culling is not None:
        L.require_cuda(what, culling=culling)
        L.require_dtype(what, 'culling', culling, torch.bool)
        L.require_shape(what, 'culling', culling, P)
    if trans_precomp is not None:
        _f32(what, trans_precomp=trans_precomp)
    L.require_shape(what, 'scales', scales, P, 2)
    L.require_shape(what, 'rotations', rotations, P, 4)
    L.require_shape(what, 'opacities', opacities, P, 1)
    L.require_shape(what, 'Tw2v', Tw2v, 4, 4)
    L.require_shape(what, 'Tv2c', Tv2c, 4, 4)
    L.require_shape(what, 'cam_pos', cam_pos, 3)
    if sh_degree < 0:
        L.require_shape(what, 'shs', shs, P, 3)

    opt = dict(dtype=torch.float32, device=means3D.device)
    colors = shs if sh_degree < 0 else torch.empty((P, 3), **opt)
    trans_mat = trans_precomp if trans_precomp is not None else torch.empty((P, 3, 3), **opt)
    preserve = means2D is not None
    means2D_ = means2D if preserve else torch.empty((P, 2), **opt)
    depths = torch.empty((P,), **opt)
    radii = torch.empty((P,), dtype=torch.int32, device=means3D.device)
    tiles_touched = torch.empty((P,), dtype=torch.int32, device=means3D.device)
    normal_opacity = torch.empty((P, 4), **opt)
    records = torch.empty((P, 20), **opt) if return_records else None
    masks = torch.empty((max(P, 1),), dtype=torch.int32, device=means3D.device) if return_masks else None
    with _timed('gs_2d_preprocess_forward'):
        rc = _lib().fsgs_gs_2d_preprocess_forward(
            P, W, H, sh_degree, M, L.ptr(means3D), L.ptr(scales), L.ptr(rotations), L.ptr(opacities), L.ptr(shs),
            L.ptr(sh_rest) if has_rest else None, L.ptr(Tw2v), L.ptr(Tv2c), L.ptr(cam_pos), L.ptr(trans_precomp),
            L.ptr(culling), int(preserve), L.ptr(means2D_), None if sh_degree < 0 else L.ptr(colors),
            None if trans_precomp is not None else L.ptr(trans_mat), L.ptr(normal_opacity), L.ptr(depths), L.ptr(radii),
            L.ptr(tiles_touched), L.ptr(records), L.ptr(masks), L.current_stream())
    L.check(rc, what)
    out = [means2D_, colors, trans_mat, normal_opacity, depths, radii, tiles_touched]
    if return_records:
        out.append(records)
    if return_masks:
        out.append(masks)
    return out


def gs_2d_preprocess_backward(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs, sh_rest,
                              Tw2v, Tv2c, cam_pos, trans_mat, radii, colors, normal_opacity,
                              grad_mean2D, grad_trans, grad_depth, grad_colors, grad_normals,
                              grad_means3D, grad_scales, grad_rotations, grad_opacities, grad_shs, grad_sh_rest,
                              grad_Tw2v=None, grad_campos=None) -> None:
    """gs_2d_preprocess.cu:423-499: fills the caller's zeroed grad_* tensors in place and overwrites grad_mean2D."""
    what = 'gs_2d_preprocess_backward'
    _f32(what, grad_mean2D=grad_mean2D, grad_colors=grad_colors, grad_normals=grad_normals,
         grad_means3D=grad_means3D, grad_trans=grad_trans, grad_scales=grad_scales, grad_rotations=grad_rotations,
         grad_opacities=grad_opacities, grad_shs=grad_shs, grad_sh_rest=grad_sh_rest)
    if grad_shs is not None and colors is None:
        raise RuntimeError('shs and clamped must not be None when need grad_shs')
    has_rest = sh_rest is not None and sh_rest.numel() > 0
    P = means3D.shape[0]
    M = sh_rest.shape[1] if has_rest else (shs.shape[1] if shs.ndim == 3 else 0)
    L.require_shape(what, 'grad_means3D', grad_means3D, P, 3)
    # optional in the reference (torch::optional, gs_2d_preprocess.cu:436, :447-448, :489-490): computed and dropped
    if grad_scales is None:
        grad_scales = torch.empty((P, 2), dtype=torch.float32, device=means3D.device)
    if grad_rotations is None:
        grad_rotations = torch.empty((P, 4), dtype=torch.float32, device=means3D.device)
    L.require_shape(what, 'grad_scales', grad_scales, P, 2)
    L.require_shape(what, 'grad_rotations', grad_rotations, P, 4)
    L.require_shape(what, 'grad_opacities', grad_opacities, P, 1)
    with _timed('gs_2d_preprocess_backward'):
        rc = _lib().fsgs_gs_2d_preprocess_backward(
            P, W, H, sh_degree, M, L.ptr(means3D), L.ptr(scales), L.ptr(rotations), L.ptr(shs),
            L.ptr(sh_rest) if has_rest else None, L.ptr(Tw2v), L.ptr(Tv2c), L.ptr(cam_pos), L.ptr(trans_mat),
            L.ptr(radii), L.ptr(colors), L.ptr(grad_mean2D), L.ptr(grad_trans), L.ptr(grad_colors), L.ptr(grad_normals),
            L.ptr(grad_means3D), L.ptr(grad_scales), L.ptr(grad_rotations), L.ptr(grad_opacities), L.ptr(grad_shs),
            L.ptr(grad_sh_rest) if has_rest else None, L.current_stream())
    L.check(rc, what)


def gs_2d_compute_transmat_forward(W, H, means3D, scales, rotations, Tw2v, Tw2c) -> Tuple[Tensor, Tensor]:
    """gs_2d_preprocess.cu:512-550 -> (trans_mat[P,3,3], normals[P,3])."""
    what = 'gs_2d_compute_transmat_forward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, Tw2v=Tw2v, Tw2c=Tw2c)
    P = means3D.shape[0]
    L.require_shape(what, 'means3D', means3D, P, 3)
    L.require_shape(what, 'scales', scales, P, 2)
    L.require_shape(what, 'rotations', rotations, P, 4)
    L.require_shape(what, 'Tw2v', Tw2v, 4, 4)
    L.require_shape(what, 'Tw2c', Tw2c, 4, 4)
    trans_mat = torch.empty((P, 3, 3), dtype=torch.float32, device=means3D.device)
    normals = torch.empty((P, 3), dtype=torch.float32, device=means3D.device)
    with _timed('gs_2d_compute_transmat_forward'):
        rc = _lib().fsgs_gs_2d_compute_transmat_forward(P, W, H, L.ptr(means3D), L.ptr(scales), L.ptr(rotations),
                                                        L.ptr(Tw2v), L.ptr(Tw2c), L.ptr(trans_mat), L.ptr(normals),
                                                        L.current_stream())
    L.check(rc, what)
    return trans_mat, normals


def gs_2d_compute_trans_mat_backward(W, H, means3D, scales, rotations, Tw2v, Tw2c, grad_matrix,
                                     grad_normals) -> List[Tensor]:
    """gs_2d_preprocess.cu:564-599 -> [grad_means3D, grad_scales, grad_rotations]."""
    what = 'gs_2d_compute_trans_mat_backward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, Tw2v=Tw2v, Tw2c=Tw2c, grad_matrix=grad_matrix,
         grad_normals=grad_normals)
    P = means3D.shape[0]
    L.require_shape(what, 'grad_matrix', grad_matrix, P, 3, 3)
    L.require_shape(what, 'grad_normals', grad_normals, P, 3)
    g_means3D = torch.empty((P, 3), dtype=torch.float32, device=means3D.device)
    g_scales = torch.empty((P, 2), dtype=torch.float32, device=means3D.device)
    g_rot = torch.empty((P, 4), dtype=torch.float32, device=means3D.device)
    with _timed('gs_2d_compute_transmat_backward'):
        rc = _lib().fsgs_gs_2d_compute_transmat_backward(P, W, H, L.ptr(means3D), L.ptr(scales), L.ptr(rotations),
                                                         L.ptr(Tw2v), L.ptr(Tw2c), L.ptr(grad_matrix),
                                                         L.ptr(grad_normals), L.ptr(g_means3D), L.ptr(g_scales),
                                                         L.ptr(g_rot), L.current_stream())
    L.check(rc, what)
    return [g_means3D, g_scales, g_rot]


# --------------------------------------------------------------------------------------------------------------------
def GS_prepare(W: int, H: int, means2D: Tensor, depths: Tensor, radii: Tensor, tiles_touched: Tensor,
               debug: bool = False, return_keys: bool = False, return_offsets: bool = False,
               overlap=None, records: Optional[Tensor] = None, cull: bool = False,
               keep_masks: Optional[Tensor] = None, store_offsets: bool = True) -> List[Tensor]:
    """gaussian_prepare.cu:282-308 -> [ranges[T,2] int64, point_list[R] int32] (+ sorted keys, + the prefix scan of
    tiles_touched, which GS_2D_render_backward can use to sum gradients without atomics). `overlap(offsets)`, if given,
    is called once the scan is queued and before the host waits for the instance count; its result is appended.
    `records` (gs_2d_preprocess_forward(..., return_records=True)): the scan stores every surfel's offset into its record
    unless `store_offsets` is False (the blend backward then takes the offsets from the scan's own output: 3.5 us less
    in the scan, but a 64-byte line more per list entry in the backward's gather, 84 MB at 300k surfels / 800x800).
    `cull` (needs `records`, or the `keep_masks` the preprocess wrote; no counterpart in the reference): instances that no pixel of their tile can blend are left
    out of the lists -- same images and gradients from shorter lists; point_list keeps its length R, the entries behind
    the last tile's end are unused, n_contrib counts positions of the shorter lists. The per-surfel keep masks [P] int32
    are appended to the result; GS_2D_render_backward must get them (`culled=masks`) when it sums ordered records."""
    what = 'GS_prepare'
    _f32(what, means2D=means2D, depths=depths)
    L.require_cuda(what, radii=radii, tiles_touched=tiles_touched)
    L.require_dtype(what, 'radii', radii, torch.int32)
    L.require_dtype(what, 'tiles_touched', tiles_touched, torch.int32)
    P = means2D.shape[0]
    dev = means2D.device
    if records is not None:
        _f32(what, records=records)
        L.require_shape(what, 'records', records, P, 20)
    if cull and records is None and keep_masks is None:
        raise RuntimeError(f'{what}: cull needs the packed records or the keep masks')
    lib = _lib()
    stream = L.current_stream()
    masks = keep_masks
    if masks is not None:
        L.require_cuda(what, keep_masks=masks)
        L.require_dtype(what, 'keep_masks', masks, torch.int32)
        L.require_shape(what, 'keep_masks', masks, max(P, 1))
    if cull and masks is None:
        masks = torch.empty((max(P, 1),), dtype=torch.int32, device=dev)
        with _timed('gs_prepare_fill'):
            rc = lib.fsgs_gs_2d_cull_masks(P, W, H, L.ptr(records), L.ptr(radii), L.ptr(masks), stream)
        L.check(rc, what)
    T = ((W + _TILE - 1) // _TILE) * ((H + _TILE - 1) // _TILE)
    ranges = torch.empty((T, 2), dtype=torch.int64, device=dev)
    offsets = torch.empty((max(P, 1),), dtype=torch.int64, device=dev)
    ws1 = _workspace(lib.fsgs_gs_prepare_scan_workspace_bytes(P), dev)
    bins = _workspace(lib.fsgs_gs_prepare_bins_bytes(P, W, H), dev)
    count = _pinned_count()
    # The host has to learn the instance count before it can size point_list. Everything that does not depend on it is
    # queued behind the count's copy first -- the per-tile counting, and whatever the caller hands in as `overlap` -- so
    # the device works while the host waits for the copy and allocates.
    with _timed('gs_prepare_scan'):
        rc = lib.fsgs_gs_prepare_scan_begin(P, L.ptr(tiles_touched), L.ptr(offsets), L.ptr(ws1), ws1.numel(),
                                            count.data_ptr(), L.ptr(records) if store_offsets else None, stream)
    L.check(rc, what)
    with _timed('gs_prepare_fill'):  # first of the operator's two parts: callers that time stages add them up
        if cull:
            rc = lib.fsgs_gs_prepare_count_culled(P, W, H, L.ptr(means2D), L.ptr(radii), L.ptr(masks), L.ptr(ranges),
                                                  L.ptr(bins), bins.numel(), stream)
        else:
            rc = lib.fsgs_gs_prepare_count(P, W, H, L.ptr(means2D), L.ptr(radii), L.ptr(ranges), L.ptr(bins),
                                           bins.numel(), stream)
    L.check(rc, what)
    overlapped = overlap(offsets) if overlap is not None else None
    L.check(lib.fsgs_gs_prepare_scan_end(), what)
    R = ctypes.c_int64.from_address(count.data_ptr()).value
    point_list = torch.empty((R,), dtype=torch.int32, device=dev)
    keys = torch.empty((R,), dtype=torch.int64, device=dev) if return_keys else None
    ws2 = _workspace(lib.fsgs_gs_prepare_fill_workspace_bytes(R), dev)
    with _timed('gs_prepare_fill'):
        if cull:
            rc = lib.fsgs_gs_prepare_fill_counted_culled(P, W, H, L.ptr(means2D), L.ptr(depths), L.ptr(radii),
                                                         L.ptr(masks), R, L.ptr(ranges), L.ptr(point_list),
                                                         L.ptr(keys), L.ptr(bins), bins.numel(), L.ptr(ws2),
                                                         ws2.numel(), stream)
        else:
            rc = lib.fsgs_gs_prepare_fill_counted(P, W, H, L.ptr(means2D), L.ptr(depths), L.ptr(radii), R,
                                                  L.ptr(ranges), L.ptr(point_list), L.ptr(keys), L.ptr(bins),
                                                  bins.numel(), L.ptr(ws2), ws2.numel(), stream)
    L.check(rc, what)
    if debug:
        torch.cuda.synchronize()
    out = [ranges, point_list]
    if return_keys:
        out.append(keys)
    if return_offsets:
        out.append(offsets)
    if overlap is not None:
        out.append(overlapped)
    if cull:
        out.append(masks)
    return out


# --------------------------------------------------------------------------------------------------------------------
def GS_2D_render_forward(width: int, height: int, means2D: Tensor, colors: Tensor, normal_opacity: Tensor,
                         trans_mat: Tensor, point_list: Tensor, ranges: Tensor, near_n: float, far_n: float,
                         only_image: bool, trans_mat_t2: Optional[Tensor] = None,
                         accum_max_count: Optional[Tensor] = None, accum_weights_p: Optional[Tensor] = None,
                         accum_weights_count: Optional[Tensor] = None, records: Optional[Tensor] = None):
    """gs_2d_redner.cu:541-629 -> (colors[3,H,W], opacity[H,W], extras[9,H,W]|None, flow[H,W,2]|None, n_contrib).
    `records` (gs_2d_pack_records) is an optional packed copy of the per-surfel inputs."""
    what = 'GS_2D_render_forward'
    _f32(what, colors=colors, trans_mat=trans_mat, means2D=means2D, normal_opacity=normal_opacity,
         trans_mat_t2=trans_mat_t2, accum_weights_p=accum_weights_p)
    if colors.ndim != 2:
        raise RuntimeError(f'{what}: colors must have 2 dimensions')
    P = colors.shape[0]
    L.require_shape(what, 'trans_mat', trans_mat, P, 3, 3)
    L.require_cuda(what, ranges=ranges, point_list=point_list, accum_max_count=accum_max_count,
                   accum_weights_count=accum_weights_count)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    for name, t, dt in (('accum_max_count', accum_max_count, torch.int32),
                        ('accum_weights_count', accum_weights_count, torch.int32)):
        if t is not None:
            L.require_dtype(what, name, t, dt)
            L.require_shape(what, name, t, P)
    if accum_weights_p is not None:
        L.require_shape(what, 'accum_weights_p', accum_weights_p, P)
    if trans_mat_t2 is not None:
        L.require_shape(what, 'trans_mat_t2', trans_mat_t2, P, 3, 3)
    opt = dict(dtype=torch.float32, device=colors.device)
    pixel_colors = torch.empty((3, height, width), **opt)
    pixel_opacity = torch.empty((height, width), **opt)
    n_contrib = torch.empty((2, height, width), dtype=torch.int32, device=colors.device)
    pixel_extras = None if only_image else torch.empty((9, height, width), **opt)
    pixel_flow = torch.empty((height, width, 2), **opt) if (not only_image and trans_mat_t2 is not None) else None
    with _timed('gs_2d_render_forward'):
        rc = _lib().fsgs_gs_2d_render_forward(
            P, width, height, float(near_n), float(far_n), int(bool(only_image)), L.ptr(means2D), L.ptr(colors),
            L.ptr(normal_opacity), L.ptr(trans_mat), L.ptr(point_list), L.ptr(ranges), L.ptr(trans_mat_t2),
            L.ptr(accum_max_count), L.ptr(accum_weights_p), L.ptr(accum_weights_count), L.ptr(pixel_colors),
            L.ptr(pixel_opacity), L.ptr(pixel_extras), L.ptr(pixel_flow), L.ptr(n_contrib), L.ptr(records),
            L.current_stream())
    L.check(rc, what)
    return pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib


def gs_cull_masks(W: int, H: int, means2D: Tensor, conic_opacity: Tensor, radii: Tensor) -> Tensor:
    """-> keep_masks[P] int32 for 3D Gaussians (no reference counterpart): a bit per tile of a Gaussian's rectangle, set
    when some pixel of the tile can reach alpha >= 1/255; `GS_prepare(..., cull=True, keep_masks=...)` leaves the other
    (Gaussian, tile) instances out of the tile lists, and `gaussian_rasterize_backward(..., culled=...)` must get the
    masks when it sums ordered records."""
    what = 'gs_cull_masks'
    _f32(what, means2D=means2D, conic_opacity=conic_opacity)
    L.require_cuda(what, radii=radii)
    L.require_dtype(what, 'radii', radii, torch.int32)
    P = means2D.shape[0]
    L.require_shape(what, 'means2D', means2D, P, 2)
    L.require_shape(what, 'conic_opacity', conic_opacity, P, 4)
    L.require_shape(what, 'radii', radii, P)
    masks = torch.empty((max(P, 1),), dtype=torch.int32, device=means2D.device)
    with _timed(what):
        rc = _lib().fsgs_gs_cull_masks(P, W, H, L.ptr(means2D.contiguous()), L.ptr(conic_opacity.contiguous()),
                                       L.ptr(radii.contiguous()), L.ptr(masks), L.current_stream())
    L.check(rc, what)
    return masks


def gs_2d_pack_records(means2D: Tensor, colors: Tensor, normal_opacity: Tensor, trans_mat: Tensor,
                       radii: Optional[Tensor] = None, point_offsets: Optional[Tensor] = None) -> Tensor:
    """-> records[P,20]: one 80-byte record per surfel with everything the blend kernels gather (no reference
    counterpart; optional input of GS_2D_render_forward / GS_2D_render_backward)."""
    what = 'gs_2d_pack_records'
    _f32(what, means2D=means2D, colors=colors, normal_opacity=normal_opacity, trans_mat=trans_mat)
    L.require_cuda(what, radii=radii, point_offsets=point_offsets)
    P = means2D.shape[0]
    L.require_shape(what, 'colors', colors, P, 3)
    L.require_shape(what, 'normal_opacity', normal_opacity, P, 4)
    L.require_shape(what, 'trans_mat', trans_mat, P, 3, 3)
    if radii is not None:
        L.require_dtype(what, 'radii', radii, torch.int32)
    if point_offsets is not None:
        L.require_dtype(what, 'point_offsets', point_offsets, torch.int64)
    records = torch.empty((P, 20), dtype=torch.float32, device=means2D.device)
    with _timed(what):
        rc = _lib().fsgs_gs_2d_pack_records(P, L.ptr(means2D.contiguous()), L.ptr(colors.contiguous()),
                                            L.ptr(normal_opacity.contiguous()), L.ptr(trans_mat.contiguous()),
                                            L.ptr(radii), L.ptr(point_offsets), L.ptr(records), L.current_stream())
    L.check(rc, what)
    return records


def GS_2D_render_backward(means2D, normal_opacity, colors, trans_mat, trans_mat2, out_opacity, out_others, out_flows,
                          dL_dout_color, dL_dout_opacity, dL_dothers, dL_dout_flows, ranges, point_list, n_contrib,
                          near_n: float, far_n: float, point_offsets: Optional[Tensor] = None,
                          radii: Optional[Tensor] = None, records: Optional[Tensor] = None,
                          culled: Optional[Tensor] = None):
    """gs_2d_redner.cu:631-717 -> (dL_dcolors[P,3], dL_dmeans2D[P,2], dL_dtrans_m[P,3,3], dL_dnorm_op[P,4]).
    With `point_offsets` (GS_prepare(..., return_offsets=True)) and `radii` the per-surfel sums are taken in a fixed
    order from per-instance records instead of with atomics. `culled`: the keep masks GS_prepare(..., cull=True) returned
    with these lists."""
    what = 'GS_2D_render_backward'
    L.require_cuda(what, dL_dout_color=dL_dout_color, dL_dout_opacity=dL_dout_opacity, dL_dothers=dL_dothers,
                   dL_dout_flows=dL_dout_flows, point_offsets=point_offsets, radii=radii)
    P = means2D.shape[0]
    H, W = dL_dout_color.shape[1], dL_dout_color.shape[2]
    R = int(point_list.numel())
    opt = dict(dtype=torch.float32, device=out_opacity.device)
    ordered = point_offsets is not None and P > 0
    if ordered and radii is None:
        raise RuntimeError(f'{what}: radii is required together with point_offsets')
    # the four outputs share one allocation; every segment starts on a 16-byte boundary. The atomic path accumulates
    # into them (one zero-fill), the ordered path writes every row itself.
    up = lambda n: (n + 3) // 4 * 4
    o1, o2, o3 = up(4 * P), up(4 * P) + up(9 * P), up(4 * P) + up(9 * P) + up(3 * P)
    flat = (torch.empty if ordered else torch.zeros)((o3 + 2 * P,), **opt)
    g_norm_op = flat[:4 * P].view(P, 4)
    g_trans = flat[o1:o1 + 9 * P].view(P, 3, 3)
    g_colors = flat[o2:o2 + 3 * P].view(P, 3)
    g_means2D = flat[o3:o3 + 2 * P].view(P, 2)
    if P == 0:
        return g_colors, g_means2D, g_trans, g_norm_op
    c = lambda t: None if t is None else t.contiguous()
    means2D, normal_opacity, colors, out_opacity = c(means2D), c(normal_opacity), c(colors), c(out_opacity)
    trans_mat, trans_mat2 = c(trans_mat), c(trans_mat2)
    if records is not None:
        L.require_cuda(what, records=records)
        L.require_dtype(what, 'records', records, torch.float32)
        L.require_shape(what, 'records', records, P, 20)
    dL_dout_color, dL_dout_opacity, dL_dothers, dL_dout_flows = (c(dL_dout_color), c(dL_dout_opacity),
                                                                c(dL_dothers), c(dL_dout_flows))
    ranges, point_list, n_contrib = c(ranges), c(point_list), c(n_contrib)
    use_aux = out_others is not None and dL_dothers is not None
    lib = _lib()
    ws = None
    if ordered:
        L.require_dtype(what, 'point_offsets', point_offsets, torch.int64)
        L.require_dtype(what, 'radii', radii, torch.int32)
        ws = _workspace(lib.fsgs_gs_2d_render_backward_workspace_bytes(R), out_opacity.device)
    if culled is not None:
        L.require_cuda(what, culled=culled)
        L.require_dtype(what, 'culled', culled, torch.int32)
        L.require_shape(what, 'culled', culled, max(P, 1))
    tail = (L.ptr(records), L.current_stream()) if culled is None else (L.ptr(records), L.ptr(culled), L.current_stream())
    with _timed('gs_2d_render_backward'):
        rc = (lib.fsgs_gs_2d_render_backward if culled is None else lib.fsgs_gs_2d_render_backward_culled)(
            P, W, H, float(near_n), float(far_n), L.ptr(means2D), L.ptr(normal_opacity), L.ptr(colors), L.ptr(trans_mat),
            L.ptr(trans_mat2), L.ptr(out_opacity), L.ptr(out_others) if use_aux else None,
            L.ptr(out_flows) if dL_dout_flows is not None else None, L.ptr(dL_dout_color), L.ptr(dL_dout_opacity),
            L.ptr(dL_dothers) if use_aux else None, L.ptr(dL_dout_flows), L.ptr(ranges), L.ptr(point_list),
            L.ptr(n_contrib), L.ptr(g_colors), L.ptr(g_means2D), L.ptr(g_trans), L.ptr(g_norm_op), R,
            L.ptr(point_offsets) if ordered else None, L.ptr(radii) if ordered else None, L.ptr(ws),
            ws.numel() if ws is not None else 0, *tail)
    L.check(rc, what)
    return g_colors, g_means2D, g_trans, g_norm_op


def gs_2d_topk_weights(topk: int, W: int, H: int, near: float, far: float, means2D: Tensor, normal_opacity: Tensor,
                       trans_mat: Tensor, ranges: Tensor, point_list: Tensor) -> Tuple[Tensor, Tensor]:
    """gaussian_topk.cu:230-250 -> (top_indices[H,W,K] int32, top_weights[H,W,K])."""
    what = 'gs_2d_topk_weights'
    _f32(what, means2D=means2D, normal_opacity=normal_opacity, trans_mat=trans_mat)
    L.require_cuda(what, ranges=ranges, point_list=point_list)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    P = means2D.shape[0]
    top_indices = torch.empty((H, W, topk), dtype=torch.int32, device=means2D.device)
    top_weights = torch.empty((H, W, topk), dtype=torch.float32, device=means2D.device)
    with _timed('gs_2d_topk_weights'):
        rc = _lib().fsgs_gs_2d_topk_weights(topk, P, W, H, float(near), float(far), L.ptr(means2D),
                                            L.ptr(normal_opacity), L.ptr(trans_mat), L.ptr(ranges), L.ptr(point_list),
                                            L.ptr(top_indices), L.ptr(top_weights), L.current_stream())
    L.check(rc, what)
    return top_indices, top_weights


# ---- "fast" surfel path ---------------------------------------------------------------------------------------------
def gs_2d_fast_preprocess_forward(W: int, H: int, sh_degree: int, is_opengl: bool, means3D: Tensor, scales: Tensor,
                                  rotations: Tensor, opacities: Tensor, shs: Tensor, sh_rest: Optional[Tensor],
                                  Tw2v: Tensor, Tv2c: Tensor, Tv2s: Tensor, cam_pos: Tensor,
                                  trans_precomp: Optional[Tensor] = None, means2D: Optional[Tensor] = None,
                                  culling: Optional[Tensor] = None, debug: bool = False,
                                  return_keys: bool = False, return_offsets: bool = False,
                                  return_masks: bool = False) -> List[Tensor]:
    """gs_2d_fast_preprocess.cu:611-782 -> [means2D, colors, trans_mat, inverse_m, normal_opacity, depths, radii,
    ranges[T,2] int64, point_list[R] int32] (point_list keeps the -1 padding entries of culled tiles at its tail)
    (+ sorted keys and tiles_touched, + the prefix scan of tiles_touched, which GS_2D_fast_render_backward can use to sum
    gradients without atomics, + keep_masks[P] int32, the corner test's verdicts per surfel that the preprocess kernel
    leaves for the binning, which the ordered sum of GS_2D_fast_render_backward can reuse)."""
    what = 'gs_2d_fast_preprocess_forward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, opacities=opacities, shs=shs, Tw2v=Tw2v,
         Tv2c=Tv2c, Tv2s=Tv2s, cam_pos=cam_pos)
    if means3D.ndim != 2 or means3D.shape[-1] != 3:
        raise RuntimeError('Error shape for means3D')
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.numel() > 0
    M = 0
    if has_rest:
        _f32(what, sh_rest=sh_rest)
        if not (sh_rest.ndim == 3 and sh_rest.shape[0] == P and sh_rest.shape[1] >= (1 + sh_degree) ** 2 - 1
                and sh_rest.shape[2] == 3):
            raise RuntimeError('Error shape for sh features')
        M = sh_rest.shape[1]
    elif sh_degree >= 0:
        if not (shs.ndim == 3 and shs.shape[0] == P and shs.shape[1] >= (1 + sh_degree) ** 2 and shs.shape[2] == 3):
            raise RuntimeError('Error shape for sh features')
        M = shs.shape[1]
    if means2D is not None:
        _f32(what, means2D=means2D)
        L.require_shape(what, 'means2D', means2D, P, 2)
    if culling is not None:
        L.require_cuda(what, culling=culling)
        L.require_dtype(what, 'culling', culling, torch.bool)
        L.require_shape(what, 'culling', culling, P)
    if trans_precomp is not None:
        _f32(what, trans_precomp=trans_precomp)
    L.require_shape(what, 'scales', scales, P, 2)
    L.require_shape(what, 'rotations', rotations, P, 4)
    L.require_shape(what, 'opacities', opacities, P, 1)
    L.require_shape(what, 'Tw2v', Tw2v, 4, 4)
    L.require_shape(what, 'Tv2c', Tv2c, 4, 4)
    L.require_shape(what, 'Tv2s', Tv2s, 3, 3)
    L.require_shape(what, 'cam_pos', cam_pos, 3)
    if sh_degree < 0:
        L.require_shape(what, 'shs', shs, P, 3)

    dev = means3D.device
    opt = dict(dtype=torch.float32, device=dev)
    lib = _lib()
    stream = L.current_stream()
    colors = shs if sh_degree < 0 else torch.empty((P, 3), **opt)
    trans_mat = trans_precomp if trans_precomp is not None else torch.empty((P, 3, 3), **opt)
    inverse_m = torch.empty((P, 3, 3), **opt)
    preserve = means2D is not None
    means2D_ = means2D if preserve else torch.empty((P, 2), **opt)
    depths = torch.empty((P,), **opt)
    radii = torch.empty((P,), dtype=torch.int32, device=dev)
    tiles_touched = torch.empty((P,), dtype=torch.int32, device=dev)
    normal_opacity = torch.empty((P, 4), **opt)
    keep_masks = torch.empty((max(P, 1),), dtype=torch.int32, device=dev)
    with _timed('gs_2d_fast_preprocess_forward'):
        rc = lib.fsgs_gs_2d_fast_preprocess_forward(
            P, W, H, sh_degree, M, L.ptr(means3D), L.ptr(scales), L.ptr(rotations), L.ptr(opacities), L.ptr(shs),
            L.ptr(sh_rest) if has_rest else None, L.ptr(Tw2v), L.ptr(Tv2s), L.ptr(cam_pos), L.ptr(trans_precomp),
            L.ptr(culling), int(preserve), L.ptr(means2D_), None if sh_degree < 0 else L.ptr(colors),
            None if trans_precomp is not None else L.ptr(trans_mat), L.ptr(inverse_m), L.ptr(normal_opacity),
            L.ptr(depths), L.ptr(radii), L.ptr(tiles_touched), L.ptr(keep_masks), stream)
    L.check(rc, what)

    T = ((W + _TILE - 1) // _TILE) * ((H + _TILE - 1) // _TILE)
    ranges = torch.empty((T, 2), dtype=torch.int64, device=dev)
    offsets = torch.empty((max(P, 1),), dtype=torch.int64, device=dev)
    ws1 = _workspace(lib.fsgs_gs_prepare_scan_workspace_bytes(P), dev)
    count = _pinned_count()
    with _timed('gs_prepare_scan'):
        rc = lib.fsgs_gs_prepare_scan(P, L.ptr(tiles_touched), L.ptr(offsets), L.ptr(ws1), ws1.numel(),
                                      count.data_ptr(), stream)
    L.check(rc, what)
    R = ctypes.c_int64.from_address(count.data_ptr()).value
    point_list = torch.empty((R,), dtype=torch.int32, device=dev)
    keys = torch.empty((R,), dtype=torch.int64, device=dev) if return_keys else None
    ws2 = _workspace(lib.fsgs_gs_2d_fast_prepare_fill_workspace_bytes(P, W, H, R), dev)
    with _timed('gs_2d_fast_prepare_fill'):
        rc = lib.fsgs_gs_2d_fast_prepare_fill(P, W, H, L.ptr(means2D_), L.ptr(inverse_m), L.ptr(depths),
                                              L.ptr(opacities), L.ptr(radii), L.ptr(offsets), R, L.ptr(ranges),
                                              L.ptr(point_list), L.ptr(keys), L.ptr(ws2), ws2.numel(),
                                              L.ptr(keep_masks), stream)
    L.check(rc, what)
    if debug:
        torch.cuda.synchronize()
    out = [means2D_, colors, trans_mat, inverse_m, normal_opacity, depths, radii, ranges, point_list]
    if return_keys:
        out += [keys, tiles_touched]
    if return_offsets:
        out.append(offsets)
    if return_masks:
        out.append(keep_masks)
    return out


def gs_2d_fast_preprocess_backward(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs, sh_rest,
                                   Tw2v, Tv2s, cam_pos, trans_mat, radii, colors, normal_opacity,
                                   grad_mean2D, grad_trans, grad_inv_m, grad_depth, grad_colors, grad_normals,
                                   grad_means3D, grad_scales, grad_rotations, grad_opacities, grad_shs, grad_sh_rest,
                                   grad_Tw2v=None, grad_campos=None) -> None:
    """gs_2d_fast_preprocess.cu:784-858: fills the caller's zeroed grad_* tensors in place and overwrites grad_mean2D."""
    what = 'gs_2d_fast_preprocess_backward'
    _f32(what, grad_mean2D=grad_mean2D, grad_colors=grad_colors, grad_normals=grad_normals,
         grad_means3D=grad_means3D, grad_trans=grad_trans, grad_inv_m=grad_inv_m, grad_scales=grad_scales,
         grad_rotations=grad_rotations, grad_opacities=grad_opacities, grad_shs=grad_shs, grad_sh_rest=grad_sh_rest)
    if grad_shs is not None and colors is None:
        raise RuntimeError('shs and clamped must not be None when need grad_shs')
    has_rest = sh_rest is not None and sh_rest.numel() > 0
    P = means3D.shape[0]
    M = sh_rest.shape[1] if has_rest else (shs.shape[1] if shs.ndim == 3 else 0)
    L.require_shape(what, 'grad_means3D', grad_means3D, P, 3)
    # optional in the reference (torch::optional, gs_2d_preprocess.cu:436, :447-448, :489-490): computed and dropped
    if grad_scales is None:
        grad_scales = torch.empty((P, 2), dtype=torch.float32, device=means3D.device)
    if grad_rotations is None:
        grad_rotations = torch.empty((P, 4), dtype=torch.float32, device=means3D.device)
    L.require_shape(what, 'grad_scales', grad_scales, P, 2)
    L.require_shape(what, 'grad_rotations', grad_rotations, P, 4)
    L.require_shape(what, 'grad_opacities', grad_opacities, P, 1)
    L.require_shape(what, 'grad_inv_m', grad_inv_m, P, 3, 3)
    with _timed('gs_2d_fast_preprocess_backward'):
        rc = _lib().fsgs_gs_2d_fast_preprocess_backward(
            P, W, H, sh_degree, M, L.ptr(means3D), L.ptr(scales), L.ptr(rotations), L.ptr(shs),
            L.ptr(sh_rest) if has_rest else None, L.ptr(Tw2v), L.ptr(Tv2s), L.ptr(cam_pos), L.ptr(trans_mat),
            L.ptr(radii), L.ptr(colors), L.ptr(grad_mean2D), L.ptr(grad_trans), L.ptr(grad_inv_m), L.ptr(grad_colors),
            L.ptr(grad_normals), L.ptr(grad_means3D), L.ptr(grad_scales), L.ptr(grad_rotations),
            L.ptr(grad_opacities), L.ptr(grad_shs), L.ptr(grad_sh_rest) if has_rest else None, L.current_stream())
    L.check(rc, what)


def gs_2d_fast_compute_transmat_forward(means3D, scales, rotations, Tw2v, Tv2s) -> Tuple[Tensor, Tensor]:
    """gs_2d_fast_preprocess.cu:871-909 -> (trans_mat[P,3,3], normals[P,3])."""
    what = 'gs_2d_fast_compute_transmat_forward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, Tw2v=Tw2v, Tv2s=Tv2s)
    P = means3D.shape[0]
    L.require_shape(what, 'means3D', means3D, P, 3)
    L.require_shape(what, 'scales', scales, P, 2)
    L.require_shape(what, 'rotations', rotations, P, 4)
    L.require_shape(what, 'Tw2v', Tw2v, 4, 4)
    L.require_shape(what, 'Tv2s', Tv2s, 3, 3)
    trans_mat = torch.empty((P, 3, 3), dtype=torch.float32, device=means3D.device)
    normals = torch.empty((P, 3), dtype=torch.float32, device=means3D.device)
    with _timed(what):
        rc = _lib().fsgs_gs_2d_fast_compute_transmat_forward(P, L.ptr(means3D), L.ptr(scales), L.ptr(rotations),
                                                             L.ptr(Tw2v), L.ptr(Tv2s), L.ptr(trans_mat),
                                                             L.ptr(normals), L.current_stream())
    L.check(rc, what)
    return trans_mat, normals


def gs_2d_fast_compute_trans_mat_backward(means3D, scales, rotations, Tw2v, Tv2s, grad_matrix,
                                          grad_normals) -> List[Tensor]:
    """gs_2d_fast_preprocess.cu:923-960 -> [grad_means3D, grad_scales, grad_rotations]."""
    what = 'gs_2d_fast_compute_trans_mat_backward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, Tw2v=Tw2v, Tv2s=Tv2s, grad_matrix=grad_matrix,
         grad_normals=grad_normals)
    P = means3D.shape[0]
    L.require_shape(what, 'grad_matrix', grad_matrix, P, 3, 3)
    L.require_shape(what, 'grad_normals', grad_normals, P, 3)
    g_means3D = torch.empty((P, 3), dtype=torch.float32, device=means3D.device)
    g_scales = torch.empty((P, 2), dtype=torch.float32, device=means3D.device)
    g_rot = torch.empty((P, 4), dtype=torch.float32, device=means3D.device)
    with _timed(what):
        rc = _lib().fsgs_gs_2d_fast_compute_transmat_backward(P, L.ptr(means3D), L.ptr(scales), L.ptr(rotations),
                                                              L.ptr(Tw2v), L.ptr(Tv2s), L.ptr(grad_matrix),
                                                              L.ptr(grad_normals), L.ptr(g_means3D), L.ptr(g_scales),
                                                              L.ptr(g_rot), L.current_stream())
    L.check(rc, what)
    return [g_means3D, g_scales, g_rot]


def GS_2D_fast_render_forward(width: int, height: int, near_n: float, far_n: float, only_image: bool,
                              means2D: Tensor, colors: Tensor, normal_opacity: Tensor, trans_mat: Tensor,
                              inverse_m: Tensor, point_list: Tensor, ranges: Tensor,
                              trans_mat_t2: Optional[Tensor] = None, accum_max_count: Optional[Tensor] = None,
                              accum_weights_p: Optional[Tensor] = None, accum_weights_count: Optional[Tensor] = None,
                              per_tile_bucket_offset: Optional[Tensor] = None):
    """gs_2d_fast_redner.cu:839-953 -> [colors[3,H,W], opacity[H,W], extras[8,H,W]|None, flow[H,W,2]|None, n_contrib]
    plus [max_contrib, bucket_to_tile, sampled_T, sampled_acc, sampled_aux[B, 8 | 10, 256]] when
    per_tile_bucket_offset is given (10 channels with trans_mat_t2)."""
    what = 'GS_2D_fast_render_forward'
    _f32(what, colors=colors, trans_mat=trans_mat, inverse_m=inverse_m, means2D=means2D,
         normal_opacity=normal_opacity, accum_weights_p=accum_weights_p, trans_mat_t2=trans_mat_t2)
    if colors.ndim != 2:
        raise RuntimeError(f'{what}: colors must have 2 dimensions')
    P = colors.shape[0]
    L.require_shape(what, 'trans_mat', trans_mat, P, 3, 3)
    L.require_shape(what, 'inverse_m', inverse_m, P, 3, 3)
    L.require_cuda(what, ranges=ranges, point_list=point_list, accum_max_count=accum_max_count,
                   accum_weights_count=accum_weights_count, per_tile_bucket_offset=per_tile_bucket_offset)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    for name, t, dt in (('accum_max_count', accum_max_count, torch.int32),
                        ('accum_weights_count', accum_weights_count, torch.int32)):
        if t is not None:
            L.require_dtype(what, name, t, dt)
            L.require_shape(what, name, t, P)
    if accum_weights_p is not None:
        L.require_shape(what, 'accum_weights_p', accum_weights_p, P)
    flow = trans_mat_t2 is not None and not only_image
    if flow:
        L.require_shape(what, 'trans_mat_t2', trans_mat_t2, P, 3, 3)
    dev = colors.device
    opt = dict(dtype=torch.float32, device=dev)
    # one block per tile writes every pixel of every output, empty tiles included
    pixel_colors = torch.empty((3, height, width), **opt)
    pixel_opacity = torch.empty((height, width), **opt)
    n_contrib = torch.empty((2, height, width), dtype=torch.int32, device=dev)
    pixel_extras = None if only_image else torch.empty((8, height, width), **opt)
    pixel_flow = torch.empty((height, width, 2), **opt) if flow else None
    outputs = [pixel_colors, pixel_opacity, pixel_extras, pixel_flow, n_contrib]
    max_contrib = bucket_to_tile = sampled_T = sampled_acc = sampled_aux = None
    fast_bwd = per_tile_bucket_offset is not None
    if fast_bwd:
        L.require_dtype(what, 'per_tile_bucket_offset', per_tile_bucket_offset, torch.int64)
        per_tile_bucket_offset = per_tile_bucket_offset.contiguous()
        B = int(per_tile_bucket_offset.reshape(-1)[-1].item())
        gy, gx = (height + _TILE - 1) // _TILE, (width + _TILE - 1) // _TILE
        max_contrib = torch.zeros((gy, gx), dtype=torch.int32, device=dev)
        nb = max(B, 1)  # keep the base pointers valid when no tile has any entry
        bucket_to_tile = torch.empty((nb,), dtype=torch.int32, device=dev)
        sampled_T = torch.empty((nb, _TILE * _TILE), **opt)
        sampled_acc = torch.empty((nb, 3, _TILE * _TILE), **opt)
        sampled_aux = torch.empty((nb, 10 if flow else 8, _TILE * _TILE), **opt)
        outputs += [max_contrib, bucket_to_tile[:B], sampled_T[:B], sampled_acc[:B], sampled_aux[:B]]
    if P == 0:
        return outputs
    with _timed('gs_2d_fast_render_forward'):
        rc = _lib().fsgs_gs_2d_fast_render_forward(
            P, width, height, float(near_n), float(far_n), int(bool(only_image)), L.ptr(means2D.contiguous()),
            L.ptr(colors.contiguous()), L.ptr(normal_opacity.contiguous()), L.ptr(trans_mat), L.ptr(inverse_m),
            L.ptr(point_list.contiguous()), L.ptr(ranges.contiguous()), L.ptr(trans_mat_t2) if flow else None,
            L.ptr(accum_max_count), L.ptr(accum_weights_p), L.ptr(accum_weights_count),
            L.ptr(per_tile_bucket_offset) if (fast_bwd and not only_image) else None, L.ptr(pixel_colors),
            L.ptr(pixel_opacity), L.ptr(pixel_extras), L.ptr(pixel_flow), L.ptr(n_contrib), L.ptr(max_contrib),
            L.ptr(bucket_to_tile), L.ptr(sampled_T), L.ptr(sampled_acc), L.ptr(sampled_aux), L.current_stream())
    L.check(rc, what)
    return outputs


# GS_2D_fast_render_backward with snapshots: the reference's per-splat kernel instead of the back-to-front one
PER_SPLAT_BACKWARD = False


def GS_2D_fast_render_backward(means2D, normal_opacity, colors, trans_mat, inverse_m, trans_mat2, images, out_opacity,
                               out_others, out_flows, dL_dout_color, dL_dout_opacity, dL_dothers, dL_dout_flow,
                               ranges, point_list, n_contrib, near_n: float, far_n: float,
                               per_tile_bucket_offset=None, bucket_to_tile=None, max_contrib=None, sampled_T=None,
                               sampled_acc=None, sampled_aux=None, point_offsets: Optional[Tensor] = None,
                               radii: Optional[Tensor] = None, per_splat_kernel: Optional[bool] = None,
                               keep_masks: Optional[Tensor] = None):
    """gs_2d_fast_redner.cu:955-1074 -> [dL_dcolors[P,3], dL_dmeans2D[P,2], dL_dtrans_m[P,3,3], dL_dinverse_m[P,3,3],
    dL_dnorm_op[P,4]]. Passing per_tile_bucket_offset selects the per-splat channel set of the reference's second
    kernel; the snapshot tensors themselves are not needed to evaluate it with the back-to-front kernel, which is the
    default (faster here). `per_splat_kernel=True` (default: PER_SPLAT_BACKWARD) runs the reference's per-splat
    decomposition itself from the snapshots (no optical flow in that form). With dL_dout_flow (and trans_mat2,
    out_flows) the optical-flow gradient is added as the reference's kernels add it. With `point_offsets`
    (gs_2d_fast_preprocess_forward(..., return_offsets=True)) and `radii` the per-surfel sums are taken in a fixed order
    from per-instance records instead of with atomics; `keep_masks` (gs_2d_fast_preprocess_forward(...,
    return_masks=True)) spares that sum the corner test it otherwise repeats."""
    what = 'GS_2D_fast_render_backward'
    if per_splat_kernel is None:
        per_splat_kernel = PER_SPLAT_BACKWARD
    L.require_cuda(what, dL_dout_color=dL_dout_color, dL_dout_opacity=dL_dout_opacity, dL_dothers=dL_dothers)
    P = means2D.shape[0]
    H, W = dL_dout_color.shape[1], dL_dout_color.shape[2]
    opt = dict(dtype=torch.float32, device=out_opacity.device)
    ordered, ws, R = _ordered_sum_inputs(what, P, point_list, point_offsets, radii,
                                         'fsgs_gs_2d_fast_render_backward_workspace_bytes', out_opacity.device)
    if keep_masks is not None:
        L.require_cuda(what, keep_masks=keep_masks)
        L.require_dtype(what, 'keep_masks', keep_masks, torch.int32)
        L.require_shape(what, 'keep_masks', keep_masks, max(P, 1))
    masks_ptr = L.ptr(keep_masks) if ordered else None
    new = torch.empty if ordered else torch.zeros  # the ordered path assigns every row, the atomic path accumulates
    g_means2D = new((P, 2), **opt)
    g_norm_op = new((P, 4), **opt)
    g_colors = new((P, 3), **opt)
    g_trans = new((P, 3, 3), **opt)
    g_inv = new((P, 3, 3), **opt)
    if P == 0:
        return [g_colors, g_means2D, g_trans, g_inv, g_norm_op]
    c = lambda t: None if t is None else t.contiguous()
    means2D, normal_opacity, colors, out_opacity = c(means2D), c(normal_opacity), c(colors), c(out_opacity)
    dL_dout_color, dL_dout_opacity, dL_dothers = c(dL_dout_color), c(dL_dout_opacity), c(dL_dothers)
    ranges, point_list, n_contrib, out_others = c(ranges), c(point_list), c(n_contrib), c(out_others)
    use_aux = out_others is not None and dL_dothers is not None
    per_splat = per_tile_bucket_offset is not None
    flow = dL_dout_flow is not None
    if flow:
        if not use_aux or trans_mat2 is None or out_flows is None:
            raise RuntimeError(f'{what}: dL_dout_flow needs trans_mat2, out_flows, out_others and dL_dothers')
        trans_mat2, out_flows, dL_dout_flow = c(trans_mat2), c(out_flows), c(dL_dout_flow)
        _f32(what, trans_mat2=trans_mat2, out_flows=out_flows, dL_dout_flow=dL_dout_flow)
        L.require_shape(what, 'trans_mat2', trans_mat2, P, 3, 3)
        L.require_shape(what, 'out_flows', out_flows, H, W, 2)
        L.require_shape(what, 'dL_dout_flow', dL_dout_flow, H, W, 2)
    if per_splat_kernel and per_splat and not flow:
        snaps = dict(images=images, bucket_to_tile=bucket_to_tile, max_contrib=max_contrib, sampled_T=sampled_T,
                     sampled_acc=sampled_acc)
        if use_aux:
            snaps['sampled_aux'] = sampled_aux
        missing = [k for k, v in snaps.items() if v is None]
        if missing:
            raise RuntimeError(f'{what}: the per-splat kernel needs {", ".join(missing)}')
        B = bucket_to_tile.shape[0]
        T_tiles = ranges.shape[0]
        images, sampled_T, sampled_acc, sampled_aux = c(images), c(sampled_T), c(sampled_acc), c(sampled_aux)
        bucket_to_tile, max_contrib, offsets = c(bucket_to_tile), c(max_contrib), c(per_tile_bucket_offset)
        _f32(what, images=images, sampled_T=sampled_T, sampled_acc=sampled_acc, sampled_aux=sampled_aux)
        L.require_shape(what, 'images', images, 3, H, W)
        L.require_shape(what, 'sampled_T', sampled_T, B, 256)
        L.require_shape(what, 'sampled_acc', sampled_acc, B, 3, 256)
        if use_aux:
            L.require_shape(what, 'sampled_aux', sampled_aux, B, 8, 256)
        for name, t, n, dt in (('bucket_to_tile', bucket_to_tile, B, torch.int32),
                               ('max_contrib', max_contrib, T_tiles, torch.int32),
                               ('per_tile_bucket_offset', offsets, T_tiles, torch.int64)):
            if t.dtype != dt or t.numel() != n:
                raise RuntimeError(f'{what}: {name} must be {dt} with {n} entries')
        with _timed('gs_2d_fast_render_backward'):
            rc = _lib().fsgs_gs_2d_fast_render_bucket_backward(
                P, W, H, float(near_n), float(far_n), B, L.ptr(means2D), L.ptr(normal_opacity), L.ptr(colors),
                L.ptr(trans_mat), L.ptr(inverse_m), L.ptr(images), L.ptr(out_opacity),
                L.ptr(out_others) if use_aux else None, L.ptr(n_contrib), L.ptr(max_contrib), L.ptr(offsets),
                L.ptr(bucket_to_tile), L.ptr(sampled_T), L.ptr(sampled_acc), L.ptr(sampled_aux) if use_aux else None,
                L.ptr(dL_dout_color), L.ptr(dL_dout_opacity), L.ptr(dL_dothers) if use_aux else None, L.ptr(ranges),
                L.ptr(point_list), L.ptr(g_colors), L.ptr(g_means2D), L.ptr(g_trans), L.ptr(g_inv), L.ptr(g_norm_op),
                R, L.ptr(point_offsets) if ordered else None, L.ptr(radii) if ordered else None, L.ptr(ws),
                ws.numel() if ws is not None else 0, masks_ptr, L.current_stream())
        L.check(rc, what)
        return [g_colors, g_means2D, g_trans, g_inv, g_norm_op]
    with _timed('gs_2d_fast_render_backward'):
        rc = _lib().fsgs_gs_2d_fast_render_backward(
            P, W, H, float(near_n), float(far_n), int(per_splat), L.ptr(means2D), L.ptr(normal_opacity), L.ptr(colors),
            L.ptr(trans_mat), L.ptr(inverse_m), L.ptr(trans_mat2) if flow else None, L.ptr(out_opacity),
            L.ptr(out_others) if use_aux else None, L.ptr(out_flows) if flow else None, L.ptr(dL_dout_color),
            L.ptr(dL_dout_opacity), L.ptr(dL_dothers) if use_aux else None, L.ptr(dL_dout_flow) if flow else None,
            L.ptr(ranges), L.ptr(point_list), L.ptr(n_contrib), L.ptr(g_colors), L.ptr(g_means2D), L.ptr(g_trans),
            L.ptr(g_inv), L.ptr(g_norm_op), R, L.ptr(point_offsets) if ordered else None,
            L.ptr(radii) if ordered else None, L.ptr(ws), ws.numel() if ws is not None else 0, masks_ptr,
            L.current_stream())
    L.check(rc, what)
    return [g_colors, g_means2D, g_trans, g_inv, g_norm_op]


# --------------------------------------------------------------------------------------------------------------------
def SH_to_RGB_forward(dir_or_pos: Tensor, campos: Optional[Tensor], sh_features: Tensor, degree: int,
                      clamp: bool) -> Tensor:
    """ops_3d/spherical_harmonics.cu:15-41 -> rgb[P,3]."""
    what = 'SH_to_RGB_forward'
    _f32(what, dir_or_pos=dir_or_pos, campos=campos, sh_features=sh_features)
    if dir_or_pos.ndim != 2 or dir_or_pos.shape[-1] != 3:
        raise RuntimeError('Error shape for dir_or_pos [P, 3]')
    if campos is not None and not (campos.ndim == 1 and campos.numel() == 3):
        raise RuntimeError('Error shape for campos')
    P, F = dir_or_pos.shape[0], sh_features.shape[-2]
    L.require_shape(what, 'sh_features', sh_features, P, F, 3)
    if not (0 <= degree <= 7 and (1 << degree) <= F):
        raise RuntimeError('degree error')
    rgb = torch.empty((P, 3), dtype=torch.float32, device=dir_or_pos.device)
    with _timed('sh_to_rgb_forward'):
        rc = _lib().fsgs_sh_to_rgb_forward(P, F, degree, int(bool(clamp)), L.ptr(dir_or_pos), L.ptr(campos),
                                           L.ptr(sh_features), L.ptr(rgb), L.current_stream())
    L.check(rc, what)
    return rgb


def SH_to_RGB_backward(degree: int, clamp: bool, dir_or_pos: Tensor, campos: Optional[Tensor], sh_features: Tensor,
                       rgb: Tensor, grad_rgb: Tensor, grad_dir: Optional[Tensor], grad_campos: Optional[Tensor],
                       grad_shs: Optional[Tensor]) -> None:
    """ops_3d/spherical_harmonics.cu:68-102: fills grad_dir / grad_shs, accumulates into grad_campos."""
    what = 'SH_to_RGB_backward'
    _f32(what, grad_rgb=grad_rgb, rgb=rgb, grad_dir=grad_dir, grad_shs=grad_shs, grad_campos=grad_campos)
    if grad_dir is not None and grad_dir.shape != dir_or_pos.shape:
        raise RuntimeError('Error shape for grad_dir')
    if grad_shs is not None and grad_shs.shape != sh_features.shape:
        raise RuntimeError('Error shape for grad_shs')
    if grad_campos is not None and grad_campos.shape != campos.shape:
        raise RuntimeError('ERROR shape for grad_campos')
    P, F = dir_or_pos.shape[0], sh_features.shape[-2]
    with _timed('sh_to_rgb_backward'):
        rc = _lib().fsgs_sh_to_rgb_backward(P, F, degree, int(bool(clamp)), L.ptr(dir_or_pos.contiguous()),
                                            L.ptr(campos), L.ptr(sh_features.contiguous()), L.ptr(rgb), L.ptr(grad_rgb),
                                            L.ptr(grad_dir), L.ptr(grad_campos), L.ptr(grad_shs), L.current_stream())
    L.check(rc, what)


def sh_encode_forward(inputs: Tensor, outputs: Tensor, B: int, D: int, C: int) -> None:
    """nerf/shencoder.cu:657-673: outputs[B,(C+1)^2] <- basis values of inputs[B,D][:, :3]."""
    what = 'sh_encode_forward'
    dtype = _same_float(what, _FLOAT_DOUBLE_HALF, inputs=inputs, outputs=outputs)
    with _timed('sh_encode_forward'):
        rc = _lib().fsgs_sh_encode_forward_typed(dtype, B, D, C, L.ptr(inputs), L.ptr(outputs), L.current_stream())
    L.check(rc, what)


def sh_encode_backward(grad: Tensor, inputs: Tensor, B: int, D: int, C: int, grad_inputs: Tensor) -> None:
    """nerf/shencoder.cu:675-691."""
    what = 'sh_encode_backward'
    dtype = _same_float(what, _FLOAT_DOUBLE_HALF, grad=grad, inputs=inputs, grad_inputs=grad_inputs)
    with _timed('sh_encode_backward'):
        rc = _lib().fsgs_sh_encode_backward_typed(dtype, B, D, C, L.ptr(grad), L.ptr(inputs), L.ptr(grad_inputs),
                                                  L.current_stream())
    L.check(rc, what)


def freq_encode_forward(inputs: Tensor, degree: int, include_inputs: bool, scale: float) -> Tensor:
    """nerf/freqencoder.cu:63-81 -> outputs[..., D * (2 * degree + include_inputs)]."""
    what = 'freq_encode_forward'
    dtype = _same_float(what, _FLOAT_DOUBLE, inputs=inputs)
    Din = inputs.shape[-1]
    Dout = Din * (degree * 2 + int(bool(include_inputs)))
    B = inputs.numel() // Din
    out = torch.empty((*inputs.shape[:-1], Dout), dtype=inputs.dtype, device=inputs.device)
    with _timed('freq_encode_forward'):
        rc = _lib().fsgs_freq_encode_forward_typed(dtype, B, Din, degree, int(bool(include_inputs)), float(scale),
                                                   L.ptr(inputs), L.ptr(out), L.current_stream())
    L.check(rc, what)
    return out


def freq_encode_backward(grad: Tensor, outputs: Tensor, degree: int, include_inputs: bool, scale: float) -> Tensor:
    """nerf/freqencoder.cu:83-104 -> grad_inputs."""
    what = 'freq_encode_backward'
    dtype = _same_float(what, _FLOAT_DOUBLE, grad=grad, outputs=outputs)
    if grad.shape != outputs.shape:
        raise RuntimeError(f'{what}: grad must have the shape of outputs')
    Dout = outputs.shape[-1]
    Din = Dout // (degree * 2 + int(bool(include_inputs)))
    B = outputs.numel() // Dout
    gin = torch.empty((*outputs.shape[:-1], Din), dtype=outputs.dtype, device=outputs.device)
    with _timed('freq_encode_backward'):
        rc = _lib().fsgs_freq_encode_backward_typed(dtype, B, Din, degree, int(bool(include_inputs)), float(scale),
                                                    L.ptr(grad), L.ptr(outputs), L.ptr(gin), L.current_stream())
    L.check(rc, what)
    return gin


# --------------------------------------------------------------------------------------------------------------------
def cdist_top(x1: Tensor, x2: Tensor, largest: bool = False) -> List[Tensor]:
    """other/cdist_top.cu:34-84 -> [distance[..., N] (the points' element type), index[..., N] int64]."""
    what = 'cdist_top'
    if x1.device != x2.device:
        raise RuntimeError('x1 and x2 must be same device')
    dtype = _same_float(what, _FLOAT_DOUBLE, x1=x1, x2=x2)
    N, M, D = x1.shape[-2], x2.shape[-2], x1.shape[-1]
    B = x1.numel() // max(N * D, 1)
    if x2.shape[-1] != D:
        raise RuntimeError(f'The dimenstion of point must be {D}')
    if x2.numel() != B * M * D:
        raise RuntimeError('The shape[:-2] of x2 must be same with x1')
    distance = torch.empty(x1.shape[:-1], dtype=x1.dtype, device=x1.device)
    index = torch.empty(x1.shape[:-1], dtype=torch.int64, device=x1.device)
    with _timed('cdist_top_forward'):
        rc = _lib().fsgs_cdist_top_forward_typed(dtype, B, N, M, D, int(bool(largest)), L.ptr(x1), L.ptr(x2),
                                                 L.ptr(distance), L.ptr(index), L.current_stream())
    L.check(rc, what)
    return [distance, index]


def cdist_top_backward(x1: Tensor, x2: Tensor, distance: Tensor, index: Tensor, grad_dist: Tensor) -> List[Tensor]:
    """other/cdist_top.cu:107-154 -> [grad_x1, grad_x2]."""
    what = 'cdist_top_backward'
    dtype = _same_float(what, _FLOAT_DOUBLE, x1=x1, x2=x2, distance=distance, grad_dist=grad_dist)
    L.require_cuda(what, index=index)
    N, D, M = x1.shape[-2], x1.shape[-1], x2.shape[-2]
    B = x1.numel() // max(N * D, 1)
    g1 = torch.zeros_like(x1)
    g2 = torch.zeros_like(x2)
    with _timed('cdist_top_backward'):
        rc = _lib().fsgs_cdist_top_backward_typed(dtype, B, N, M, D, L.ptr(x1), L.ptr(x2), L.ptr(distance),
                                                  L.ptr(index), L.ptr(grad_dist), L.ptr(g1), L.ptr(g2),
                                                  L.current_stream())
    L.check(rc, what)
    return [g1, g2]


def AdamMasksedUpdated(param: Tensor, param_grad: Tensor, exp_avg: Tensor, exp_avg_sq: Tensor, tiles_touched: Tensor,
                       lr: float, b1: float, b2: float, eps: float, N: int, M: int) -> None:
    """other/adam_masked_update.cu:30-35 (name kept as spelled there)."""
    what = 'AdamMasksedUpdated'
    _f32(what, param=param, exp_avg=exp_avg, exp_avg_sq=exp_avg_sq)
    param_grad = param_grad.contiguous()
    tiles_touched = tiles_touched.contiguous()
    L.require_cuda(what, param_grad=param_grad, tiles_touched=tiles_touched)
    L.require_dtype(what, 'tiles_touched', tiles_touched, torch.bool)
    if param.numel() < N * M or tiles_touched.numel() < N:
        raise RuntimeError(f'{what}: tensors are smaller than N x M = {N} x {M}')
    with _timed('adam_masked_update'):
        rc = _lib().fsgs_adam_masked_update(int(N), int(M), L.ptr(tiles_touched), float(lr), float(b1), float(b2),
                                            float(eps), L.ptr(param), L.ptr(param_grad), L.ptr(exp_avg),
                                            L.ptr(exp_avg_sq), L.current_stream())
    L.check(rc, what)


def deform_apply_forward(points: Tensor, d_xyz: Tensor, scales: Tensor, d_scale: Tensor, rotations: Tensor,
                         d_rotation: Tensor, log_scales: bool):
    """network.py:630, :643, :645 in one kernel -> (points + d_xyz, act(scales) + d_scale, normalize(rot + d_rot))."""
    what = 'deform_apply_forward'
    _f32(what, points=points, d_xyz=d_xyz, scales=scales, d_scale=d_scale, rotations=rotations, d_rotation=d_rotation)
    N, S = scales.shape
    for name, t, c in (('points', points, 3), ('d_xyz', d_xyz, 3), ('d_scale', d_scale, S), ('rotations', rotations, 4),
                       ('d_rotation', d_rotation, 4)):
        L.require_shape(what, name, t, N, c)
    out_p, out_s, out_r = torch.empty_like(points), torch.empty_like(scales), torch.empty_like(rotations)
    with _timed(what):
        rc = _lib().fsgs_deform_apply_forward(N, S, int(bool(log_scales)), L.ptr(points), L.ptr(d_xyz), L.ptr(scales),
                                              L.ptr(d_scale), L.ptr(rotations), L.ptr(d_rotation), L.ptr(out_p),
                                              L.ptr(out_s), L.ptr(out_r), L.current_stream())
    L.check(rc, what)
    return out_p, out_s, out_r


def deform_apply_backward(scales: Tensor, rotations: Tensor, d_rotation: Tensor, grad_scales: Optional[Tensor],
                          grad_rot: Tensor, log_scales: bool):
    """-> (g_scales | None, g_rot): the two gradients of `deform_apply_forward` that are not its upstream gradients
    themselves (g_scales only for logarithmic scales)."""
    what = 'deform_apply_backward'
    _f32(what, scales=scales, rotations=rotations, d_rotation=d_rotation, grad_scales=grad_scales, grad_rot=grad_rot)
    N, S = scales.shape
    L.require_shape(what, 'grad_rot', grad_rot, N, 4)
    g_rot = torch.empty_like(rotations)
    g_scales = None
    if log_scales:
        L.require_shape(what, 'grad_scales', grad_scales, N, S)
        g_scales = torch.empty_like(scales)
    with _timed(what):
        rc = _lib().fsgs_deform_apply_backward(N, S, int(bool(log_scales)), L.ptr(scales), L.ptr(rotations),
                                               L.ptr(d_rotation), L.ptr(grad_scales), L.ptr(grad_rot), L.ptr(g_scales),
                                               L.ptr(g_rot), L.current_stream())
    L.check(rc, what)
    return g_scales, g_rot


def AdamMasksedUpdatedMulti(params: List[Tensor], grads: List[Tensor], exp_avgs: List[Tensor],
                            exp_avg_sqs: List[Tensor], tiles_touched: Tensor, lrs: List[float], b1: float, b2: float,
                            epss: List[float], N: int) -> None:
    """`AdamMasksedUpdated` for all parameter tensors [N, ...] of a point set in one launch (the loop of
    sparse_gaussian_adam.py:20-45); bit-identical to the calls one by one."""
    what = 'AdamMasksedUpdatedMulti'
    lib = _lib()
    n = len(params)
    if not (len(grads) == len(exp_avgs) == len(exp_avg_sqs) == len(lrs) == len(epss) == n):
        raise RuntimeError(f'{what}: one gradient, two moments, a rate and an eps per parameter tensor')
    if n > lib.fsgs_adam_masked_update_max_tensors():
        raise RuntimeError(f'{what}: at most {lib.fsgs_adam_masked_update_max_tensors()} tensors per call')
    tiles_touched = tiles_touched.contiguous()
    L.require_cuda(what, tiles_touched=tiles_touched)
    L.require_dtype(what, 'tiles_touched', tiles_touched, torch.bool)
    grads = [g.contiguous() for g in grads]
    Ms = []
    for i, (p_, g, m, v) in enumerate(zip(params, grads, exp_avgs, exp_avg_sqs)):
        _f32(what, **{f'param{i}': p_, f'grad{i}': g, f'exp_avg{i}': m, f'exp_avg_sq{i}': v})
        if N <= 0 or p_.numel() % N or not (g.numel() == m.numel() == v.numel() == p_.numel()):
            raise RuntimeError(f'{what}: tensor {i} is not [N, M] with N = {N}, or its gradient / moments differ in size')
        Ms.append(p_.numel() // N)
    if n == 0 or N == 0:
        return
    if tiles_touched.numel() < N:
        raise RuntimeError(f'{what}: the mask has fewer than N = {N} entries')
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    a_p, a_g, a_m, a_v = ptrs(params), ptrs(grads), ptrs(exp_avgs), ptrs(exp_avg_sqs)
    a_M = (ctypes.c_int64 * n)(*Ms)
    a_lr, a_eps = (ctypes.c_double * n)(*map(float, lrs)), (ctypes.c_double * n)(*map(float, epss))
    with _timed('adam_masked_update'):
        rc = lib.fsgs_adam_masked_update_multi(n, int(N), ctypes.addressof(a_M), L.ptr(tiles_touched),
                                               ctypes.addressof(a_lr), float(b1), float(b2), ctypes.addressof(a_eps),
                                               ctypes.addressof(a_p), ctypes.addressof(a_g), ctypes.addressof(a_m),
                                               ctypes.addressof(a_v), L.current_stream())
    L.check(rc, what)


# --------------------------------------------------------------------------------------------------------------------
def knn_topk(x: Tensor, y: Tensor, K: int) -> Tuple[Tensor, Tensor]:
    """K nearest rows of y[M,D] for each row of x[N,D] -> (dist2[N,K] ascending, index[N,K] int64).
    Stands in for pytorch3d.ops.knn_points at fast_2d_gs/network.py:504 (squared distances, ties -> lower index)."""
    what = 'knn_topk'
    _f32(what, x=x, y=y)
    N, D = x.shape
    M = y.shape[0]
    if y.shape[1] != D:
        raise RuntimeError(f'{what}: feature dimensions differ')
    dist2 = torch.empty((N, K), dtype=torch.float32, device=x.device)
    index = torch.empty((N, K), dtype=torch.int64, device=x.device)
    with _timed('knn_topk'):
        rc = _lib().fsgs_knn_topk(N, M, D, K, L.ptr(x), L.ptr(y), L.ptr(dist2), L.ptr(index), L.current_stream())
    L.check(rc, what)
    return dist2, index


_LBS_WARP = {None: 0, 'none': 0, 'LBS': 1, 'LBS_c': 2}
_LBS_WEIGHT = {'dist': 0, 'kernel': 1, 'weighted_kernel': 1, 'W': 2, 'logits': 2, 'given': 3}


def _lbs_modes(what, warp_method, weight_method, sp_rot, sp_log_radius, sp_weight_logit):
    if weight_method not in _LBS_WEIGHT:
        raise RuntimeError(f'{what}: unknown weight method {weight_method!r} (one of {sorted(_LBS_WEIGHT)})')
    if sp_rot is None:
        warp = 0  # warp() without a local rotation blends the translations only, whatever the method (network.py:563-564)
    else:
        if warp_method not in ('LBS', 'LBS_c'):
            raise RuntimeError(f'{what}: warp method must be LBS or LBS_c when sp_rot is given, got {warp_method!r}')
        warp = _LBS_WARP[warp_method]
    weight = _LBS_WEIGHT[weight_method]
    if weight == 1 and sp_log_radius is None:
        raise RuntimeError(f'{what}: the kernel weights need sp_log_radius')
    if weight_method == 'weighted_kernel' and sp_weight_logit is None:
        raise RuntimeError(f'{what}: weighted_kernel needs sp_weight_logit')
    return warp, weight


def lbs_blend(points: Tensor, sp_points: Tensor, sp_t: Tensor, sp_r: Tensor, sp_s: Optional[Tensor], pair_in: Tensor,
              index: Tensor, temperature: float = 1.0, warp_method: Optional[str] = None,
              sp_rot: Optional[Tensor] = None, weight_method: str = 'dist', sp_log_radius: Optional[Tensor] = None,
              sp_weight_logit: Optional[Tensor] = None):
    """Neighbour weights and warp of fast_2d_gs/network.py:507-517, 545-573 ->
    (d_xyz[N,3], d_rot[N,4], d_scale[N,S]|None, weights[N,K]). `pair_in`[N,K]: squared distances ('dist', 'kernel',
    'weighted_kernel'), gathered logits ('W') or finished weights ('given'). Without `sp_rot` the translations alone are
    blended; with it `warp_method` is 'LBS' or 'LBS_c'."""
    what = 'lbs_blend'
    _f32(what, points=points, sp_points=sp_points, sp_t=sp_t, sp_r=sp_r, sp_s=sp_s, pair_in=pair_in, sp_rot=sp_rot,
         sp_log_radius=sp_log_radius, sp_weight_logit=sp_weight_logit)
    L.require_cuda(what, index=index)
    L.require_dtype(what, 'index', index, torch.int64)
    warp, weight = _lbs_modes(what, warp_method, weight_method, sp_rot, sp_log_radius, sp_weight_logit)
    N, K = pair_in.shape
    M = sp_points.shape[0]
    S = 0 if sp_s is None else sp_s.shape[1]
    L.require_shape(what, 'index', index, N, K)
    L.require_shape(what, 'sp_t', sp_t, M, 3)
    L.require_shape(what, 'sp_r', sp_r, M, 4)
    if sp_rot is not None:
        L.require_shape(what, 'sp_rot', sp_rot, M, 4)
    opt = dict(dtype=torch.float32, device=points.device)
    d_xyz, d_rot = torch.empty((N, 3), **opt), torch.empty((N, 4), **opt)
    d_scale = torch.empty((N, S), **opt) if S else None
    weights = torch.empty((N, K), **opt)
    lib = _lib()
    ws = _workspace(lib.fsgs_lbs_blend_workspace_bytes(M), points.device)
    with _timed('lbs_blend'):
        rc = lib.fsgs_lbs_blend(N, M, K, warp, weight, float(temperature), L.ptr(points), L.ptr(sp_points),
                                L.ptr(sp_t), L.ptr(sp_rot), L.ptr(sp_r), L.ptr(sp_s), S, L.ptr(pair_in), L.ptr(index),
                                L.ptr(sp_log_radius) if weight == 1 else None,
                                L.ptr(sp_weight_logit) if weight == 1 else None, L.ptr(weights), L.ptr(d_xyz),
                                L.ptr(d_rot), L.ptr(d_scale), L.ptr(ws), ws.numel(), L.current_stream())
    L.check(rc, what)
    return d_xyz, d_rot, d_scale, weights


def lbs_blend_backward(points: Tensor, sp_points: Tensor, sp_t: Tensor, sp_r: Tensor, sp_s: Optional[Tensor],
                       pair_in: Tensor, index: Tensor, grad_xyz: Tensor, grad_rot: Tensor,
                       grad_scale: Optional[Tensor], temperature: float = 1.0, warp_method: Optional[str] = None,
                       sp_rot: Optional[Tensor] = None, weight_method: str = 'dist',
                       sp_log_radius: Optional[Tensor] = None, sp_weight_logit: Optional[Tensor] = None,
                       need_points: bool = True):
    """Gradients of `lbs_blend` (what autograd gives for fast_2d_gs/network.py:507-517, 545-573) -> dict with g_points
    [N,3]|None, g_pair[N,K] (gradient of `pair_in`), g_sp_points[M,3], g_sp_t[M,3], g_sp_rot[M,4]|None, g_sp_r[M,4],
    g_sp_s[M,S]|None, g_log_radius[M]|None, g_weight_logit[M]|None."""
    what = 'lbs_blend_backward'
    _f32(what, points=points, sp_points=sp_points, sp_t=sp_t, sp_r=sp_r, sp_s=sp_s, pair_in=pair_in, grad_xyz=grad_xyz,
         grad_rot=grad_rot, grad_scale=grad_scale, sp_rot=sp_rot, sp_log_radius=sp_log_radius,
         sp_weight_logit=sp_weight_logit)
    L.require_cuda(what, index=index)
    L.require_dtype(what, 'index', index, torch.int64)
    warp, weight = _lbs_modes(what, warp_method, weight_method, sp_rot, sp_log_radius, sp_weight_logit)
    N, K = pair_in.shape
    M = sp_points.shape[0]
    S = 0 if sp_s is None else sp_s.shape[1]
    if S and grad_scale is None:
        raise RuntimeError(f'{what}: grad_scale is required when sp_s is given')
    if tuple(grad_xyz.shape) != (N, 3) or tuple(grad_rot.shape) != (N, 4) or tuple(index.shape) != (N, K) or \
            (S and tuple(grad_scale.shape) != (N, S)):
        raise RuntimeError(f'{what}: gradient / index shapes do not match pair_in {tuple(pair_in.shape)}')
    opt = dict(dtype=torch.float32, device=points.device)
    g_points = torch.empty((N, 3), **opt) if need_points else None
    g_pair = torch.empty((N, K), **opt)
    g_sp_points, g_sp_t, g_sp_r = torch.empty((M, 3), **opt), torch.empty((M, 3), **opt), torch.empty((M, 4), **opt)
    g_sp_rot = torch.empty((M, 4), **opt) if warp else None
    g_sp_s = torch.empty((M, S), **opt) if S else None
    g_rad = torch.empty((M,), **opt) if weight == 1 else None
    g_wl = torch.empty((M,), **opt) if weight == 1 and sp_weight_logit is not None else None
    lib = _lib()
    ws = _workspace(lib.fsgs_lbs_blend_backward_workspace_bytes(N, M, S), points.device)
    with _timed('lbs_blend_backward'):
        rc = lib.fsgs_lbs_blend_backward(
            N, M, K, warp, weight, float(temperature), L.ptr(points), L.ptr(sp_points), L.ptr(sp_t), L.ptr(sp_rot),
            L.ptr(sp_r), L.ptr(sp_s), S, L.ptr(pair_in), L.ptr(index), L.ptr(sp_log_radius) if weight == 1 else None,
            L.ptr(sp_weight_logit) if weight == 1 else None, L.ptr(grad_xyz), L.ptr(grad_rot), L.ptr(grad_scale),
            L.ptr(g_points), L.ptr(g_pair), L.ptr(g_sp_points), L.ptr(g_sp_t), L.ptr(g_sp_rot), L.ptr(g_sp_r),
            L.ptr(g_sp_s), L.ptr(g_rad), L.ptr(g_wl), L.ptr(ws), ws.numel(), L.current_stream())
    L.check(rc, what)
    return dict(g_points=g_points, g_pair=g_pair, g_sp_points=g_sp_points, g_sp_t=g_sp_t, g_sp_rot=g_sp_rot,
                g_sp_r=g_sp_r, g_sp_s=g_sp_s, g_log_radius=g_rad, g_weight_logit=g_wl)


def knn_topk_backward(x: Tensor, y: Tensor, index: Tensor, grad_dist2: Tensor, need_x: bool = True):
    """Gradients of `knn_topk`'s squared distances -> (g_x[N,D]|None, g_y[M,D])."""
    what = 'knn_topk_backward'
    _f32(what, x=x, y=y, grad_dist2=grad_dist2)
    L.require_cuda(what, index=index)
    L.require_dtype(what, 'index', index, torch.int64)
    N, D = x.shape
    M = y.shape[0]
    K = index.shape[1]
    if y.shape[1] != D or tuple(index.shape) != (N, K) or tuple(grad_dist2.shape) != (N, K):
        raise RuntimeError(f'{what}: shapes do not match')
    g_x = torch.empty_like(x) if need_x else None
    g_y = torch.empty_like(y)
    lib = _lib()
    ws = _workspace(lib.fsgs_knn_topk_backward_workspace_bytes(N, M, D), x.device)
    with _timed('knn_topk_backward'):
        rc = lib.fsgs_knn_topk_backward(N, M, D, K, L.ptr(x), L.ptr(y), L.ptr(index), L.ptr(grad_dist2), L.ptr(g_x),
                                        L.ptr(g_y), L.ptr(ws), ws.numel(), L.current_stream())
    L.check(rc, what)
    return g_x, g_y


# --------------------------------------------------------------------------------------------------------------------
def mlp_pack_weights(weights: List[Tensor], head_weights: Tensor, skip: int) -> Tensor:
    """bf16 weight buffer of the fused deformation MLP: layer i as a [256][round_up(K_i, 16)] matrix, then the stacked
    heads as [32][256], each in the tile order the matrix cores read (see fsgs_pack_bf16). `weights` are torch.nn.Linear
    weights [256, K_i] in layer order (network.py:1723-1727)."""
    what = 'mlp_pack_weights'
    _f32(what, head_weights=head_weights, **{f'w{i}': w for i, w in enumerate(weights)})
    Din, n_layers = weights[0].shape[1], len(weights)
    lib = _lib()
    total = lib.fsgs_mlp_packed_elems(Din, n_layers, skip)
    packed = torch.empty((total,), dtype=torch.int16, device=weights[0].device)
    off = 0
    stream = L.current_stream()
    for i, w in enumerate(weights):
        K = w.shape[1]
        K_pad = (K + 15) // 16 * 16
        expect = Din if i == 0 else (Din + 256 if i == skip + 1 else 256)
        if w.shape[0] != 256 or K != expect:
            raise RuntimeError(f'{what}: layer {i} weight has shape {tuple(w.shape)}, expected (256, {expect})')
        rc = lib.fsgs_pack_bf16(256, K, 256, K_pad, L.ptr(w), packed.data_ptr() + 2 * off, stream)
        L.check(rc, what)
        off += 256 * K_pad
    n_out, Kh = head_weights.shape
    if n_out > 32 or Kh != 256:
        raise RuntimeError(f'{what}: stacked heads must be [<=32, 256], got {tuple(head_weights.shape)}')
    rc = lib.fsgs_pack_bf16(n_out, Kh, 32, 256, L.ptr(head_weights), packed.data_ptr() + 2 * off, stream)
    L.check(rc, what)
    return packed


def mlp_pack_all(weights: List[Tensor], biases: List[Tensor], head_weights: List[Tensor], head_biases: List[Tensor],
                 skip: int, transposed: bool = True):
    """`mlp_pack_weights` + `mlp_pack_transposed` + the bias and head concatenations in one launch
    -> (packed, packed_t | None, bias[n_layers*256 + n_out], heads_w[n_out, 256])."""
    what = 'mlp_pack_all'
    named = {f'w{i}': w for i, w in enumerate(weights)}
    named.update({f'b{i}': b for i, b in enumerate(biases)})
    named.update({f'hw{i}': w for i, w in enumerate(head_weights)})
    named.update({f'hb{i}': b for i, b in enumerate(head_biases)})
    _f32(what, **named)
    Din, n_layers, n_heads = weights[0].shape[1], len(weights), len(head_weights)
    if len(biases) != n_layers or len(head_biases) != n_heads:
        raise RuntimeError(f'{what}: one bias per weight')
    for i, (w, b) in enumerate(zip(weights, biases)):
        expect = Din if i == 0 else (Din + 256 if i == skip + 1 else 256)
        if tuple(w.shape) != (256, expect) or b.numel() != 256:
            raise RuntimeError(f'{what}: layer {i} has weight {tuple(w.shape)} / bias {tuple(b.shape)}, expected '
                               f'(256, {expect}) / (256,)')
    rows = [w.shape[0] for w in head_weights]
    if sum(rows) > 32 or any(w.shape[1] != 256 for w in head_weights) or \
            any(b.numel() != r for b, r in zip(head_biases, rows)):
        raise RuntimeError(f'{what}: the heads must be [rows, 256] with at most 32 rows together')
    lib, dev = _lib(), weights[0].device
    packed = torch.empty((lib.fsgs_mlp_packed_elems(Din, n_layers, skip),), dtype=torch.int16, device=dev)
    packed_t = torch.empty((max(n_layers - 1, 1), 256, 256), dtype=torch.int16, device=dev) if transposed else None
    bias = torch.empty((n_layers * 256 + sum(rows),), dtype=torch.float32, device=dev)
    heads_w = torch.empty((sum(rows), 256), dtype=torch.float32, device=dev)
    arr = lambda ts: (ctypes.c_void_p * max(len(ts), 1))(*[t.data_ptr() for t in ts])
    a_w, a_b, a_hw, a_hb = arr(weights), arr(biases), arr(head_weights), arr(head_biases)
    a_rows = (ctypes.c_int * max(n_heads, 1))(*rows)
    rc = lib.fsgs_mlp_pack_all(Din, n_layers, skip, ctypes.addressof(a_w), ctypes.addressof(a_b), n_heads,
                               ctypes.addressof(a_hw), ctypes.addressof(a_hb), ctypes.addressof(a_rows), L.ptr(packed),
                               L.ptr(packed_t) if n_layers > 1 else None, L.ptr(bias), L.ptr(heads_w),
                               L.current_stream())
    L.check(rc, what)
    return packed, packed_t, bias, heads_w


def mlp_forward(inputs: Tensor, packed: Tensor, bias: Tensor, n_layers: int, skip: int, n_out: int,
                save: bool = False):
    """Fused n_layers x (Linear(256)+ReLU) + heads forward on the matrix cores (bf16 in, fp32 accumulate);
    network.py:1757-1776. inputs[B,Din] fp32, bias[n_layers*256 + n_out] fp32 -> out[B,n_out] fp32; with `save` also
    the [n_layers,B,256] bf16 (stored as int16) post-ReLU states that `mlp_backward` needs -> (out, saved)."""
    what = 'mlp_forward'
    _f32(what, inputs=inputs, bias=bias)
    L.require_cuda(what, packed=packed)
    B, Din = inputs.shape
    if bias.numel() != n_layers * 256 + n_out:
        raise RuntimeError(f'{what}: bias must have {n_layers * 256 + n_out} elements')
    if packed.numel() != _lib().fsgs_mlp_packed_elems(Din, n_layers, skip):
        raise RuntimeError(f'{what}: packed weight buffer has the wrong size')
    out = torch.empty((B, n_out), dtype=torch.float32, device=inputs.device)
    saved = torch.empty((n_layers, B, 256), dtype=torch.int16, device=inputs.device) if save else None
    with _timed('mlp_forward'):
        rc = _lib().fsgs_mlp_forward(B, Din, 256, n_layers, skip, n_out, L.ptr(inputs),
                                     L.ptr(packed), L.ptr(bias),
                                     L.ptr(out), L.ptr(saved), L.current_stream())
    L.check(rc, what)
    return (out, saved) if save else out


def mlp_pack_transposed(weights: List[Tensor]) -> Tensor:
    """bf16 copy, transposed to [256 in][256 out], of the last 256 input columns of every layer's weight except the
    first: what `mlp_backward` multiplies dZ with. -> int16 [n_layers-1, 256, 256]."""
    what = 'mlp_pack_transposed'
    _f32(what, **{f'w{i}': w for i, w in enumerate(weights)})
    n = len(weights) - 1
    packed_t = torch.empty((max(n, 1), 256, 256), dtype=torch.int16, device=weights[0].device)
    if n > 0:
        src = torch.stack([w[:, -256:].t() for w in weights[1:]]).contiguous()
        rc = _lib().fsgs_pack_bf16(n * 256, 256, n * 256, 256, L.ptr(src), L.ptr(packed_t), L.current_stream())
        L.check(rc, what)
    return packed_t


def mlp_backward(inputs: Tensor, packed_t: Tensor, head_weights: Tensor, saved: Tensor, grad_out: Tensor,
                 n_layers: int, skip: int, return_dz: bool = False):
    """Weight and bias gradients of `mlp_forward` (autograd through nn.Linear / relu in the reference,
    network.py:1757-1776) -> (g_w flat: layers' [256,K_l] back to back then heads [n_out,256]; g_b[n_layers*256+n_out]).
    With `return_dz` also dZ[n_layers,B,256] (bf16): the gradient of every layer's pre-activation, from which a caller
    forms the gradient of the network's input (dZ_0 W_0 + dZ_{skip+1} W_{skip+1}[:, :Din])."""
    what = 'mlp_backward'
    _f32(what, inputs=inputs, head_weights=head_weights, grad_out=grad_out)
    L.require_cuda(what, packed_t=packed_t, saved=saved)
    B, Din = inputs.shape
    n_out = head_weights.shape[0]
    if tuple(saved.shape) != (n_layers, B, 256) or saved.dtype != torch.int16:
        raise RuntimeError(f'{what}: saved must be the int16 [{n_layers},{B},256] tensor mlp_forward(save=True) returned')
    if tuple(grad_out.shape) != (B, n_out) or head_weights.shape[1] != 256:
        raise RuntimeError(f'{what}: grad_out / head_weights shapes do not match')
    if packed_t.numel() < max(n_layers - 1, 1) * 65536:
        raise RuntimeError(f'{what}: packed_t is too small for {n_layers} layers')
    n_w = 256 * Din + (n_layers - 1) * 65536 + 256 * Din + n_out * 256
    g = torch.empty((n_w + n_layers * 256 + n_out,), dtype=torch.float32, device=inputs.device)
    g_w, g_b = g[:n_w], g[n_w:]
    lib = _lib()
    ws = _workspace(lib.fsgs_mlp_backward_workspace_bytes(B, n_layers), inputs.device)
    with _timed('mlp_backward'):
        rc = lib.fsgs_mlp_backward(B, Din, 256, n_layers, skip, n_out, L.ptr(inputs), L.ptr(packed_t),
                                   L.ptr(head_weights), L.ptr(saved), L.ptr(grad_out), L.ptr(g_w), L.ptr(g_b),
                                   L.ptr(ws), ws.numel(), L.current_stream())
    L.check(rc, what)
    if return_dz:
        return g_w, g_b, ws[:n_layers * B * 256 * 2].view(torch.bfloat16).view(n_layers, B, 256)
    return g_w, g_b


# --------------------------------------------------------------------------------------------------------------------
def fusedssim(C1: float, C2: float, img1: Tensor, img2: Tensor, train: bool):
    """structural_similarity.cu:340-363 -> (ssim_map, dm_dmu1, dm_dsigma1_sq, dm_dsigma12), all [B,CH,H,W]; the three
    partial-derivative maps are empty tensors when `train` is false."""
    what = 'fusedssim'
    img1, img2 = _cuda_f32(what, img1=img1, img2=img2)
    if img1.ndim != 4 or img1.shape != img2.shape:
        raise RuntimeError(f'{what}: img1 and img2 must be [B,CH,H,W] tensors of the same shape')
    B, CH, H, W = img1.shape
    ssim_map = torch.empty_like(img1)
    if train:
        d1, d2, d3 = torch.empty_like(img1), torch.empty_like(img1), torch.empty_like(img1)
    else:
        d1 = d2 = d3 = None
    with _timed(what):
        rc = _lib().fsgs_fusedssim_forward(B, CH, H, W, float(C1), float(C2), L.ptr(img1), L.ptr(img2),
                                           L.ptr(ssim_map), L.ptr(d1), L.ptr(d2), L.ptr(d3), L.current_stream())
    L.check(rc, what)
    if not train:
        d1, d2, d3 = (torch.empty(0) for _ in range(3))
    return ssim_map, d1, d2, d3


def fusedssim_backward(C1: float, C2: float, img1: Tensor, img2: Tensor, dL_dmap: Tensor, dm_dmu1: Tensor,
                       dm_dsigma1_sq: Tensor, dm_dsigma12: Tensor) -> Tensor:
    """structural_similarity.cu:365-380 -> dL_dimg1[B,CH,H,W]."""
    what = 'fusedssim_backward'
    img1, img2, dL_dmap, dm_dmu1, dm_dsigma1_sq, dm_dsigma12 = _cuda_f32(
        what, img1=img1, img2=img2, dL_dmap=dL_dmap, dm_dmu1=dm_dmu1, dm_dsigma1_sq=dm_dsigma1_sq,
        dm_dsigma12=dm_dsigma12)
    B, CH, H, W = img1.shape
    for name, t in (('img2', img2), ('dL_dmap', dL_dmap), ('dm_dmu1', dm_dmu1), ('dm_dsigma1_sq', dm_dsigma1_sq),
                    ('dm_dsigma12', dm_dsigma12)):
        L.require_shape(what, name, t, B, CH, H, W)
    grad = torch.empty_like(img1)
    with _timed(what):
        rc = _lib().fsgs_fusedssim_backward(B, CH, H, W, L.ptr(img1), L.ptr(img2), L.ptr(dL_dmap),
                                            L.ptr(dm_dmu1), L.ptr(dm_dsigma1_sq), L.ptr(dm_dsigma12), L.ptr(grad),
                                            L.current_stream())
    L.check(rc, what)
    return grad


def image_loss_forward(C1: float, C2: float, lambda_dssim: float, img: Tensor, target: Tensor, train: bool):
    """(1 - lambda) * L1 + lambda * (1 - mean SSIM) of [B,CH,H,W] images without image-sized intermediates
    (gaussian_splatting.py:321 with losses/ssim.py:24-47) -> (loss[3] = (loss, L1 mean, SSIM mean), dm_dmu1,
    dm_dsigma1_sq, dm_dsigma12); the three maps are None when `train` is false."""
    what = 'image_loss_forward'
    _f32(what, img=img, target=target)
    if img.ndim != 4 or img.shape != target.shape or img.numel() == 0:
        raise RuntimeError(f'{what}: img and target must be non-empty [B,CH,H,W] tensors of the same shape')
    B, CH, H, W = img.shape
    lib = _lib()
    loss = torch.empty((3,), dtype=torch.float32, device=img.device)
    d1, d2, d3 = (torch.empty_like(img) for _ in range(3)) if train else (None, None, None)
    nbytes = lib.fsgs_image_loss_workspace_bytes(B, H, W)
    ws = _workspace(nbytes, img.device)
    with _timed(what):
        rc = lib.fsgs_image_loss_forward(B, CH, H, W, float(C1), float(C2), float(lambda_dssim), L.ptr(img),
                                         L.ptr(target), L.ptr(loss), L.ptr(d1), L.ptr(d2), L.ptr(d3), L.ptr(ws), nbytes,
                                         L.current_stream())
    L.check(rc, what)
    return loss, d1, d2, d3


def image_loss_backward(lambda_dssim: float, img: Tensor, target: Tensor, grad_loss: Tensor, dm_dmu1: Tensor,
                        dm_dsigma1_sq: Tensor, dm_dsigma12: Tensor) -> Tensor:
    """Gradient of `image_loss_forward`'s loss[0] with respect to img; grad_loss is the one-element upstream gradient."""
    what = 'image_loss_backward'
    _f32(what, img=img, target=target, grad_loss=grad_loss, dm_dmu1=dm_dmu1, dm_dsigma1_sq=dm_dsigma1_sq,
         dm_dsigma12=dm_dsigma12)
    B, CH, H, W = img.shape
    for name, t in (('target', target), ('dm_dmu1', dm_dmu1), ('dm_dsigma1_sq', dm_dsigma1_sq),
                    ('dm_dsigma12', dm_dsigma12)):
        L.require_shape(what, name, t, B, CH, H, W)
    if grad_loss.numel() != 1:
        raise RuntimeError(f'{what}: grad_loss must have one element')
    grad = torch.empty_like(img)
    with _timed(what):
        rc = _lib().fsgs_image_loss_backward(B, CH, H, W, float(lambda_dssim), L.ptr(img), L.ptr(target),
                                             L.ptr(grad_loss), L.ptr(dm_dmu1), L.ptr(dm_dsigma1_sq),
                                             L.ptr(dm_dsigma12), L.ptr(grad), L.current_stream())
    L.check(rc, what)
    return grad


# --------------------------------------------------------------------------------------------------------------------
def gs_2d_epilogue_forward(W: int, H: int, depth_ratio: float, Tw2v: Tensor, Tv2c: Tensor, extras: Tensor,
                           opacity: Tensor, images: Optional[Tensor] = None, background: Optional[Tensor] = None):
    """The per-pixel tail of GS_2D_render (renderer/gs_2d_render.py:608-617, helpers :439-470) and, with `images` and
    `background[3]`, the composite of network.py:725-726, in one kernel ->
    (normals[3,H,W], depths[1,H,W], surf_depth[1,H,W], surf_normal[3,H,W], composited[3,H,W]|None)."""
    what = 'gs_2d_epilogue_forward'
    _f32(what, Tw2v=Tw2v, Tv2c=Tv2c, extras=extras, opacity=opacity, images=images, background=background)
    if tuple(extras.shape) != (9, H, W) or opacity.numel() != H * W or Tw2v.numel() != 16 or Tv2c.numel() != 16:
        raise RuntimeError(f'{what}: extras must be [9,{H},{W}], opacity [{H},{W}], the matrices 4x4')
    if (images is None) != (background is None):
        raise RuntimeError(f'{what}: images and background go together')
    if images is not None and (tuple(images.shape) != (3, H, W) or background.numel() != 3):
        raise RuntimeError(f'{what}: images must be [3,{H},{W}] and background [3]')
    opt = dict(dtype=torch.float32, device=extras.device)
    normals, surf_normal = torch.empty((3, H, W), **opt), torch.empty((3, H, W), **opt)
    depths, surf_depth = torch.empty((1, H, W), **opt), torch.empty((1, H, W), **opt)
    comp = torch.empty((3, H, W), **opt) if images is not None else None
    with _timed('gs_2d_epilogue_forward'):
        rc = _lib().fsgs_gs_2d_epilogue_forward(W, H, float(depth_ratio), L.ptr(Tw2v), L.ptr(Tv2c), L.ptr(extras),
                                                L.ptr(opacity), L.ptr(images), L.ptr(background), L.ptr(normals),
                                                L.ptr(depths), L.ptr(surf_depth), L.ptr(surf_normal), L.ptr(comp),
                                                L.current_stream())
    L.check(rc, what)
    return normals, depths, surf_depth, surf_normal, comp


def gs_2d_epilogue_backward(W: int, H: int, depth_ratio: float, Tw2v: Tensor, Tv2c: Tensor, extras: Tensor,
                            opacity: Tensor, background: Optional[Tensor], g_normals: Optional[Tensor],
                            g_depths: Optional[Tensor], g_surf_depth: Optional[Tensor], g_surf_normal: Optional[Tensor],
                            g_distortion: Optional[Tensor], g_composited: Optional[Tensor]):
    """Backward of `gs_2d_epilogue_forward` -> (g_extras[9,H,W], g_opacity[H,W]|None). The gradient of `images` is
    g_composited itself; the opacity only receives the composite's term (it is detached in surf_normal)."""
    what = 'gs_2d_epilogue_backward'
    grads = dict(g_normals=g_normals, g_depths=g_depths, g_surf_depth=g_surf_depth, g_surf_normal=g_surf_normal,
                 g_distortion=g_distortion, g_composited=g_composited)
    _f32(what, Tw2v=Tw2v, Tv2c=Tv2c, extras=extras, opacity=opacity, background=background, **grads)
    if tuple(extras.shape) != (9, H, W) or opacity.numel() != H * W:
        raise RuntimeError(f'{what}: extras must be [9,{H},{W}] and opacity [{H},{W}]')
    for k, (t, c) in dict(g_normals=(g_normals, 3), g_depths=(g_depths, 1), g_surf_depth=(g_surf_depth, 1),
                          g_surf_normal=(g_surf_normal, 3), g_distortion=(g_distortion, 1),
                          g_composited=(g_composited, 3)).items():
        if t is not None and t.numel() != c * H * W:
            raise RuntimeError(f'{what}: {k} must have {c} x {H} x {W} elements')
    if g_composited is not None and background is None:
        raise RuntimeError(f'{what}: g_composited needs the background')
    g_extras = torch.empty_like(extras)
    g_opacity = torch.empty((H, W), dtype=torch.float32, device=extras.device) if g_composited is not None else None
    with _timed('gs_2d_epilogue_backward'):
        rc = _lib().fsgs_gs_2d_epilogue_backward(
            W, H, float(depth_ratio), L.ptr(Tw2v), L.ptr(Tv2c), L.ptr(extras), L.ptr(opacity), L.ptr(background),
            L.ptr(g_normals), L.ptr(g_depths), L.ptr(g_surf_depth), L.ptr(g_surf_normal), L.ptr(g_distortion),
            L.ptr(g_composited), L.ptr(g_extras), L.ptr(g_opacity), L.current_stream())
    L.check(rc, what)
    return g_extras, g_opacity


# --------------------------------------------------------------------------------------------------------------------
def simple_knn(points: Tensor) -> Tensor:
    """other/knn.cu:180-205: mean squared distance of every point to its three nearest neighbours -> [P]."""
    what = 'simple_knn'
    if not isinstance(points, Tensor) or not points.is_cuda:
        raise RuntimeError(f'{what}: points must be a CUDA tensor')
    L.require_dtype(what, 'points', points, torch.float32)
    if points.ndim != 2 or points.shape[-1] != 3:
        raise RuntimeError(f'{what}: Error shape for points')
    points = points.contiguous()
    P = points.shape[0]
    means = torch.empty((P,), dtype=torch.float32, device=points.device)
    lib = _lib()
    ws = _workspace(lib.fsgs_simple_knn_workspace_bytes(P), points.device)
    with _timed('simple_knn'):
        rc = lib.fsgs_simple_knn(P, L.ptr(points), L.ptr(means), L.ptr(ws), ws.numel(), L.current_stream())
    L.check(rc, what)
    return means


# ---- adaptive density control as stream compaction ---------------------------------------------------------------------
def _as_bytes(what: str, name: str, mask: Tensor) -> Tensor:
    if not isinstance(mask, Tensor) or not mask.is_cuda:
        raise RuntimeError(f'{what}: {name} must be a CUDA tensor')
    if mask.dtype not in (torch.bool, torch.uint8):
        raise RuntimeError(f'{what}: {name} must be a bool or uint8 tensor')
    mask = mask.contiguous()
    return mask.view(torch.uint8) if mask.dtype == torch.bool else mask


def select_indices(mask: Tensor, invert: bool = False) -> Tensor:
    """Ascending positions of the set (or, with invert, the clear) entries of a 1-D mask, int32 -- the index form of the
    reference's `tensor[mask]` / `tensor[~mask]` (gaussian_splatting.py:526-527, :558)."""
    what = 'select_indices'
    m = _as_bytes(what, 'mask', mask)
    if m.ndim != 1:
        raise RuntimeError(f'{what}: mask must be one-dimensional')
    P, dev = m.shape[0], m.device
    indices = torch.empty((max(P, 1),), dtype=torch.int32, device=dev)
    lib = _lib()
    ws = _workspace(lib.fsgs_select_indices_workspace_bytes(P), dev)
    count = _pinned_count()
    with _timed('select_indices'):
        rc = lib.fsgs_select_indices(P, L.ptr(m), int(bool(invert)), L.ptr(indices), L.ptr(ws), ws.numel(),
                                     count.data_ptr(), L.current_stream())
    L.check(rc, what)
    return indices[:ctypes.c_int64.from_address(count.data_ptr()).value]


def gather_rows(tensors: Sequence[Tensor], source_row: Tensor) -> List[Tensor]:
    """For every tensor t: out[r] = t[source_row[r]], or a row of zeros where source_row[r] < 0 -- `old[mask]`, `torch.cat`
    with copies of selected rows and the zero Adam moments of new points (gaussian_splatting.py:524-551) for all per-point
    tensors in one launch per 24 tensors."""
    what = 'gather_rows'
    if not isinstance(source_row, Tensor) or not source_row.is_cuda or source_row.dtype != torch.int32 or \
            source_row.ndim != 1:
        raise RuntimeError(f'{what}: source_row must be a one-dimensional int32 CUDA tensor')
    source_row = source_row.contiguous()
    n_rows, dev = source_row.shape[0], source_row.device
    srcs, outs = [], []
    for i, t in enumerate(tensors):
        if not isinstance(t, Tensor) or not t.is_cuda or t.ndim < 1:
            raise RuntimeError(f'{what}: tensor {i} must be a CUDA tensor with a leading point dimension')
        t = t.detach().contiguous()
        srcs.append(t)
        outs.append(torch.empty((n_rows,) + tuple(t.shape[1:]), dtype=t.dtype, device=dev))
    lib = _lib()
    step = lib.fsgs_gather_rows_max_tensors()
    stream = L.current_stream()
    for lo in range(0, len(srcs), step):
        # tensors without bytes (no rows in, none out, or an empty trailing shape) have nothing to move
        part = [(a, b) for a, b in zip(srcs[lo:lo + step], outs[lo:lo + step]) if b.numel() > 0]
        if not part:
            continue
        for a, _ in part:
            if a.shape[0] == 0:
                raise RuntimeError(f'{what}: cannot gather rows from an empty tensor')
        n = len(part)
        src_arr = (ctypes.c_void_p * n)(*[a.data_ptr() for a, _ in part])
        dst_arr = (ctypes.c_void_p * n)(*[b.data_ptr() for _, b in part])
        row_arr = (ctypes.c_int64 * n)(*[b[0].numel() * b.element_size() for _, b in part])
        with _timed('gather_rows'):
            rc = lib.fsgs_gather_rows(n, ctypes.addressof(src_arr), ctypes.addressof(dst_arr),
                                      ctypes.addressof(row_arr), n_rows, L.ptr(source_row), stream)
        L.check(rc, what)
    return outs


def _point_scalars(what: str, name: str, t: Tensor, P: int) -> Tensor:
    L.require_cuda(what, **{name: t})
    L.require_dtype(what, name, t, torch.float32)
    if t.numel() != P:
        raise RuntimeError(f'{what}: {name} must have {P} elements')
    return t


def densify_masks(grad_accum: Tensor, denom: Tensor, scaling: Tensor, grad_threshold: float,
                  scale_threshold: float) -> Tuple[Tensor, Tensor]:
    """Clone and split selections of gaussian_splatting.py:623-626, :612-615, :585-589 from the accumulated screen-space
    gradient statistics and the ACTIVATED scales [P,S] -> two bool masks [P]."""
    what = 'densify_masks'
    L.require_cuda(what, scaling=scaling)
    L.require_dtype(what, 'scaling', scaling, torch.float32)
    if scaling.ndim != 2 or not 1 <= scaling.shape[1] <= 3:
        raise RuntimeError(f'{what}: Error shape for scaling')
    P, S = scaling.shape
    _point_scalars(what, 'grad_accum', grad_accum, P)
    _point_scalars(what, 'denom', denom, P)
    clone = torch.empty((P,), dtype=torch.bool, device=scaling.device)
    split = torch.empty((P,), dtype=torch.bool, device=scaling.device)
    with _timed('densify_masks'):
        rc = _lib().fsgs_densify_masks(P, S, L.ptr(grad_accum), L.ptr(denom), L.ptr(scaling), float(grad_threshold),
                                       float(scale_threshold), L.ptr(clone), L.ptr(split), L.current_stream())
    L.check(rc, what)
    return clone, split


def prune_mask(opacity: Tensor, max_radii2D: Optional[Tensor], scaling: Optional[Tensor], min_opacity: float,
               max_screen_size: Optional[float], world_threshold: float = 0.0) -> Tensor:
    """Prune selection of gaussian_splatting.py:630-635 from ACTIVATED opacities [P,1] and scales [P,S] -> bool [P]. A
    false `max_screen_size` (None or 0) keeps only the opacity test, as the reference's `if max_screen_size:` does."""
    what = 'prune_mask'
    L.require_cuda(what, opacity=opacity, max_radii2D=max_radii2D, scaling=scaling)
    L.require_dtype(what, 'opacity', opacity, torch.float32)
    P = opacity.numel()
    use_size = bool(max_screen_size)
    S = 1
    if use_size:
        if max_radii2D is None or scaling is None:
            raise RuntimeError(f'{what}: max_radii2D and scaling are needed with max_screen_size')
        _point_scalars(what, 'max_radii2D', max_radii2D, P)
        L.require_dtype(what, 'scaling', scaling, torch.float32)
        if scaling.ndim != 2 or scaling.shape[0] != P or not 1 <= scaling.shape[1] <= 3:
            raise RuntimeError(f'{what}: Error shape for scaling')
        S = scaling.shape[1]
    mask = torch.empty((P,), dtype=torch.bool, device=opacity.device)
    with _timed('prune_mask'):
        rc = _lib().fsgs_prune_mask(P, S, L.ptr(opacity), L.ptr(max_radii2D) if use_size else None,
                                    L.ptr(scaling) if use_size else None, float(min_opacity), int(use_size),
                                    float(max_screen_size or 0.0), float(world_threshold), L.ptr(mask),
                                    L.current_stream())
    L.check(rc, what)
    return mask


def split_children(selected: Tensor, N: int, xyz: Tensor, scaling: Tensor, rotations: Tensor,
                   noise: Tensor) -> Tuple[Tensor, Tensor]:
    """Positions and raw (log) scales of the N children of every selected point (gaussian_splatting.py:591-597,
    network.py:1170-1183): `R(q) (noise * scale) + xyz` and `log(scale / (0.8 N))`, children ordered as
    `x[selected].repeat(N, 1)`. scaling [P,S] is ACTIVATED, noise [N * len(selected), 3] standard normal."""
    what = 'split_children'
    L.require_cuda(what, selected=selected, xyz=xyz, scaling=scaling, rotations=rotations, noise=noise)
    L.require_dtype(what, 'selected', selected, torch.int32)
    for name, t in (('xyz', xyz), ('scaling', scaling), ('rotations', rotations), ('noise', noise)):
        L.require_dtype(what, name, t, torch.float32)
    P = xyz.shape[0]
    if scaling.ndim != 2 or scaling.shape[0] != P or scaling.shape[1] not in (2, 3):
        raise RuntimeError(f'{what}: Error shape for scaling')
    S, n_sel = scaling.shape[1], selected.numel()
    L.require_shape(what, 'xyz', xyz, P, 3)
    L.require_shape(what, 'rotations', rotations, P, 4)
    L.require_shape(what, 'noise', noise, n_sel * N, 3)
    out_xyz = torch.empty((n_sel * N, 3), dtype=torch.float32, device=xyz.device)
    out_scaling = torch.empty((n_sel * N, S), dtype=torch.float32, device=xyz.device)
    with _timed('split_children'):
        rc = _lib().fsgs_split_children(P, n_sel, int(N), S, L.ptr(selected), L.ptr(xyz), L.ptr(scaling),
                                        L.ptr(rotations), L.ptr(noise), L.ptr(out_xyz), L.ptr(out_scaling),
                                        L.current_stream())
    L.check(rc, what)
    return out_xyz, out_scaling


def densification_stats(radii: Tensor, grad: Tensor, max_radii2D: Tensor, grad_accum: Tensor, denom: Tensor,
                        factor: Optional[Tensor] = None) -> Tensor:
    """Per-step statistics of network.py:1276-1282 (+ gaussian_splatting.py:486-495): for points with radii > 0 updates
    max_radii2D, grad_accum (+= |grad[:, :2]|, times factor if given) and denom IN PLACE; returns `radii > 0` (bool)."""
    what = 'densification_stats'
    L.require_cuda(what, radii=radii, grad=grad, max_radii2D=max_radii2D, grad_accum=grad_accum, denom=denom,
                   factor=factor)
    L.require_dtype(what, 'radii', radii, torch.int32)
    L.require_dtype(what, 'grad', grad, torch.float32)
    P = radii.numel()
    if grad.ndim != 2 or grad.shape[0] != P or grad.shape[1] < 2:
        raise RuntimeError(f'{what}: Error shape for grad')
    _point_scalars(what, 'max_radii2D', max_radii2D, P)
    _point_scalars(what, 'grad_accum', grad_accum, P)
    _point_scalars(what, 'denom', denom, P)
    if factor is not None:
        _point_scalars(what, 'factor', factor, P)
    visible = torch.empty((P,), dtype=torch.bool, device=radii.device)
    with _timed('densification_stats'):
        rc = _lib().fsgs_densification_stats(P, grad.shape[1], L.ptr(radii), L.ptr(grad), L.ptr(factor),
                                             L.ptr(max_radii2D), L.ptr(grad_accum), L.ptr(denom), L.ptr(visible),
                                             L.current_stream())
    L.check(rc, what)
    return visible


# ---- 3D-Gaussian (EWA) path ------------------------------------------------------------------------------------------
def _tan_fov(tanFoV) -> Tuple[float, float]:
    if isinstance(tanFoV, Tensor):
        if tanFoV.numel() != 2:
            raise RuntimeError('tanFoV must have 2 elements')
        v = tanFoV.detach().cpu().tolist()  # the reference reads it with .item() too (gaussian_preprocess.cu:424-425)
        return float(v[0]), float(v[1])
    return float(tanFoV[0]), float(tanFoV[1])


def gaussian_topk_weights(topk: int, W: int, H: int, P: int, R: int, means2D: Tensor, conic_opacity: Tensor,
                          ranges: Tensor, point_list: Tensor) -> Tuple[Tensor, Tensor]:
    """gaussian_topk.cu:212-228 -> (top_indices[H,W,K] int32, top_weights[H,W,K])."""
    what = 'gaussian_topk_weights'
    _f32(what, means2D=means2D, conic_opacity=conic_opacity)
    L.require_cuda(what, ranges=ranges, point_list=point_list)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    top_indices = torch.empty((H, W, topk), dtype=torch.int32, device=means2D.device)
    top_weights = torch.empty((H, W, topk), dtype=torch.float32, device=means2D.device)
    with _timed(what):
        rc = _lib().fsgs_gaussian_topk_weights(topk, means2D.shape[0], W, H, L.ptr(means2D), L.ptr(conic_opacity),
                                               L.ptr(ranges), L.ptr(point_list), L.ptr(top_indices),
                                               L.ptr(top_weights), L.current_stream())
    L.check(rc, what)
    return top_indices, top_weights


def gaussian_rasterize_extra_forward(W: int, H: int, extras: Tensor, means2D: Tensor, conic_opacity: Tensor,
                                     ranges: Tensor, point_list: Tensor, n_contrib: Tensor) -> Tensor:
    """gaussian_rasterizer_extra.cu:317-339: extras[P,E] -> pixel_extras[H,W,E] with the blend weights of the main pass."""
    what = 'gaussian_rasterize_extra_forward'
    extras = extras.contiguous()  # as the reference's host function does
    _f32(what, extras=extras, means2D=means2D, conic_opacity=conic_opacity)
    L.require_cuda(what, ranges=ranges, point_list=point_list, n_contrib=n_contrib)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    L.require_dtype(what, 'n_contrib', n_contrib, torch.int32)
    if extras.ndim != 2:
        raise RuntimeError(f'{what}: Error shape for extras')
    P, E = extras.shape
    if means2D.shape[0] != P or conic_opacity.shape[0] != P or n_contrib.numel() != W * H:
        raise RuntimeError(f'{what}: extras, means2D, conic_opacity share P and n_contrib is [H,W]')
    out = torch.empty((H, W, E), dtype=torch.float32, device=extras.device)
    if E == 0:
        return out
    with _timed(what):
        rc = _lib().fsgs_gaussian_rasterize_extra_forward(
            P, W, H, E, L.ptr(extras), L.ptr(means2D), L.ptr(conic_opacity), L.ptr(ranges),
            L.ptr(point_list), L.ptr(n_contrib), L.ptr(out), L.current_stream())
    L.check(rc, what)
    return out


def gaussian_rasterize_extra_backward(W: int, H: int, extras: Tensor, out_opacity: Tensor, grad_out: Tensor,
                                      means2D: Tensor, conic_opacity: Tensor, ranges: Tensor, point_list: Tensor,
                                      n_contrib: Tensor, grad_extra: Optional[Tensor], grad_means2D: Optional[Tensor],
                                      grad_conic: Optional[Tensor]) -> None:
    """gaussian_rasterizer_extra.cu:341-365: adds into the gradient tensors that are given."""
    what = 'gaussian_rasterize_extra_backward'
    extras, grad_out = extras.contiguous(), grad_out.contiguous()  # as the reference's host function does
    _f32(what, extras=extras, out_opacity=out_opacity, grad_out=grad_out, means2D=means2D,
         conic_opacity=conic_opacity, grad_extra=grad_extra, grad_means2D=grad_means2D, grad_conic=grad_conic)
    L.require_cuda(what, ranges=ranges, point_list=point_list, n_contrib=n_contrib)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    L.require_dtype(what, 'n_contrib', n_contrib, torch.int32)
    P, E = extras.shape
    if grad_out.numel() != W * H * E or out_opacity.numel() != W * H or n_contrib.numel() != W * H:
        raise RuntimeError(f'{what}: grad_out is [H,W,E], out_opacity and n_contrib are [H,W]')
    for name, g, like in (('grad_extra', grad_extra, extras), ('grad_means2D', grad_means2D, means2D),
                          ('grad_conic', grad_conic, conic_opacity)):
        if g is not None and (tuple(g.shape) != tuple(like.shape) or not g.is_contiguous()):
            raise RuntimeError(f'{what}: {name} must be contiguous and shaped like its input')
    if E == 0:
        return
    with _timed(what):
        rc = _lib().fsgs_gaussian_rasterize_extra_backward(
            P, W, H, E, L.ptr(extras), L.ptr(out_opacity), L.ptr(grad_out), L.ptr(means2D),
            L.ptr(conic_opacity), L.ptr(ranges), L.ptr(point_list), L.ptr(n_contrib), L.ptr(grad_extra),
            L.ptr(grad_means2D), L.ptr(grad_conic), L.current_stream())
    L.check(rc, what)


def gaussian_rasterize_extra_backward_v2(W, H, extras, out_opacity, grad_out, means2D, conic_opacity, ranges,
                                         point_list, n_contrib, grad_extra, grad_means2D, grad_conic) -> None:
    """gaussian_rasterizer_extra.cu:367-391: the variant that assumes all three gradient tensors are given."""
    if grad_extra is None or grad_means2D is None or grad_conic is None:
        raise RuntimeError('gaussian_rasterize_extra_backward_v2: all three gradient tensors are required')
    gaussian_rasterize_extra_backward(W, H, extras, out_opacity, grad_out, means2D, conic_opacity, ranges, point_list,
                                      n_contrib, grad_extra, grad_means2D, grad_conic)


def gs_compute_cov3D_forward(q: Tensor, s: Tensor) -> Tensor:
    """gaussian_compute_cov3D.cu:122-137: q[..., 4] (x, y, z, w), s[..., 3] -> cov3D[..., 6]."""
    what = 'gs_compute_cov3D_forward'
    _f32(what, q=q, s=s)
    if s.shape[-1] != 3 or tuple(q.shape) != tuple(s.shape[:-1]) + (4,):
        raise RuntimeError(f'{what}: q.shape[:-1] == s.shape[:-1]')
    N = s.numel() // 3
    cov3D = torch.empty(tuple(s.shape[:-1]) + (6,), dtype=torch.float32, device=s.device)
    with _timed(what):
        rc = _lib().fsgs_gs_compute_cov3D_forward(N, L.ptr(q), L.ptr(s), L.ptr(cov3D), L.current_stream())
    L.check(rc, what)
    return cov3D


def gs_compute_cov3D_backward(q: Tensor, s: Tensor, dL_dCov3D: Tensor) -> List[Tensor]:
    """gaussian_compute_cov3D.cu:151-161 -> [dq, ds]."""
    what = 'gs_compute_cov3D_backward'
    dL_dCov3D = dL_dCov3D.contiguous()
    _f32(what, q=q, s=s, dL_dCov3D=dL_dCov3D)
    N = s.numel() // 3
    if dL_dCov3D.numel() != 6 * N or q.numel() != 4 * N:
        raise RuntimeError(f'{what}: Error shape')
    dq, ds = torch.empty_like(q), torch.empty_like(s)
    with _timed(what):
        rc = _lib().fsgs_gs_compute_cov3D_backward(N, L.ptr(q), L.ptr(s), L.ptr(dL_dCov3D), L.ptr(dq), L.ptr(ds),
                                                   L.current_stream())
    L.check(rc, what)
    return [dq, ds]


def gs_compute_cov2D_forward(cov3D: Tensor, mean: Tensor, viewmatrix: Tensor, focal_x: float, focal_y: float,
                             tan_fovx: float, tan_fovy: float) -> Tensor:
    """gaussian_compute_cov2D.cu:199-210: cov3D[N,6], mean[N,3], row-major Tw2v[4,4] -> cov2D[N,3]."""
    what = 'gs_compute_cov2D_forward'
    _f32(what, cov3D=cov3D, mean=mean, viewmatrix=viewmatrix)
    N = mean.numel() // 3
    if cov3D.numel() != 6 * N or viewmatrix.numel() != 16:
        raise RuntimeError(f'{what}: Error shape')
    cov2D = torch.empty_like(mean)
    with _timed(what):
        rc = _lib().fsgs_gs_compute_cov2D_forward(N, L.ptr(cov3D), L.ptr(mean), L.ptr(viewmatrix), float(focal_x),
                                                  float(focal_y), float(tan_fovx), float(tan_fovy), L.ptr(cov2D),
                                                  L.current_stream())
    L.check(rc, what)
    return cov2D


def gs_compute_cov2D_backward(cov3D: Tensor, mean: Tensor, viewmatrix: Tensor, focal_x: float, focal_y: float,
                              tan_fovx: float, tan_fovy: float, grad_cov2D: Tensor,
                              grad_vm: Optional[Tensor] = None) -> List[Tensor]:
    """gaussian_compute_cov2D.cu:229-248 -> [grad_cov3D, grad_mean]; with grad_vm[4,4] the view matrix's gradient is
    added to its first three rows in place."""
    what = 'gs_compute_cov2D_backward'
    grad_cov2D = grad_cov2D.contiguous()
    _f32(what, cov3D=cov3D, mean=mean, viewmatrix=viewmatrix, grad_cov2D=grad_cov2D, grad_vm=grad_vm)
    N = mean.numel() // 3
    if cov3D.numel() != 6 * N or viewmatrix.numel() != 16 or grad_cov2D.numel() != 3 * N:
        raise RuntimeError(f'{what}: Error shape')
    if grad_vm is not None and grad_vm.numel() != 16:
        raise RuntimeError(f'{what}: grad_vm must have 16 elements')
    g_cov3D, g_mean = torch.empty_like(cov3D), torch.empty_like(mean)
    with _timed(what):
        rc = _lib().fsgs_gs_compute_cov2D_backward(N, L.ptr(cov3D), L.ptr(mean), L.ptr(viewmatrix), float(focal_x),
                                                   float(focal_y), float(tan_fovx), float(tan_fovy),
                                                   L.ptr(grad_cov2D), L.ptr(g_cov3D), L.ptr(g_mean), L.ptr(grad_vm),
                                                   L.current_stream())
    L.check(rc, what)
    return [g_cov3D, g_mean]


def gs_preprocess_forward(W: int, H: int, sh_degree: int, is_opengl: bool, means3D: Tensor, scales: Tensor,
                          rotations: Tensor, opacities: Tensor, shs: Tensor, sh_rest: Optional[Tensor], Tw2v: Tensor,
                          Tv2c: Tensor, cam_pos: Tensor, tanFoV, cov3D_precomp: Optional[Tensor] = None,
                          cov2D_precomp: Optional[Tensor] = None, means2D: Optional[Tensor] = None,
                          culling: Optional[Tensor] = None) -> List[Tensor]:
    """gaussian_preprocess.cu:372-466 -> [means2D, depths, colors, radii, tiles_touched, cov3Ds, conic_opacity]."""
    what = 'gs_preprocess_forward'
    _f32(what, means3D=means3D, scales=scales, rotations=rotations, opacities=opacities, shs=shs, Tw2v=Tw2v,
         Tv2c=Tv2c, cam_pos=cam_pos, cov3D_precomp=cov3D_precomp, cov2D_precomp=cov2D_precomp)
    if means3D.ndim != 2 or means3D.shape[-1] != 3:
        raise RuntimeError('Error shape for means3D')
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.numel() > 0
    M = 0
    if has_rest:
        _f32(what, sh_rest=sh_rest)
        if not (sh_rest.ndim == 3 and sh_rest.shape[0] == P and sh_rest.shape[1] >= (1 + sh_degree) ** 2 - 1
                and sh_rest.shape[2] == 3):
            raise RuntimeError('Error shape for sh features')
        M = sh_rest.shape[1]
    elif sh_degree >= 0:
        if not (shs.ndim == 3 and shs.shape[0] == P and shs.shape[1] >= (1 + sh_degree) ** 2 and shs.shape[2] == 3):
            raise RuntimeError('Error shape for sh features')
        M = shs.shape[1]
    if means2D is not None:
        _f32(what, means2D=means2D)
        L.require_shape(what, 'means2D', means2D, P, 2)
    if culling is not None:
        L.require_cuda(what, culling=culling)
        L.require_dtype(what, 'culling', culling, torch.bool)
        L.require_shape(what, 'culling', culling, P)
    L.require_shape(what, 'scales', scales, P, 3)
    L.require_shape(what, 'rotations', rotations, P, 4)
    L.require_shape(what, 'opacities', opacities, P, 1)
    L.require_shape(what, 'Tw2v', Tw2v, 4, 4)
    L.require_shape(what, 'Tv2c', Tv2c, 4, 4)
    L.require_shape(what, 'cam_pos', cam_pos, 3)
    if sh_degree < 0:
        L.require_shape(what, 'shs', shs, P, 3)
    if cov3D_precomp is not None:
        L.require_shape(what, 'cov3D_precomp', cov3D_precomp, P, 6)
    if cov2D_precomp is not None:
        L.require_shape(what, 'cov2D_precomp', cov2D_precomp, P, 3)
    tx, ty = _tan_fov(tanFoV)
    opt = dict(dtype=torch.float32, device=means3D.device)
    colors = shs if sh_degree < 0 else torch.empty((P, 3), **opt)
    preserve = means2D is not None
    means2D_ = means2D if preserve else torch.empty((P, 2), **opt)
    depths, conic_opacity = torch.empty((P,), **opt), torch.empty((P, 4), **opt)
    # the reference hands a pre-computed cov3D back as the cov3Ds output (gaussian_preprocess.cu:424)
    cov3Ds = cov3D_precomp if cov3D_precomp is not None else torch.empty((P, 6), **opt)
    radii = torch.empty((P,), dtype=torch.int32, device=means3D.device)
    tiles_touched = torch.empty((P,), dtype=torch.int32, device=means3D.device)
    with _timed('gs_preprocess_forward'):
        rc = _lib().fsgs_gs_preprocess_forward(
            P, W, H, sh_degree, M, int(bool(is_opengl)), L.ptr(means3D), L.ptr(scales), L.ptr(rotations),
            L.ptr(opacities), L.ptr(shs), L.ptr(sh_rest) if has_rest else None, L.ptr(Tw2v), L.ptr(Tv2c),
            L.ptr(cam_pos), tx, ty, L.ptr(culling), L.ptr(cov3D_precomp), L.ptr(cov2D_precomp), int(preserve),
            L.ptr(means2D_), L.ptr(depths), None if sh_degree < 0 else L.ptr(colors), L.ptr(radii),
            L.ptr(tiles_touched), None if cov3D_precomp is not None else L.ptr(cov3Ds), L.ptr(conic_opacity),
            L.current_stream())
    L.check(rc, what)
    return [means2D_, depths, colors, radii, tiles_touched, cov3Ds, conic_opacity]


def gs_preprocess_backward(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs, sh_rest, Tw2v,
                           Tv2c, cam_pos, tanFoV, cov3Ds, cov2Ds, radii, colors, grad_mean2D, grad_depth, grad_colors,
                           grad_conic, grad_means3D, grad_scales, grad_rotations, grad_opacities, grad_shs,
                           grad_sh_rest, grad_cov=None, grad_Tw2v=None, grad_campos=None) -> None:
    """gaussian_preprocess.cu:567-636: fills the caller's grad_* tensors in place (every row is assigned) and rewrites
    grad_mean2D as the reference does. grad_depth is ignored there too. With cov2Ds (pre-computed 2D covariances)
    grad_cov is [P,3] and grad_scales / grad_rotations must be None; grad_Tw2v[4,4] and grad_campos[3] are added to."""
    what = 'gs_preprocess_backward'
    _f32(what, grad_mean2D=grad_mean2D, grad_colors=grad_colors, grad_conic=grad_conic, grad_means3D=grad_means3D,
         grad_scales=grad_scales, grad_rotations=grad_rotations, grad_opacities=grad_opacities, grad_shs=grad_shs,
         grad_sh_rest=grad_sh_rest, grad_cov=grad_cov, cov3Ds=cov3Ds, cov2Ds=cov2Ds, grad_Tw2v=grad_Tw2v,
         grad_campos=grad_campos)
    if cov2Ds is not None and (grad_scales is not None or grad_rotations is not None):
        raise RuntimeError(f'{what}: grad_scales / grad_rotations must be None with pre-computed 2D covariances')
    if cov2Ds is None and cov3Ds is None:
        raise RuntimeError(f"{what}: cov3Ds (the forward's output) or cov2Ds is required")
    if grad_Tw2v is not None and grad_Tw2v.numel() != 16:
        raise RuntimeError(f'{what}: grad_Tw2v must be [4,4]')
    if grad_campos is not None and grad_campos.numel() != 3:
        raise RuntimeError(f'{what}: grad_campos must be [3]')
    has_rest = sh_rest is not None and sh_rest.numel() > 0
    P = means3D.shape[0]
    M = sh_rest.shape[1] if has_rest else (shs.shape[1] if shs.ndim == 3 else 0)
    L.require_shape(what, 'grad_means3D', grad_means3D, P, 3)
    L.require_shape(what, 'grad_conic', grad_conic, P, 4)
    L.require_shape(what, 'grad_opacities', grad_opacities, P, 1)
    if grad_cov is not None:
        L.require_shape(what, 'grad_cov', grad_cov, P, 3 if cov2Ds is not None else 6)
    if sh_degree >= 0 and grad_colors is None:
        raise RuntimeError(f'{what}: grad_colors is required with SH colours')
    tx, ty = _tan_fov(tanFoV)
    with _timed('gs_preprocess_backward'):
        rc = _lib().fsgs_gs_preprocess_backward(
            P, W, H, sh_degree, M, int(bool(is_opengl)), L.ptr(means3D), L.ptr(scales), L.ptr(rotations), L.ptr(shs),
            L.ptr(sh_rest) if has_rest else None, L.ptr(Tw2v), L.ptr(Tv2c), L.ptr(cam_pos), tx, ty, L.ptr(radii),
            L.ptr(colors), L.ptr(cov3Ds), L.ptr(cov2Ds), L.ptr(grad_mean2D), L.ptr(grad_colors), L.ptr(grad_conic),
            L.ptr(grad_means3D), L.ptr(grad_scales), L.ptr(grad_rotations), L.ptr(grad_opacities), L.ptr(grad_shs),
            L.ptr(grad_sh_rest) if has_rest else None, L.ptr(grad_cov), L.ptr(grad_Tw2v), L.ptr(grad_campos),
            L.current_stream())
    L.check(rc, what)


def gaussian_rasterize_forward(width: int, height: int, means2D: Tensor, conic_opacity: Tensor, colors: Tensor,
                               extras: Optional[Tensor], point_list: Tensor, ranges: Tensor,
                               accum_max_count: Optional[Tensor] = None, accum_weights_p: Optional[Tensor] = None,
                               accum_weights_count: Optional[Tensor] = None,
                               per_tile_bucket_offset: Optional[Tensor] = None):
    """gaussian_render.cu:212-293 -> [pixel_colors[3,H,W], pixel_opacity[H,W], pixel_extras[E,H,W]|None,
    n_contrib[H,W]] and, with per_tile_bucket_offset, [max_contrib[Ty,Tx], bucket_to_tile[B], sampled_T[B,256],
    sampled_ar[B,3+E,256]] (the snapshots the per-Gaussian backward takes)."""
    what = 'gaussian_rasterize_forward'
    _f32(what, means2D=means2D, conic_opacity=conic_opacity, colors=colors, extras=extras,
         accum_weights_p=accum_weights_p)
    L.require_cuda(what, point_list=point_list, ranges=ranges, accum_max_count=accum_max_count,
                   accum_weights_count=accum_weights_count)
    if colors.ndim != 2:
        raise RuntimeError(f'{what}: colors must be [P,3]')
    P = colors.shape[0]
    E = 0
    if extras is not None:
        if extras.ndim != 2 or extras.shape[0] != P:
            raise RuntimeError(f'{what}: extras must be [P,E]')
        E = extras.shape[1]
        if E > 4:
            raise RuntimeError('Only support NUM_EXTRA=0,1,2,3,4')
    L.require_shape(what, 'colors', colors, P, 3)
    L.require_dtype(what, 'point_list', point_list, torch.int32)
    L.require_dtype(what, 'ranges', ranges, torch.int64)
    for name, t, dt in (('accum_max_count', accum_max_count, torch.int32),
                        ('accum_weights_count', accum_weights_count, torch.int32)):
        if t is not None:
            L.require_dtype(what, name, t, dt)
            L.require_shape(what, name, t, P)
    if accum_weights_p is not None:
        L.require_shape(what, 'accum_weights_p', accum_weights_p, P)
    opt = dict(dtype=torch.float32, device=colors.device)
    pixel_colors, pixel_opacity = torch.empty((3, height, width), **opt), torch.empty((height, width), **opt)
    pixel_extras = torch.empty((E, height, width), **opt) if extras is not None else None
    n_contrib = torch.empty((height, width), dtype=torch.int32, device=colors.device)
    snap = [None] * 4
    if per_tile_bucket_offset is not None:
        L.require_cuda(what, per_tile_bucket_offset=per_tile_bucket_offset)
        L.require_dtype(what, 'per_tile_bucket_offset', per_tile_bucket_offset, torch.int64)
        per_tile_bucket_offset = per_tile_bucket_offset.contiguous()
        B = int(per_tile_bucket_offset.reshape(-1)[-1].item()) if per_tile_bucket_offset.numel() else 0
        gy, gx = (height + _TILE - 1) // _TILE, (width + _TILE - 1) // _TILE
        nb = max(B, 1)  # keep the base pointers valid when no tile has any entry
        snap = [torch.zeros((gy, gx), dtype=torch.int32, device=colors.device),
                torch.empty((nb,), dtype=torch.int32, device=colors.device),
                torch.empty((nb, _TILE * _TILE), **opt), torch.empty((nb, 3 + E, _TILE * _TILE), **opt)]
    with _timed('gaussian_rasterize_forward'):
        rc = _lib().fsgs_gaussian_rasterize_forward(
            P, width, height, E, L.ptr(means2D), L.ptr(conic_opacity), L.ptr(colors), L.ptr(extras) if E else None,
            L.ptr(point_list), L.ptr(ranges), L.ptr(accum_max_count), L.ptr(accum_weights_p),
            L.ptr(accum_weights_count), L.ptr(per_tile_bucket_offset), L.ptr(pixel_colors), L.ptr(pixel_opacity),
            L.ptr(pixel_extras) if E else None, L.ptr(n_contrib), *[L.ptr(t) for t in snap], L.current_stream())
    L.check(rc, what)
    out = [pixel_colors, pixel_opacity, pixel_extras, n_contrib]
    if per_tile_bucket_offset is not None:
        out += [snap[0], snap[1][:B], snap[2][:B], snap[3][:B]]
    return out


def gaussian_rasterize_backward(means2D: Tensor, conic_opacity: Tensor, colors: Tensor, extras: Optional[Tensor],
                                out_opacity: Tensor, dL_dout_color: Tensor, dL_dout_opacity: Tensor,
                                dL_dout_extra: Optional[Tensor], ranges: Tensor, point_list: Tensor,
                                n_contrib: Tensor, point_offsets: Optional[Tensor] = None,
                                radii: Optional[Tensor] = None, culled: Optional[Tensor] = None):
    """gaussian_render.cu:486-536 -> (dL_dcolors[P,3], dL_dextras[P,E]|None, dL_dmeans2D[P,2], dL_dconic_opacity[P,4]).
    With `point_offsets` (GS_prepare(..., return_offsets=True)) and `radii` the per-Gaussian sums are taken in a fixed
    order from per-instance records instead of with atomics; `culled`: the keep masks, when the lists were built by
    GS_prepare(..., cull=True) (the records of the instances left out are zeroed first)."""
    what = 'gaussian_rasterize_backward'
    L.require_cuda(what, dL_dout_color=dL_dout_color, dL_dout_opacity=dL_dout_opacity, dL_dout_extra=dL_dout_extra)
    P = means2D.shape[0]
    H, W = dL_dout_color.shape[1], dL_dout_color.shape[2]
    E = extras.shape[-1] if (dL_dout_extra is not None and extras is not None) else 0
    if E > 4:
        raise RuntimeError('Only support NUM_EXTRA=0,1,2,3,4')
    opt = dict(dtype=torch.float32, device=out_opacity.device)
    ordered, ws, R = _ordered_sum_inputs(what, P, point_list, point_offsets, radii,
                                         'fsgs_gaussian_rasterize_backward_workspace_bytes', out_opacity.device)
    # means2D 2 | conic_opacity 4 | colours 3 | extras E in one allocation: zero-filled for the atomic path, written row
    # by row by the ordered path
    grads = (torch.empty if ordered else torch.zeros)((P, 9 + E), **opt)
    g_flat = grads.view(-1)
    dL_dmeans2D = g_flat[:2 * P].view(P, 2)
    dL_dconic_o = g_flat[2 * P:6 * P].view(P, 4)
    dL_dcolors = g_flat[6 * P:9 * P].view(P, 3)
    dL_dextras = g_flat[9 * P:].view(P, E) if E else None
    if P == 0:
        return dL_dcolors, dL_dextras, dL_dmeans2D, dL_dconic_o
    c = lambda t: None if t is None else t.contiguous()
    args = [c(means2D), c(conic_opacity), c(colors), c(extras) if E else None, c(out_opacity), c(n_contrib),
            c(dL_dout_color), c(dL_dout_extra) if E else None, c(dL_dout_opacity), c(point_list), c(ranges)]
    with _timed('gaussian_rasterize_backward'):
        if ordered and culled is not None:
            _clear_culled_records(what, P, R, point_offsets, culled, ws)
        rc = _lib().fsgs_gaussian_rasterize_backward(
            P, W, H, E, *[L.ptr(a) for a in args], L.ptr(dL_dmeans2D), L.ptr(dL_dconic_o), L.ptr(dL_dcolors),
            L.ptr(dL_dextras), R, L.ptr(point_offsets) if ordered else None, L.ptr(radii) if ordered else None,
            L.ptr(ws), ws.numel() if ws is not None else 0, L.current_stream())
    L.check(rc, what)
    return dL_dcolors, dL_dextras, dL_dmeans2D, dL_dconic_o


def _clear_culled_records(what, P, R, point_offsets, keep_masks, ws):
    L.require_cuda(what, culled=keep_masks)
    L.require_dtype(what, 'culled', keep_masks, torch.int32)
    L.require_shape(what, 'culled', keep_masks, max(P, 1))
    L.check(_lib().fsgs_gaussian_rasterize_clear_culled(P, R, L.ptr(point_offsets), L.ptr(keep_masks), L.ptr(ws),
                                                        ws.numel(), L.current_stream()), what)


def _ordered_sum_inputs(what, P, point_list, point_offsets, radii, workspace_bytes_fn, device):
    """Checks the optional inputs of a backward's ordered-sum path and allocates its workspace:
    -> (ordered, workspace | None, instance count R)."""
    R = int(point_list.numel())
    ordered = point_offsets is not None and P > 0
    if not ordered:
        return False, None, R
    if radii is None:
        raise RuntimeError(f'{what}: radii is required together with point_offsets')
    L.require_cuda(what, point_offsets=point_offsets, radii=radii)
    L.require_dtype(what, 'point_offsets', point_offsets, torch.int64)
    L.require_dtype(what, 'radii', radii, torch.int32)
    return True, _workspace(getattr(_lib(), workspace_bytes_fn)(R), device), R


# Which kernel gaussian_rasterize_fast_backward runs when the caller does not say: the reference's per-Gaussian
# decomposition (True) or the back-to-front kernel that gives the same derivative faster on this chip (False).
PER_GAUSSIAN_BACKWARD = False


def gaussian_rasterize_fast_backward(means2D: Tensor, conic_opacity: Tensor, colors: Tensor, extras: Optional[Tensor],
                                     images: Tensor, out_extras: Optional[Tensor], out_opacity: Tensor,
                                     dL_dout_color: Tensor, dL_dout_opacity: Tensor, dL_dout_extra: Optional[Tensor],
                                     ranges: Tensor, point_list: Tensor, n_contrib: Tensor, max_contrib: Tensor,
                                     per_tile_bucket_offset: Tensor, bucket_to_tile: Tensor, sampled_T: Tensor,
                                     sampled_ar: Tensor, point_offsets: Optional[Tensor] = None,
                                     radii: Optional[Tensor] = None, per_gaussian: Optional[bool] = None,
                                     culled: Optional[Tensor] = None):
    """gaussian_render.cu:760-812 -> (dL_dcolors[P,3], dL_dextras[P,E]|None, dL_dmeans2D[P,2], dL_dconic_opacity[P,4]):
    the reference's per-Gaussian backward over the forward's bucket snapshots. The same derivative as
    gaussian_rasterize_backward; by default it is evaluated by that operator's back-to-front kernel (the faster one on
    this chip; the snapshot tensors are checked and not read). `per_gaussian=True` (default: PER_GAUSSIAN_BACKWARD of
    this module) runs the reference's decomposition instead: one lane per list entry, pixels passed from lane to lane,
    started from the snapshots. `point_offsets` / `radii` as for gaussian_rasterize_backward."""
    what = 'gaussian_rasterize_fast_backward'
    L.require_cuda(what, images=images, max_contrib=max_contrib, per_tile_bucket_offset=per_tile_bucket_offset,
                   bucket_to_tile=bucket_to_tile, sampled_T=sampled_T, sampled_ar=sampled_ar)
    L.require_dtype(what, 'per_tile_bucket_offset', per_tile_bucket_offset, torch.int64)
    L.require_dtype(what, 'bucket_to_tile', bucket_to_tile, torch.int32)
    L.require_dtype(what, 'max_contrib', max_contrib, torch.int32)
    P = means2D.shape[0]
    H, W = dL_dout_color.shape[1], dL_dout_color.shape[2]
    E = extras.shape[-1] if (dL_dout_extra is not None and extras is not None) else 0
    if E > 4:
        raise RuntimeError('Only support NUM_EXTRA=0,1,2,3,4')
    if E and out_extras is None:
        raise RuntimeError(f'{what}: out_extras is required with extras')
    B = int(bucket_to_tile.numel())
    if tuple(sampled_T.shape) != (B, _TILE * _TILE) or tuple(sampled_ar.shape)[0] != B:
        raise RuntimeError(f'{what}: the snapshot tensors do not match bucket_to_tile')
    opt = dict(dtype=torch.float32, device=out_opacity.device)
    ordered, ws, R = _ordered_sum_inputs(what, P, point_list, point_offsets, radii,
                                         'fsgs_gaussian_rasterize_backward_workspace_bytes', out_opacity.device)
    grads = (torch.empty if ordered else torch.zeros)((P, 9 + E), **opt)  # means2D 2 | conic_opacity 4 | colours 3 | extras E
    g_flat = grads.view(-1)
    dL_dmeans2D = g_flat[:2 * P].view(P, 2)
    dL_dconic_o = g_flat[2 * P:6 * P].view(P, 4)
    dL_dcolors = g_flat[6 * P:9 * P].view(P, 3)
    dL_dextras = g_flat[9 * P:].view(P, E) if E else None
    if P == 0:
        return dL_dcolors, dL_dextras, dL_dmeans2D, dL_dconic_o
    c = lambda t: None if t is None else t.contiguous()
    args = [c(means2D), c(conic_opacity), c(colors), c(extras) if E else None, c(images), c(out_extras) if E else None,
            c(out_opacity), c(n_contrib), c(max_contrib), c(per_tile_bucket_offset), c(bucket_to_tile), c(sampled_T),
            c(sampled_ar), c(dL_dout_color), c(dL_dout_extra) if E else None, c(dL_dout_opacity), c(point_list),
            c(ranges)]
    tail = (L.ptr(dL_dmeans2D), L.ptr(dL_dconic_o), L.ptr(dL_dcolors), L.ptr(dL_dextras), R,
            L.ptr(point_offsets) if ordered else None, L.ptr(radii) if ordered else None, L.ptr(ws),
            ws.numel() if ws is not None else 0, L.current_stream())
    if ordered and culled is not None:  # lists from GS_prepare(..., cull=True): see gaussian_rasterize_backward
        _clear_culled_records(what, P, R, point_offsets, culled, ws)
    if PER_GAUSSIAN_BACKWARD if per_gaussian is None else per_gaussian:
        with _timed('gaussian_rasterize_bucket_backward'):
            rc = _lib().fsgs_gaussian_rasterize_bucket_backward(P, W, H, E, B, *[L.ptr(a) for a in args], *tail)
    else:
        with _timed('gaussian_rasterize_backward'):
            rc = _lib().fsgs_gaussian_rasterize_fast_backward(P, W, H, E, *[L.ptr(a) for a in args], *tail)
    L.check(rc, what)
    return dL_dcolors, dL_dextras, dL_dmeans2D, dL_dconic_o
