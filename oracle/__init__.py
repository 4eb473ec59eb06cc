"""TEST INFRASTRUCTURE ONLY: ctypes loader and numpy-level wrappers of the CPU parity oracle (liboracle.so).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the product package
never does. Every wrapper takes and returns numpy arrays (host memory).
"""
from __future__ import annotations

import ctypes
import re
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "_build" / "liboracle.so"

_SCALARS = {"int": ctypes.c_int, "int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64, "size_t": ctypes.c_size_t,
            "double": ctypes.c_double, "float": ctypes.c_float, "uint32_t": ctypes.c_uint32}


def build() -> Path:
    proc = subprocess.run(["make", "-C", str(HERE), "-B"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + proc.stdout + proc.stderr)
    return LIB_PATH


def _parse(text: str):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    out = {}
    for m in re.finditer(r"([A-Za-z_]\w*)\s+(oracle_\w+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        argtypes = []
        if args not in ("", "void"):
            for a in args.split(","):
                argtypes.append(ctypes.c_void_p if "*" in a else _SCALARS[a.replace("const", "").split()[0]])
        out[name] = (_SCALARS[ret], argtypes)
    return out


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        L = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in _parse((HERE / "oracle.h").read_text()).items():
            for n in {name, name.replace("_f32", "_f64")}:
                fn = getattr(L, n)
                fn.restype, fn.argtypes = restype, argtypes
        _lib = L
    return _lib


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "oracle wants C-contiguous numpy arrays"
    return a.ctypes.data


def _suffix(dtype) -> str:
    return {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}[np.dtype(dtype)]


def call(name: str, *args):
    """Calls oracle_<name> converting numpy arrays to addresses; raises on a non-zero status."""
    fn = getattr(lib(), "oracle_" + name)
    rc = fn(*[_p(a) if isinstance(a, np.ndarray) or a is None else a for a in args])
    return rc


def num_threads() -> int:
    return int(lib().oracle_num_threads())


# ---- numpy-level wrappers mirroring the operator signatures ------------------------------------------------------
def preprocess_forward(W, H, sh_degree, means3D, scales, rotations, opacities, shs, sh_rest, Tw2v, Tv2c, campos,
                       trans_precomp=None, means2D=None, culling=None):
    dt = means3D.dtype
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.size > 0
    n_sh = sh_rest.shape[1] if has_rest else (shs.shape[1] if sh_degree >= 0 else 0)
    preserve = means2D is not None
    m2 = means2D if preserve else np.zeros((P, 2), dt)
    colors = shs if sh_degree < 0 else np.zeros((P, 3), dt)
    tm = trans_precomp if trans_precomp is not None else np.zeros((P, 3, 3), dt)
    no, dep = np.zeros((P, 4), dt), np.zeros((P,), dt)
    radii, tt = np.zeros((P,), np.int32), np.zeros((P,), np.int32)
    cul = None if culling is None else np.ascontiguousarray(culling.astype(np.uint8))
    rc = call(f"gs_2d_preprocess_forward_{_suffix(dt)}", P, W, H, sh_degree, n_sh, means3D, scales, rotations,
              opacities, shs, sh_rest if has_rest else None, Tw2v, Tv2c, campos, trans_precomp, cul, int(preserve), m2,
              None if sh_degree < 0 else colors, None if trans_precomp is not None else tm, no, dep, radii, tt)
    assert rc == 0
    return m2, colors, tm, no, dep, radii, tt


def preprocess_backward(W, H, sh_degree, means3D, scales, rotations, shs, sh_rest, Tw2v, Tv2c, campos, trans_mat,
                        radii, colors, grad_mean2D, grad_trans, grad_colors, grad_normal_opacity):
    """Returns (g_means3D, g_scales, g_rot, g_opac, g_shs, g_sh_rest, grad_mean2D_after)."""
    dt = means3D.dtype
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.size > 0
    n_sh = sh_rest.shape[1] if has_rest else (shs.shape[1] if sh_degree >= 0 else 0)
    g3, gs, gr, go = np.zeros((P, 3), dt), np.zeros((P, 2), dt), np.zeros((P, 4), dt), np.zeros((P, 1), dt)
    gsh = np.zeros_like(shs) if sh_degree >= 0 else None
    gshr = np.zeros_like(sh_rest) if has_rest else None
    gm2 = grad_mean2D.copy()
    rc = call(f"gs_2d_preprocess_backward_{_suffix(dt)}", P, W, H, sh_degree, n_sh, means3D, scales, rotations, shs,
              sh_rest if has_rest else None, Tw2v, Tv2c, campos, trans_mat, radii, colors, gm2, grad_trans,
              grad_colors, grad_normal_opacity, g3, gs, gr, go, gsh, gshr)
    assert rc == 0
    return g3, gs, gr, go, gsh, gshr, gm2


def prepare(W, H, means2D, depths, radii, tiles_touched, return_keys=False):
    P = means2D.shape[0]
    offsets = np.zeros((max(P, 1),), np.int64)
    R = int(lib().oracle_gs_prepare_count(P, _p(np.ascontiguousarray(tiles_touched)), _p(offsets)))
    T = ((W + 15) // 16) * ((H + 15) // 16)
    ranges, pl = np.zeros((T, 2), np.int64), np.zeros((R,), np.int32)
    keys = np.zeros((R,), np.int64) if return_keys else None
    rc = call("gs_prepare_fill", P, W, H, means2D, depths, radii, offsets, R, ranges, pl, keys)
    assert rc == 0
    return (ranges, pl, keys) if return_keys else (ranges, pl)


def render_forward(W, H, means2D, colors, normal_opacity, trans_mat, point_list, ranges, near, far, only_image,
                   trans_mat_t2=None, accum_max_count=None, accum_weights_p=None, accum_weights_count=None):
    dt = means2D.dtype
    P = colors.shape[0]
    oc, oo = np.zeros((3, H, W), dt), np.zeros((H, W), dt)
    oe = None if only_image else np.zeros((9, H, W), dt)
    of = np.zeros((H, W, 2), dt) if (not only_image and trans_mat_t2 is not None) else None
    nc = np.zeros((2, H, W), np.int32)
    rc = call(f"gs_2d_render_forward_{_suffix(dt)}", P, W, H, float(near), float(far), int(only_image), means2D,
              colors, normal_opacity, trans_mat, point_list, ranges, trans_mat_t2, accum_max_count, accum_weights_p,
              accum_weights_count, oc, oo, oe, of, nc)
    assert rc == 0
    return oc, oo, oe, of, nc


def render_backward(means2D, normal_opacity, colors, trans_mat, trans_mat_t2, out_opacity, out_extras, out_flow,
                    dL_dpix, dL_dopacity, dL_dextras, dL_dflow, ranges, point_list, n_contrib, near, far):
    dt = means2D.dtype
    P = means2D.shape[0]
    H, W = dL_dpix.shape[1:]
    gc, gm, gt, gn = np.zeros((P, 3), dt), np.zeros((P, 2), dt), np.zeros((P, 3, 3), dt), np.zeros((P, 4), dt)
    rc = call(f"gs_2d_render_backward_{_suffix(dt)}", P, W, H, float(near), float(far), means2D, normal_opacity,
              colors, trans_mat, trans_mat_t2, out_opacity, out_extras, out_flow, dL_dpix, dL_dopacity, dL_dextras,
              dL_dflow, ranges, point_list, n_contrib, gc, gm, gt, gn)
    assert rc == 0
    return gc, gm, gt, gn


# ---- "fast" path ---------------------------------------------------------------------------------------------------
def fast_preprocess_forward(W, H, sh_degree, means3D, scales, rotations, opacities, shs, sh_rest, Tw2v, Tv2s, campos,
                            trans_precomp=None, means2D=None, culling=None):
    """-> (means2D, colors, trans_mat, inverse_m, normal_opacity, depths, radii, tiles_touched)."""
    dt = means3D.dtype
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.size > 0
    n_sh = sh_rest.shape[1] if has_rest else (shs.shape[1] if sh_degree >= 0 else 0)
    preserve = means2D is not None
    m2 = means2D if preserve else np.zeros((P, 2), dt)
    colors = shs if sh_degree < 0 else np.zeros((P, 3), dt)
    tm = trans_precomp if trans_precomp is not None else np.zeros((P, 3, 3), dt)
    im, no, dep = np.zeros((P, 3, 3), dt), np.zeros((P, 4), dt), np.zeros((P,), dt)
    radii, tt = np.zeros((P,), np.int32), np.zeros((P,), np.int32)
    cul = None if culling is None else np.ascontiguousarray(culling.astype(np.uint8))
    rc = call(f"gs_2d_fast_preprocess_forward_{_suffix(dt)}", P, W, H, sh_degree, n_sh, means3D, scales, rotations,
              opacities, shs, sh_rest if has_rest else None, Tw2v, Tv2s, campos, trans_precomp, cul, int(preserve), m2,
              None if sh_degree < 0 else colors, tm, im, no, dep, radii, tt)
    assert rc == 0
    return m2, colors, tm, im, no, dep, radii, tt


def fast_prepare(W, H, means2D, inverse_m, depths, opacities, radii, tiles_touched, return_keys=False):
    P = means2D.shape[0]
    offsets = np.zeros((max(P, 1),), np.int64)
    R = int(lib().oracle_gs_prepare_count(P, _p(np.ascontiguousarray(tiles_touched)), _p(offsets)))
    T = ((W + 15) // 16) * ((H + 15) // 16)
    ranges, pl = np.zeros((T, 2), np.int64), np.zeros((R,), np.int32)
    keys = np.zeros((R,), np.int64) if return_keys else None
    rc = call("gs_fast_prepare_fill", P, W, H, means2D, inverse_m, depths, np.ascontiguousarray(opacities), radii,
              offsets, R, ranges, pl, keys)
    assert rc == 0
    return (ranges, pl, keys) if return_keys else (ranges, pl)


def fast_preprocess_backward(W, H, sh_degree, means3D, scales, rotations, shs, sh_rest, Tw2v, Tv2s, campos, trans_mat,
                             radii, colors, grad_mean2D, grad_trans, grad_inv_m, grad_colors, grad_normal_opacity):
    dt = means3D.dtype
    P = means3D.shape[0]
    has_rest = sh_rest is not None and sh_rest.size > 0
    n_sh = sh_rest.shape[1] if has_rest else (shs.shape[1] if sh_degree >= 0 else 0)
    g3, gs, gr, go = np.zeros((P, 3), dt), np.zeros((P, 2), dt), np.zeros((P, 4), dt), np.zeros((P, 1), dt)
    gsh = np.zeros_like(shs) if sh_degree >= 0 else None
    gshr = np.zeros_like(sh_rest) if has_rest else None
    gm2 = grad_mean2D.copy()
    rc = call(f"gs_2d_fast_preprocess_backward_{_suffix(dt)}", P, W, H, sh_degree, n_sh, means3D, scales, rotations,
              shs, sh_rest if has_rest else None, Tw2v, Tv2s, campos, trans_mat, radii, colors, gm2, grad_trans,
              grad_inv_m, grad_colors, grad_normal_opacity, g3, gs, gr, go, gsh, gshr)
    assert rc == 0
    return g3, gs, gr, go, gsh, gshr, gm2


def fast_render_forward(W, H, near, far, only_image, means2D, colors, normal_opacity, trans_mat, inverse_m, point_list,
                        ranges, bucket_offset=None, trans_mat_t2=None, accum_max_count=None, accum_weights_p=None,
                        accum_weights_count=None):
    """-> (colors, opacity, extras[8], n_contrib, max_contrib, bucket_to_tile, sampled_T, sampled_acc, sampled_aux
    [B, 8 | 10, 256]) and, when trans_mat_t2 is given, the flow [H,W,2] as a tenth element."""
    dt = means2D.dtype
    oc, oo = np.zeros((3, H, W), dt), np.zeros((H, W), dt)
    oe = None if only_image else np.zeros((8, H, W), dt)
    flow = trans_mat_t2 is not None and not only_image
    of = np.zeros((H, W, 2), dt) if flow else None
    nc = np.zeros((2, H, W), np.int32)
    snap = [None] * 5
    if bucket_offset is not None and not only_image:
        B = int(bucket_offset[-1])
        T = ranges.shape[0]
        snap = [np.zeros((T,), np.int32), np.zeros((B,), np.int32), np.zeros((B, 256), dt), np.zeros((B, 3, 256), dt),
                np.zeros((B, 10 if flow else 8, 256), dt)]
    rc = call(f"gs_2d_fast_render_forward_{_suffix(dt)}", W, H, float(near), float(far), int(only_image), means2D,
              colors, normal_opacity, trans_mat, inverse_m, point_list, ranges, bucket_offset, trans_mat_t2,
              accum_max_count, accum_weights_p, accum_weights_count, oc, oo, oe, of, nc, *snap)
    assert rc == 0
    return (oc, oo, oe, nc) + tuple(snap) + ((of,) if flow else ())


def fast_render_backward(near, far, per_splat_form, means2D, normal_opacity, colors, trans_mat, inverse_m, out_opacity,
                         out_extras, dL_dpix, dL_dopacity, dL_dextras, ranges, point_list, n_contrib,
                         trans_mat_t2=None, out_flow=None, dL_dflow=None):
    dt = means2D.dtype
    P = means2D.shape[0]
    H, W = dL_dpix.shape[1:]
    gc, gm, gt, gi, gn = (np.zeros((P, 3), dt), np.zeros((P, 2), dt), np.zeros((P, 3, 3), dt), np.zeros((P, 3, 3), dt),
                          np.zeros((P, 4), dt))
    rc = call(f"gs_2d_fast_render_backward_{_suffix(dt)}", P, W, H, float(near), float(far), int(per_splat_form),
              means2D, normal_opacity, colors, trans_mat, inverse_m, trans_mat_t2, out_opacity, out_extras, out_flow,
              dL_dpix, dL_dopacity, dL_dextras, dL_dflow, ranges, point_list, n_contrib, gc, gm, gt, gi, gn)
    assert rc == 0
    return gc, gm, gt, gi, gn


# ---- 3D-Gaussian (EWA) path ------------------------------------------------------------------------------------------
def gs3d_preprocess_forward(W, H, sh_degree, is_opengl, means3D, scales, rotations, opacities, shs, sh_rest, Tw2v,
                            Tv2c, campos, tan_fov, culling=None, means2D=None, cov3D_precomp=None,
                            cov2D_precomp=None):
    dt = means3D.dtype
    P = means3D.shape[0]
    n_sh = 0 if sh_degree < 0 else (sh_rest.shape[1] if sh_rest is not None else shs.shape[1])
    m2 = np.zeros((P, 2), dt) if means2D is None else means2D
    depths, conic = np.zeros((P,), dt), np.zeros((P, 4), dt)
    cov3D = cov3D_precomp if cov3D_precomp is not None else np.zeros((P, 6), dt)  # the host returns the input itself
    colors = np.zeros((P, 3), dt) if sh_degree >= 0 else shs
    radii, tt = np.zeros((P,), np.int32), np.zeros((P,), np.int32)
    cull = None if culling is None else np.ascontiguousarray(culling.astype(np.uint8))
    rc = call(f"gs3d_preprocess_forward_{_suffix(dt)}", P, W, H, sh_degree, n_sh, int(is_opengl), means3D, scales,
              rotations, opacities, shs, sh_rest, Tw2v, Tv2c, campos, float(tan_fov[0]), float(tan_fov[1]), cull,
              cov3D_precomp, cov2D_precomp, m2, depths, colors, radii, tt, cov3D, conic)
    assert rc == 0
    return m2, depths, colors, radii, tt, cov3D, conic


def gs3d_preprocess_backward(W, H, sh_degree, is_opengl, means3D, scales, rotations, shs, sh_rest, Tw2v, Tv2c, campos,
                             tan_fov, radii, colors, cov3D, grad_mean2D, grad_colors, grad_conic, cov2D=None,
                             precomputed=False, camera=False):
    """-> (g_means3D, g_scales, g_rot, g_opac, g_shs, g_sh_rest, g_cov, grad_mean2D rewritten) and, with `camera`,
    (g_Tw2v[4,4], g_campos[3]) appended. `cov2D` (pre-computed 2D covariances): g_cov is [P,3]; `precomputed` (cov3D or
    cov2D given by the caller): no scale / rotation gradients, as the reference's wrapper passes None for them."""
    dt = means3D.dtype
    P = means3D.shape[0]
    n_sh = 0 if sh_degree < 0 else (sh_rest.shape[1] if sh_rest is not None else shs.shape[1])
    g3, go = np.zeros((P, 3), dt), np.zeros((P, 1), dt)
    no_sr = precomputed or cov2D is not None
    gs, gq = (None, None) if no_sr else (np.zeros((P, 3), dt), np.zeros((P, 4), dt))
    gsh = np.zeros_like(shs) if sh_degree >= 0 else None
    grest = np.zeros_like(sh_rest) if (sh_degree >= 0 and sh_rest is not None) else None
    gcov = np.zeros((P, 3 if cov2D is not None else 6), dt)
    gm2 = np.ascontiguousarray(grad_mean2D.copy())
    gv, gcam = (np.zeros((4, 4), dt), np.zeros((3,), dt)) if camera else (None, None)
    rc = call(f"gs3d_preprocess_backward_{_suffix(dt)}", P, W, H, sh_degree, n_sh, int(is_opengl), means3D, scales,
              rotations, shs, sh_rest, Tw2v, Tv2c, campos, float(tan_fov[0]), float(tan_fov[1]), radii, colors, cov3D,
              cov2D, gm2, grad_colors, grad_conic, g3, gs, gq, go, gsh, grest, gcov, gv, gcam)
    assert rc == 0
    out = (g3, gs, gq, go, gsh, grest, gcov, gm2)
    return out + (gv, gcam) if camera else out


def gs3d_extra_forward(W, H, extras, means2D, conic_opacity, ranges, point_list, n_contrib):
    """gaussian_rasterize_extra_forward -> pixel_extras [H,W,E] (gaussian_rasterizer_extra.cu:317-339)."""
    E = extras.shape[1]
    out = np.zeros((H, W, E), extras.dtype)
    assert call(f"gs3d_extra_forward_{_suffix(extras.dtype)}", W, H, E, extras, means2D, conic_opacity, ranges,
                point_list, n_contrib, out) == 0
    return out


def gs3d_extra_backward(W, H, extras, out_opacity, grad_out, means2D, conic_opacity, ranges, point_list, n_contrib,
                        want=(True, True, True)):
    """gaussian_rasterize_extra_backward -> (g_extras, g_means2D, g_conic_opacity), None where not wanted
    (gaussian_rasterizer_extra.cu:341-365)."""
    P, E = extras.shape
    dt = extras.dtype
    ge = np.zeros((P, E), dt) if want[0] else None
    gm = np.zeros((P, 2), dt) if want[1] else None
    gc = np.zeros((P, 4), dt) if want[2] else None
    assert call(f"gs3d_extra_backward_{_suffix(dt)}", W, H, E, extras, out_opacity, np.ascontiguousarray(grad_out),
                means2D, conic_opacity, ranges, point_list, n_contrib, ge, gm, gc) == 0
    return ge, gm, gc


def gs3d_topk_weights(topk, W, H, means2D, conic_opacity, ranges, point_list):
    """gaussian_topk_weights -> (top_indices[H,W,K] int32, top_weights[H,W,K]) (gaussian_topk.cu:212-228)."""
    ti = np.zeros((H, W, topk), np.int32)
    tw = np.zeros((H, W, topk), means2D.dtype)
    assert call(f"gs3d_topk_weights_{_suffix(means2D.dtype)}", topk, W, H, means2D, conic_opacity, ranges, point_list,
                ti, tw) == 0
    return ti, tw


def gs3d_compute_cov3D(q, s):
    """gs_compute_cov3D_forward(q, s) -> cov3D [N,6] (gaussian_compute_cov3D.cu:122-137)."""
    N = s.shape[0]
    out = np.zeros((N, 6), s.dtype)
    assert call(f"gs3d_compute_cov3D_{_suffix(s.dtype)}", N, q, s, out) == 0
    return out


def gs3d_compute_cov3D_backward(q, s, g):
    """gs_compute_cov3D_backward(q, s, dL_dcov3D) -> (dq, ds) (gaussian_compute_cov3D.cu:151-161)."""
    N = s.shape[0]
    gq, gs = np.zeros((N, 4), s.dtype), np.zeros((N, 3), s.dtype)
    assert call(f"gs3d_compute_cov3D_backward_{_suffix(s.dtype)}", N, q, s, g, gq, gs) == 0
    return gq, gs


def gs3d_compute_cov2D(cov3D, mean, Tw2v, fx, fy, tanx, tany):
    """gs_compute_cov2D_forward -> cov2D [N,3] with the 0.3 low-pass term (gaussian_compute_cov2D.cu:199-210)."""
    N = mean.shape[0]
    out = np.zeros((N, 3), mean.dtype)
    assert call(f"gs3d_compute_cov2D_{_suffix(mean.dtype)}", N, cov3D, mean, Tw2v, float(fx), float(fy), float(tanx),
                float(tany), out) == 0
    return out


def gs3d_compute_cov2D_backward(cov3D, mean, Tw2v, fx, fy, tanx, tany, g, grad_vm=None):
    """gs_compute_cov2D_backward -> (grad_cov3D, grad_mean); with grad_vm[4,4] the view matrix's gradient is added to
    its first three rows (gaussian_compute_cov2D.cu:229-248)."""
    N = mean.shape[0]
    gc, gm = np.zeros((N, 6), mean.dtype), np.zeros((N, 3), mean.dtype)
    assert call(f"gs3d_compute_cov2D_backward_{_suffix(mean.dtype)}", N, cov3D, mean, Tw2v, float(fx), float(fy),
                float(tanx), float(tany), g, gc, gm, grad_vm) == 0
    return gc, gm


def gs3d_render_forward(W, H, means2D, conic_opacity, colors, extras, point_list, ranges, accum_max_count=None,
                        accum_weights_p=None, accum_weights_count=None, bucket_offset=None):
    """-> (colors, opacity, extras, n_contrib) and, with bucket_offset, (max_contrib[T], bucket_to_tile[B],
    sampled_T[B,256], sampled_ar[B,3+E,256]) appended."""
    dt = means2D.dtype
    E = 0 if extras is None else extras.shape[1]
    oc, oo = np.zeros((3, H, W), dt), np.zeros((H, W), dt)
    oe = np.zeros((E, H, W), dt) if E else None
    nc = np.zeros((H, W), np.int32)
    snap = [None] * 4
    if bucket_offset is not None:
        B = int(bucket_offset[-1]) if bucket_offset.size else 0
        snap = [np.zeros((ranges.shape[0],), np.int32), np.zeros((B,), np.int32), np.zeros((B, 256), dt),
                np.zeros((B, 3 + E, 256), dt)]
    rc = call(f"gs3d_render_forward_{_suffix(dt)}", W, H, E, means2D, conic_opacity, colors, extras, point_list, ranges,
              oc, oo, oe, nc, accum_max_count, accum_weights_p, accum_weights_count, bucket_offset, *snap)
    assert rc == 0
    return (oc, oo, oe, nc) + (tuple(snap) if bucket_offset is not None else ())


def gs3d_render_fast_backward(W, H, means2D, conic_opacity, colors, extras, images, out_extras, out_opacity, n_contrib,
                              max_contrib, bucket_offset, bucket_to_tile, sampled_T, sampled_ar, dL_dpix, dL_dextras,
                              dL_dopacity, point_list, ranges):
    """gaussian_rasterize_fast_backward -> (g_colors, g_extras, g_means2D, g_conic_opacity)"""
    dt = means2D.dtype
    P = means2D.shape[0]
    E = 0 if extras is None else extras.shape[1]
    gm, gc, gcol = np.zeros((P, 2), dt), np.zeros((P, 4), dt), np.zeros((P, 3), dt)
    gex = np.zeros((P, E), dt) if E else None
    B = int(bucket_offset[-1]) if bucket_offset.size else 0
    rc = call(f"gs3d_render_fast_backward_{_suffix(dt)}", W, H, E, means2D, conic_opacity, colors, extras, images,
              out_extras, out_opacity, n_contrib, max_contrib, bucket_offset, bucket_to_tile, sampled_T, sampled_ar,
              dL_dpix, dL_dextras, dL_dopacity, point_list, ranges, B, gm, gc, gcol, gex)
    assert rc == 0
    return gcol, gex, gm, gc


def gs3d_render_backward(W, H, means2D, conic_opacity, colors, extras, out_opacity, n_contrib, dL_dpix, dL_dextras,
                         dL_dopacity, point_list, ranges):
    """-> (g_colors, g_extras, g_means2D, g_conic_opacity)"""
    dt = means2D.dtype
    P = means2D.shape[0]
    E = 0 if extras is None else extras.shape[1]
    gm, gc, gcol = np.zeros((P, 2), dt), np.zeros((P, 4), dt), np.zeros((P, 3), dt)
    gex = np.zeros((P, E), dt) if E else None
    rc = call(f"gs3d_render_backward_{_suffix(dt)}", W, H, E, means2D, conic_opacity, colors, extras, out_opacity,
              n_contrib, dL_dpix, dL_dextras, dL_dopacity, point_list, ranges, gm, gc, gcol, gex)
    assert rc == 0
    return gcol, gex, gm, gc
