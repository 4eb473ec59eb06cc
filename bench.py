#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: forward + backward frames/s of the 2DGS surfel renderer on the
300k-surfel 800x800 synthetic scene (preprocess -> binning -> blend -> blend backward -> preprocess backward),
with the roofline position of the dominant kernel and the CPU oracle timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line. Only one GPU is supported: --gpus N with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

import numpy as np
import torch

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
ROOT = os.path.dirname(os.path.abspath(__file__))
# Hardware-counter summary of the dominant kernel (two rocprofv3 --pmc passes, calibrated against the copy probe).
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gs_2d_render_backward_300k_800x800.pmc_traffic.txt")
SQ_SUMMARY = os.path.join(ROOT, "profiles", "blend_knn_mlp_kernels_default_bench.pmc_sq.txt")


# The operator whose kernels take the largest share of a step; the run checks that this is still so.
DOMINANT = 'gs_2d_render_backward'


def measured_traffic(kernel: str):
    """HBM bytes per launch of `kernel` from the committed counter summary (a line `<kernel>.traffic_bytes = N`)."""
    try:
        with open(TRAFFIC_SUMMARY) as f:
            for line in f:
                if line.startswith(kernel + ".traffic_bytes"):
                    return int(float(line.split("=")[1].split()[0]))
    except OSError:
        pass
    return None


def measured_valu_issue(kernel: str):
    """Share of the chip's vector-ALU issue slots the operator's blend kernel filled, from the committed counter summary
    (a line `<kernel>.valu_issue_frac = x`)."""
    try:
        with open(SQ_SUMMARY) as f:
            for line in f:
                if line.startswith(kernel + ".valu_issue_frac"):
                    return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def copy_probe_gbps(dev, nbytes: int = 1 << 30, reps: int = 10) -> float:
    """Achievable HBM bandwidth: read + write bytes of a plain streaming copy kernel per second."""
    from fast_sp_gs_amd import lib as L
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    lib, stream = L.load(), L.current_stream()
    for _ in range(2):
        L.check(lib.fsgs_copy_probe(L.ptr(src), L.ptr(dst), nbytes, stream), 'copy_probe')
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        lib.fsgs_copy_probe(L.ptr(src), L.ptr(dst), nbytes, stream)
    e1.record()
    torch.cuda.synchronize()
    return 2.0 * nbytes * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9


def algorithmic_bytes(stage: str, P: int, Pv: int, R: int, T: int, HW: int) -> int:
    """Algorithmic HBM bytes of one launch of each stage at SH degree 3 (192 B of SH per surfel), 6 sort passes."""
    S = 192
    table = {
        'gs_2d_preprocess_forward': P * (12 + 8 + 16 + 4 + S) + Pv * 76 + P * 8,
        'gs_prepare_scan': P * 12,
        'gs_prepare_fill': P * 24 + R * 12 + R * 12 * 2 * 6 + R * 8 + R * 8 + T * 16,
        'gs_2d_render_forward': 76 * R + 16 * T + 60 * HW,
        'gs_2d_render_backward': 76 * R + 16 * T + 60 * HW + 72 * (P + Pv),
        'gs_2d_preprocess_backward': 4 * P + Pv * (352 + 240),
        'gs_2d_pack_records': P * (72 + 12 + 80),  # optional packed per-surfel records: read 4 tensors, write 80 B
        # fused per-pixel epilogue: reads extras 0-4, opacity, image (9 planes), writes 11; the backward reads 2 depth
        # planes, opacity and 9 gradient planes, writes dL/dextras (9) and dL/dopacity (1)
        'gs_2d_epilogue_forward': HW * 4 * (9 + 11),
        'gs_2d_epilogue_backward': HW * 4 * (12 + 10),
    }
    return int(table[stage])


def cpu_baseline(scene, cam, budget_s: float = 20.0):
    """The CPU oracle (scalar C++ restatement, OpenMP over pixels/surfels) on the same workload, whole frames until
    about `budget_s` seconds are spent. A reported baseline, not a target."""
    import oracle as O
    n = lambda t: np.ascontiguousarray(t.cpu().numpy())
    s = {k: n(getattr(scene, k)) for k in ('means3D', 'scales', 'rotations', 'opacities', 'shs')}
    Tw2v, Tv2c, campos = n(cam.Tw2v), n(cam.Tv2c), n(cam.campos)
    gi, ge = n(scene.extra['grad_image']), n(scene.extra['grad_extras'])
    W, H = cam.W, cam.H
    frames, t0 = 0, time.perf_counter()
    while True:
        m2, colors, tm, no, dep, radii, tt = O.preprocess_forward(W, H, 3, s['means3D'], s['scales'], s['rotations'],
                                                                  s['opacities'], s['shs'], None, Tw2v, Tv2c, campos)
        ranges, pl = O.prepare(W, H, m2, dep, radii, tt)
        oc, oo, oe, _, nc = O.render_forward(W, H, m2, colors, no, tm, pl, ranges, cam.near, cam.far, False)
        # the per-pixel epilogue between the two blend passes, as in the GPU step
        z = lambda *shape: np.zeros(shape, np.float32)
        bg = np.ones(3, np.float32)
        O.call("gs_2d_epilogue_forward_f32", W, H, 1.0, Tw2v, Tv2c, oe, oo, oc, bg, z(3, H, W), z(1, H, W), z(1, H, W),
               z(3, H, W), z(3, H, W))
        ge2, go = z(9, H, W), z(H, W)
        O.call("gs_2d_epilogue_backward_f32", W, H, 1.0, Tw2v, Tv2c, oe, oo, bg, np.ascontiguousarray(ge[1:4]),
               np.ascontiguousarray(ge[4:5]), np.ascontiguousarray(ge[0:1]), None, np.ascontiguousarray(ge[5:6]), gi,
               ge2, go)
        gc, gm, gt, gn = O.render_backward(m2, no, colors, tm, None, oo, oe, None, gi, go, ge2, None, ranges, pl, nc,
                                           cam.near, cam.far)
        O.preprocess_backward(W, H, 3, s['means3D'], s['scales'], s['rotations'], s['shs'], None, Tw2v, Tv2c, campos,
                              tm, radii, colors, gm, gt, gc, gn)
        frames += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or frames >= 8:
            break
    return {"value": frames / dt, "unit": "frames/s", "cores": O.num_threads(), "kind": "port",
            "sample": f"{frames} full fwd+bwd frame(s) of the same 300k-surfel 800x800 workload ({dt:.1f} s), "
                      f"host has {os.cpu_count()} logical cpus"}


def dynamic_step_rate(dev, steps: int = 50, warmup: int = 10):
    """Config 3 (dynamic scene, 200k surfels, 512 control points): bf16 MFMA deformation MLP on the control points ->
    K-NN (k = 4) -> LBS -> render forward -> 0.8 L1 + 0.2 (1 - SSIM) (fused SSIM kernel) -> render backward -> masked Adam
    on the surfel parameters + Adam on the MLP weights and the control points (gradients reach them through the LBS and
    K-NN backward kernels and the MLP's MFMA backward kernels). The render takes `accum_max_count` as the reference's
    training render does (network.py:706). Ten warm-up steps: the caching allocator and the optimisers' state settle
    over the first few."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd.dynamic_step import DynamicStep
    scene_h, cam_h = scenes.config2(P=200_000, size=800, seed=2)
    scene, cam = scene_h.to(dev), cam_h.to(dev)
    g = torch.Generator().manual_seed(2)
    ctrl = (torch.rand(512, 3, generator=g) * 2 - 1).to(dev)
    target = torch.rand(3, cam.H, cam.W, generator=g).to(dev)
    # the fourth head gives each control point its rotation (6-DoF warp). A tiny rate for the network and the control
    # points keeps the random-target synthetic scene from drifting (Adam's steps are |lr| whatever the gradient, and the
    # scale residuals are added after the activation, network.py:643), so every timed step sees the same workload
    state = DynamicStep(scene, cam, ctrl, target, K=4, temperature=0.01, local_frame=True, warp_method='LBS',
                        LBS_method='dist', lr=1.6e-4, net_lr=1e-7, lambda_dssim=0.2)

    def step(i):
        state.step(torch.full((1,), (i % 17) / 17.0, device=dev))

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()  # as in the main measurement: no cyclic-collector stalls inside the timed region
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    gc.enable()
    return steps / dt


def _timed_ms(fn, reps: int = 20, warm: int = 3) -> float:
    """Average device time of `fn` (events on the current stream, the one the operators launch on)."""
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def standalone_ops(dev, copy_gbps: float):
    """The operators of the stand-alone benchmark configuration (1M directions, 200 000 x 512 points) and the optimiser, each with its algorithmic bytes, the rate those
    bytes give over the measured time, and that rate as a share of the 8 TB/s peak and of the copy probe:
    SH encoder forward / backward at 1M directions (shencoder.cu:657-691), SH -> RGB forward / backward at 1M points
    (ops_3d/spherical_harmonics.cu:15-16, 68-70), the LBS blend forward / backward at 200 000 x 512, K = 4
    (network.py:545-573), the masked Adam at 300 000 x 58 floats (adam_masked_update.cu:9-38), one launch per parameter
    tensor as the reference's optimiser loop does and all six in one launch. Output tensors are allocated outside the
    timed calls wherever the operator takes them as arguments."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    c1 = scenes.config1()
    out = {}

    def record(name, ms, nbytes, unit_count=None, unit=None):
        gbps = nbytes / (ms * 1e-3) / 1e9
        out[name] = {"ms": round(ms, 4), "algorithmic_bytes": int(nbytes), "GBps": round(gbps, 1),
                     "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "frac_of_copy_probe": round(gbps / copy_gbps, 4)}
        if unit_count:
            out[name][unit] = unit_count / (ms * 1e-3)

    # ---- SH encoder, degree 3: [B,3] -> [B,16]
    dirs = c1['dirs'].to(dev)
    B, deg = dirs.shape[0], 3
    n_coef = (deg + 1) ** 2
    enc = torch.empty(B, n_coef, device=dev)
    g_enc, g_dirs = torch.randn(B, n_coef, device=dev), torch.zeros(B, 3, device=dev)
    record("sh_encode_forward_1m", _timed_ms(lambda: f('sh_encode_forward')(dirs, enc, B, 3, deg)),
           B * (12 + 4 * n_coef), B, "directions_per_s")
    record("sh_encode_backward_1m", _timed_ms(lambda: f('sh_encode_backward')(g_enc, dirs, B, 3, deg, g_dirs)),
           B * (4 * n_coef + 12 + 12), B, "directions_per_s")
    # ---- SH -> RGB, degree 3: positions + camera centre + [B,16,3] coefficients -> rgb; backward writes dSH and d(pos)
    shs = c1['shs'].to(dev)
    campos = torch.tensor([0.0, 0.0, 4.0], device=dev)
    rgb = f('SH_to_RGB_forward')(dirs, campos, shs, deg, True)
    g_rgb, g_sh, g_pos, g_cam = torch.randn_like(rgb), torch.empty_like(shs), torch.empty_like(dirs), torch.zeros(3, device=dev)
    record("sh_to_rgb_forward_1m", _timed_ms(lambda: f('SH_to_RGB_forward')(dirs, campos, shs, deg, True)),
           B * (12 + 12 * n_coef + 12), B, "points_per_s")
    record("sh_to_rgb_backward_1m",
           _timed_ms(lambda: f('SH_to_RGB_backward')(deg, True, dirs, campos, shs, rgb, g_rgb, g_pos, g_cam, g_sh)),
           B * (12 + 12 * n_coef + 12 + 12) + B * (12 * n_coef + 12), B, "points_per_s")
    del enc, g_enc, g_dirs, shs, g_sh, g_pos, rgb, g_rgb
    # ---- LBS blend, 200 000 points x 512 control points, K = 4, weights softmax(-d^2 / 0.01), rigid transforms
    pts, ctrl = c1['points'].to(dev), c1['ctrl'].to(dev)
    sp_t, sp_r, sp_s = c1['sp_t'].to(dev), c1['sp_r'].to(dev), c1['sp_s'].to(dev)
    sp_rot = sp_r.clone()
    N, M, K, S = pts.shape[0], ctrl.shape[0], 4, sp_s.shape[1]
    d2, idx = f('knn_topk')(pts, ctrl, K)
    fwd = lambda: f('lbs_blend')(pts, ctrl, sp_t, sp_r, sp_s, d2, idx, 0.01, 'LBS', sp_rot, 'dist')
    g_xyz, g_rot, g_scale = torch.randn(N, 3, device=dev), torch.randn(N, 4, device=dev), torch.randn(N, S, device=dev)
    bwd = lambda: f('lbs_blend_backward')(pts, ctrl, sp_t, sp_r, sp_s, d2, idx, g_xyz, g_rot, g_scale, 0.01, 'LBS',
                                          sp_rot, 'dist')
    record("lbs_blend_forward_200k_512_k4", _timed_ms(fwd), N * (12 + K * (8 + 4)) + M * 28 + N * 12, N, "points_per_s")
    # backward: points, pair inputs, indices and the three upstream gradients in; g_points and g_pair out; per
    # control point 3 + 3 + 4 + 4 + S floats in and out
    record("lbs_blend_backward_200k_512_k4", _timed_ms(bwd),
           N * (12 + K * 12 + 12 + 16 + 4 * S) + N * (12 + 4 * K) + 2 * M * 4 * (14 + S), N, "points_per_s")
    # ---- masked Adam: the six parameter tensors of a 2DGS point set (3 + 3 + 45 + 1 + 2 + 4 = 58 floats per surfel)
    P, widths = 300_000, (3, 3, 45, 1, 2, 4)
    g = torch.Generator().manual_seed(4)
    mask = (torch.rand(P, generator=g) < 0.9).to(dev)
    params = [torch.randn(P, w, generator=g).to(dev) for w in widths]
    grads = [torch.randn(P, w, generator=g).to(dev) for w in widths]
    m1, m2 = [torch.zeros_like(t) for t in params], [torch.zeros_like(t) for t in params]
    n_vis = int(mask.sum())
    adam_bytes = len(widths) * P + n_vis * sum(widths) * 28  # the mask is read once per tensor
    one = f('AdamMasksedUpdated')

    def per_tensor():
        for t, gr, a, b, w in zip(params, grads, m1, m2, widths):
            one(t, gr, a, b, mask, 1.6e-4, 0.9, 0.999, 1e-15, P, w)

    record("adam_masked_6_launches_300k_58", _timed_ms(per_tensor), adam_bytes)
    multi = f('AdamMasksedUpdatedMulti')
    record("adam_masked_1_launch_300k_58",
           _timed_ms(lambda: multi(params, grads, m1, m2, mask, [1.6e-4] * 6, 0.9, 0.999, [1e-15] * 6, P)), adam_bytes)
    out["workload"] = ("config 1: 1M unit directions / points at SH degree 3; 200000 x 512 control points, K = 4, rigid "
                       "transforms, 'dist' weights; masked Adam on 300000 surfels x 58 floats, 90 % visible. Times are "
                       "device time per call including the Python wrapper's output allocation where the operator allocates")
    return out


def simple_knn_ms(dev, scene):
    """simple_knn (mean squared 3-NN distance, used to initialise the surfel scales) on the benchmark scene's 300k
    centres and on 3M uniform points."""
    from fast_sp_gs_amd._C import get_C_function
    fn = get_C_function('simple_knn')
    out = {}
    big = torch.rand(3_000_000, 3, generator=torch.Generator().manual_seed(5)).to(dev)
    for name, pts in (("simple_knn_300k_ms", scene.means3D.contiguous()), ("simple_knn_3m_ms", big)):
        fn(pts)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            fn(pts)
        torch.cuda.synchronize()
        out[name] = (time.perf_counter() - t0) / 3 * 1e3
    return out


def reference_note_blend_ms(dev, reps: int = 100):
    """The only timing the reference records for this path (developer note at
    fast_2d_gs/renderer/gs_2d_fast_render.py:1288-1292, GPU not stated): the two standard blend kernels alone on
    102 400 surfels with means ~ N(0,1), scales ~ U[0,1], opacity ~ U[0,1], 128 x 128 pixels, focal 500, camera at
    (0,0,4), auxiliary maps and optical flow on (_gen_random_data :883-910, test_rasterize_fast :1185-1287), 100
    iterations after a warm-up. Same workload, same two operators, same arguments here."""
    import math
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function as f
    g = torch.Generator().manual_seed(1234)
    P, W, H = 102_400, 128, 128
    means3D = torch.randn(P, 3, generator=g).to(dev)
    scales = torch.rand(P, 2, generator=g).to(dev)
    rot = torch.nn.functional.normalize(torch.randn(P, 4, generator=g), dim=-1).to(dev)
    opac = torch.rand(P, 1, generator=g).to(dev)
    shs = torch.randn(P, 1, 3, generator=g).to(dev)
    cam = scenes.pinhole(W, H, math.degrees(2 * math.atan(W / 2 / 500.0)), torch.tensor([0.0, 0.0, 4.0])).to(dev)
    m2, colors, tm, no, depths, radii, tt = f('gs_2d_preprocess_forward')(
        W, H, 0, False, means3D, scales, rot, opac, shs, None, cam.Tw2v, cam.Tv2c, cam.campos, None, None, None)
    ranges, point_list = f('GS_prepare')(W, H, m2, depths, radii, tt, False)
    Tw2c = (cam.Tv2c @ cam.Tw2v).contiguous()
    t2 = f('gs_2d_compute_transmat_forward')(W, H, (means3D + 0.1 * torch.randn(P, 3, generator=g).to(dev)).contiguous(),
                                             scales, rot, cam.Tw2v, Tw2c)[0]
    t2 = (t2 * (radii[:, None, None] > 0)).contiguous()
    fwd, bwd = f('GS_2D_render_forward'), f('GS_2D_render_backward')
    run_f = lambda: fwd(W, H, m2, colors, no, tm, point_list, ranges, 0.2, 100.0, False, t2, None, None, None)
    oc, oo, oe, of, nc = run_f()
    gi, go = torch.randn(3, H, W, generator=g).to(dev), torch.randn(H, W, generator=g).to(dev)
    ge = torch.randn(9, H, W, generator=g).to(dev)
    ge[5:] = 0
    gf = torch.randn(H, W, 2, generator=g).to(dev)
    run_b = lambda: bwd(m2, no, colors, tm, t2, oo, oe, of, gi, go, ge, gf, ranges, point_list, nc, 0.2, 100.0)
    run_b()
    torch.cuda.synchronize()
    e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    e[0].record()
    for _ in range(reps):
        run_f()
    e[1].record()
    for _ in range(reps):
        run_b()
    e[2].record()
    torch.cuda.synchronize()
    return {"reference_note_blend_forward_ms": e[0].elapsed_time(e[1]) / reps,
            "reference_note_blend_backward_ms": e[1].elapsed_time(e[2]) / reps,
            "reference_note_workload": f"102400 surfels N(0,1), scales U[0,1], 128x128, focal 500, aux + flow, "
                                       f"R = {int(point_list.numel())}; the reference's own note for its CUDA kernels on "
                                       f"an unnamed GPU: forward 0.092-0.100 ms, backward 0.678-0.718 ms"}


def gs3d_path_rate(dev, scene, cam, gi, steps: int = 30, warmup: int = 5):
    """The 3D-Gaussian (EWA) path on the benchmark scene with a third scale per Gaussian: preprocess -> binning ->
    conic blend -> blend backward -> preprocess backward through the raw operators."""
    from fast_sp_gs_amd._C import get_C_function as f
    g = torch.Generator().manual_seed(11)
    scales = torch.cat([scene.scales.cpu(), scene.scales[:, :1].cpu() * (0.5 + torch.rand(scene.P, 1, generator=g))],
                       1).to(dev).contiguous()
    W, H = cam.W, cam.H
    tan_fov = (W / 2 / float(cam.Tv2s[0, 0]), H / 2 / float(cam.Tv2s[1, 1]))
    go = -gi.sum(0)  # white-background composite
    R = [0]

    def step(ordered=True, cull=False):
        m2, dep, col, rad, tt, c3, co = f('gs_preprocess_forward')(
            W, H, 3, False, scene.means3D, scales, scene.rotations, scene.opacities, scene.shs, None, cam.Tw2v,
            cam.Tv2c, cam.campos, tan_fov, None, None, None, None)
        # cull: lists without the (Gaussian, tile) instances that no pixel of their tile can blend (what
        # RasterizeGaussians bins by default); otherwise the reference's lists
        keep = f('gs_cull_masks')(W, H, m2, co, rad) if cull else None
        ranges, pl, offsets = f('GS_prepare')(W, H, m2, dep, rad, tt, False, return_offsets=True, cull=cull,
                                              keep_masks=keep)[:3]
        oc, oo, _, nc = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges)
        # per-Gaussian sums through ordered per-instance records, or the reference's atomics (RasterizeGaussians' default)
        g_col, _, g_m2, g_co = f('gaussian_rasterize_backward')(m2, co, col, None, oo, gi, go, None, ranges, pl, nc,
                                                                offsets if ordered else None, rad if ordered else None,
                                                                culled=keep if ordered else None)
        g3, gs, gq = torch.empty_like(scene.means3D), torch.empty_like(scales), torch.empty_like(scene.rotations)
        gop, gsh = torch.empty_like(scene.opacities), torch.empty_like(scene.shs)
        f('gs_preprocess_backward')(W, H, 3, False, scene.means3D, scales, scene.rotations, scene.opacities, scene.shs,
                                    None, cam.Tw2v, cam.Tv2c, cam.campos, tan_fov, c3, None, rad, col, g_m2, None, g_col,
                                    g_co, g3, gs, gq, gop, gsh, None, None)
        if not cull:
            R[0] = pl.numel()
        return m2, co, ranges, pl, nc, oo

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()
    t0 = time.perf_counter()
    for _ in range(steps):
        state = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for _ in range(warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(False)
    torch.cuda.synchronize()
    dt_atomic = time.perf_counter() - t0
    for _ in range(warmup):
        culled_state = step(False, True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(False, True)
    torch.cuda.synchronize()
    dt_culled = time.perf_counter() - t0
    gc.enable()
    R_culled = int((culled_state[2][:, 1] - culled_state[2][:, 0]).sum())
    del culled_state

    # a 16-channel feature table blended with the finished view's weights, and its backward
    m2, co, ranges, pl, nc, oo = state
    feat = torch.randn(scene.P, 16, generator=g).to(dev)
    g_out = torch.randn(H, W, 16, generator=g).to(dev)
    g_feat, g_m2, g_co = torch.zeros_like(feat), torch.zeros_like(m2), torch.zeros_like(co)
    x_f = lambda: f('gaussian_rasterize_extra_forward')(W, H, feat, m2, co, ranges, pl, nc)
    x_b = lambda: f('gaussian_rasterize_extra_backward')(W, H, feat, oo, g_out, m2, co, ranges, pl, nc, g_feat, g_m2,
                                                         g_co)
    x_f(), x_b()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    ev[0].record()
    for _ in range(10):
        x_f()
    ev[1].record()
    for _ in range(10):
        x_b()
    ev[2].record()
    torch.cuda.synchronize()
    # the two backward decompositions on that view: one block per tile walking its list back to front (both operator
    # names by default) against the reference's second algorithm, one lane per list entry with the pixels passed from
    # lane to lane from the forward's bucket snapshots (gaussian_render.cu:540-694)
    col = f('gs_preprocess_forward')(W, H, 3, False, scene.means3D, scales, scene.rotations, scene.opacities,
                                     scene.shs, None, cam.Tw2v, cam.Tv2c, cam.campos, tan_fov, None, None, None, None)[2]
    lens = ranges[:, 1] - ranges[:, 0]
    b_off = torch.cumsum((lens + 31) // 32, 0).contiguous()
    oc, oo2, _, nc2, max_c, b2t, s_T, s_ar = f('gaussian_rasterize_forward')(W, H, m2, co, col, None, pl, ranges, None,
                                                                           None, None, b_off)
    fast_bwd = f('gaussian_rasterize_fast_backward')
    bwd_ms = {}
    for name, per_gaussian in (("tile", False), ("per_gaussian", True)):
        call = lambda: fast_bwd(m2, co, col, None, oc, None, oo2, gi, go, None, ranges, pl, nc2, max_c, b_off, b2t, s_T,
                                s_ar, per_gaussian=per_gaussian)
        bwd_ms[name] = _timed_ms(call, reps=10)

    return {"gs3d_path_frames_per_s": steps / dt,
            "gs3d_path_atomic_sums_frames_per_s": steps / dt_atomic,
            "gs3d_path_culled_lists_atomic_sums_frames_per_s": steps / dt_culled,
            "gs3d_path_culled_lists_instances": R_culled,
            "gs3d_backward_tile_kernel_ms": bwd_ms["tile"],
            "gs3d_backward_per_gaussian_kernel_ms": bwd_ms["per_gaussian"],
            "gs3d_backward_workload": f"gaussian_rasterize_fast_backward on that view with atomic sums, {b2t.numel()} "
                                      f"buckets of 32 entries: back-to-front tile kernel / the reference's "
                                      f"per-Gaussian decomposition (wavefront = 64 entries)",
            "gs3d_path_workload": f"same 300k centres as 3D Gaussians (third scale added), 800x800, SH degree 3, "
                                  f"R = {R[0]}: gs_preprocess fwd/bwd + GS_prepare + gaussian_rasterize fwd/bwd",
            "gs3d_extra16_forward_ms": ev[0].elapsed_time(ev[1]) / 10,
            "gs3d_extra16_backward_ms": ev[1].elapsed_time(ev[2]) / 10,
            "gs3d_extra16_workload": "gaussian_rasterize_extra_forward / _backward, a [300000,16] table on that view"}


def density_control_ms(dev, scene, reps: int = 5):
    """Densify (clone + split) and prune of the 300k-point set with populated Adam moments: the table-driven kernels
    against the same operations done the reference's way (boolean indexing / cat / repeat per tensor and per moment,
    gaussian_splatting.py:497-636) with torch on the same GPU."""
    from fast_sp_gs_amd.adaptive_control import GaussianPoints
    from fast_sp_gs_amd._C import get_C_function as f
    P = scene.P
    g = torch.Generator().manual_seed(5)
    acc = (torch.rand(P, 1, generator=g) * 4e-4).to(dev)
    den = torch.randint(1, 3, (P, 1), generator=g).float().to(dev)
    radii = (torch.rand(P, generator=g) * 30).to(dev)

    def fresh():
        m = GaussianPoints(scene.means3D, scene.shs[:, :1].contiguous(), scene.shs[:, 1:].contiguous(),
                           torch.log(scene.scales), scene.rotations, torch.logit(scene.opacities.clamp(1e-4, 1 - 1e-4)))
        opt = torch.optim.Adam(m.param_groups(1e-3), eps=1e-15)
        for grp in opt.param_groups:
            grp['params'][0].grad = torch.zeros_like(grp['params'][0])
        opt.step()
        m.xyz_gradient_accum, m.denom, m.max_radii2D = acc.clone(), den.clone(), radii.clone()
        return m, opt

    def ours(m, opt):
        m.densify(opt, 2e-4, 4.0, 0.01)
        m.max_radii2D = radii[:1].expand(m._xyz.shape[0]).contiguous()
        m.prune(opt, 0.05, 4.0, 20.0, 0.1)

    def reference_way(m, opt):  # the reference's sequence with torch indexing, one tensor and one moment at a time
        names = m.param_names_map

        def change(tensors, op):
            for grp in opt.param_groups:
                old = grp['params'][0]
                t = tensors[grp['name']] if isinstance(tensors, dict) else tensors
                new = torch.nn.Parameter(torch.cat([old, t]) if op == 'concat' else old[t])
                st = opt.state.pop(old)
                for k in ('exp_avg', 'exp_avg_sq'):
                    st[k] = torch.cat([st[k], torch.zeros_like(t)]) if op == 'concat' else st[k][t]
                grp['params'][0] = new
                opt.state[new] = st
                setattr(m, [a for a, n in names.items() if n == grp['name']][0], new)
            m.training_setup() if op == 'concat' else None

        grads = m.xyz_gradient_accum / m.denom
        grads[grads.isnan()] = 0.0
        sel = (torch.norm(grads, dim=-1) >= 2e-4) & (torch.amax(m.get_scaling, dim=1) <= 0.04)
        change({n: getattr(m, a)[sel] for a, n in names.items()}, 'concat')
        Pn = m._xyz.shape[0]
        padded = torch.zeros(Pn, device=dev)
        padded[:grads.shape[0]] = grads.squeeze()
        sel = (padded >= 2e-4) & (torch.amax(m.get_scaling, dim=1) > 0.04)
        stds = m.get_scaling[sel].repeat(2, 1)
        stds = torch.cat([stds, 0 * torch.ones_like(stds[:, :1])], dim=-1)
        samples = torch.normal(mean=torch.zeros_like(stds), std=stds)
        q = torch.nn.functional.normalize(m._rotation[sel], dim=-1)
        x, y, z, w = q.unbind(-1)
        R = torch.stack([1 - 2 * y * y - 2 * z * z, 2 * x * y - 2 * w * z, 2 * w * y + 2 * x * z,
                         2 * x * y + 2 * w * z, 1 - 2 * x * x - 2 * z * z, 2 * y * z - 2 * w * x,
                         2 * x * z - 2 * w * y, 2 * w * x + 2 * y * z, 1 - 2 * x * x - 2 * y * y], -1).reshape(-1, 3, 3)
        new = {n: getattr(m, a)[sel].repeat(2, *[1] * (getattr(m, a).ndim - 1)) for a, n in names.items()}
        new['xyz'] = torch.bmm(R.repeat(2, 1, 1), samples[..., None]).squeeze(-1) + m._xyz[sel].repeat(2, 1)
        new['scaling'] = torch.log(m.get_scaling[sel].repeat(2, 1) / 1.6)
        change(new, 'concat')
        change(~torch.cat((sel, sel.new_zeros(2 * sel.sum()))), 'prune')
        m.max_radii2D = radii[:1].expand(m._xyz.shape[0]).contiguous()
        mask = (m.get_opacity < 0.05).squeeze() | (m.max_radii2D > 20.0) | (m.get_scaling.amax(dim=1) > 0.4)
        change(~mask, 'prune')

    out = {}
    with torch.no_grad():
        for name, fn in (("density_control_ms", ours), ("density_control_torch_indexing_ms", reference_way)):
            times = []
            for _ in range(reps + 1):
                m, opt = fresh()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                fn(m, opt)
                torch.cuda.synchronize()
                times.append((time.perf_counter() - t0) * 1e3)
            out[name] = min(times[1:])
            out[name.replace("_ms", "_points_after")] = int(m._xyz.shape[0])
        # the gather alone: all 6 parameters + 12 moments of a prune that keeps 90 %
        m, opt = fresh()
        tensors = [grp['params'][0] for grp in opt.param_groups]
        tensors += [opt.state[t][k] for t in tensors for k in ('exp_avg', 'exp_avg_sq')]
        rows = f('select_indices')(torch.rand(P, device=dev) < 0.9)
        for _ in range(3):
            f('gather_rows')(tensors, rows)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            f('gather_rows')(tensors, rows)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 10
        nbytes = 2 * rows.numel() * sum(t[0].numel() * 4 for t in tensors) + 4 * rows.numel()
    out["gather_rows_ms"] = ms
    out["gather_rows_GBps"] = nbytes / (ms * 1e-3) / 1e9
    out["density_control_workload"] = (f"{P} surfels with Adam moments (177 floats per point): densify (clone + split, "
                                       "N = 2) then prune; gather_rows = 18 tensors, 90 % of the rows kept, allocation "
                                       "of the outputs included")
    return out


def large_scene_ms(dev, views: int = 4, reps: int = 3, cull: bool = False):
    """The large-scene configuration: 3M surfels, a batch of 4 views at 1352x1014 rendered forward + backward one after the other,
    and the K-NN of the 3M centres against 2048 control points with k = 8."""
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function
    from fast_sp_gs_amd.renderer import render_step
    scene_h, cams = scenes.config4()
    scene = scene_h.to(dev)
    bg = torch.ones(3, device=dev)
    g = torch.Generator().manual_seed(9)
    cams = [c.to(dev) for c in cams[:views]]
    gi = torch.randn(3, cams[0].H, cams[0].W, generator=g).to(dev)
    ge = torch.cat([torch.randn(6, cams[0].H, cams[0].W, generator=g), torch.zeros(3, cams[0].H, cams[0].W)]).to(dev)

    def batch():
        for cam in cams:
            out = render_step(scene, cam, gi, ge, None, background=bg, cull=cull)
        return out

    out = batch()
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()
    t0 = time.perf_counter()
    for _ in range(reps):
        batch()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    gc.enable()
    knn = get_C_function('knn_topk')
    ctrl = (torch.randn(2048, 3, generator=g) * 2).to(dev)
    knn(scene.means3D, ctrl, 8)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        knn(scene.means3D, ctrl, 8)
    torch.cuda.synchronize()
    knn_ms = (time.perf_counter() - t0) / 3 * 1e3
    return {"large_scene_batch_ms": dt * 1e3, "large_scene_views_per_s": views / dt,
            "large_scene_knn_ms": knn_ms, "large_scene_knn_queries_per_s": scene.P / (knn_ms * 1e-3),
            "large_scene_workload": f"{scene.P} surfels, {views} views {cams[0].W}x{cams[0].H} forward + backward in "
                                    f"sequence (R = {out['point_list'].numel()} instances in the last view); K-NN "
                                    f"{scene.P} x 2048, k = 8"}


def ssim_rate(dev, reps: int = 20):
    """Fused SSIM forward (with the partial-derivative maps) + backward on one 3 x 800 x 800 image pair."""
    from fast_sp_gs_amd._C import get_C_function
    fwd, bwd = get_C_function('fusedssim'), get_C_function('fusedssim_backward')
    g = torch.Generator().manual_seed(3)
    a, b, gm = (torch.rand(1, 3, 800, 800, generator=g).to(dev) for _ in range(3))
    for _ in range(3):
        m, d1, d2, d3 = fwd(1e-4, 9e-4, a, b, True)
        bwd(1e-4, 9e-4, a, b, gm, d1, d2, d3)
    torch.cuda.synchronize()
    e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    e[0].record()
    for _ in range(reps):
        m, d1, d2, d3 = fwd(1e-4, 9e-4, a, b, True)
    e[1].record()
    for _ in range(reps):
        bwd(1e-4, 9e-4, a, b, gm, d1, d2, d3)
    e[2].record()
    torch.cuda.synchronize()
    n = a.numel() * 4
    f_ms, b_ms = e[0].elapsed_time(e[1]) / reps, e[1].elapsed_time(e[2]) / reps
    return {"fusedssim_forward_ms": f_ms, "fusedssim_backward_ms": b_ms,
            "fusedssim_forward_GBps": 6 * n / (f_ms * 1e-3) / 1e9,   # 2 images in, map + 3 partial maps out
            "fusedssim_backward_GBps": 7 * n / (b_ms * 1e-3) / 1e9,  # 2 images + dL/dmap + 3 maps in, gradient out
            "fusedssim_workload": "1 x 3 x 800 x 800, train = true (times include output allocation)"}


def topk_weights_ms(dev, scene, cam, reps: int = 20):
    """Per-pixel top-k blend weights (k = 4) of the benchmark view: `gs_2d_topk_weights` on the binned scene."""
    from fast_sp_gs_amd._C import get_C_function as f
    W, H = cam.W, cam.H
    m2, colors, tm, no, depths, radii, tt = f('gs_2d_preprocess_forward')(
        W, H, 3, False, scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs, None, cam.Tw2v,
        cam.Tv2c, cam.campos, None, None, None)
    ranges, point_list = f('GS_prepare')(W, H, m2, depths, radii, tt, False)
    run = lambda: f('gs_2d_topk_weights')(4, W, H, cam.near, cam.far, m2, no, tm, ranges, point_list)
    run()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    return {"gs_2d_topk_weights_ms": ms, "gs_2d_topk_weights_pixels_per_s": W * H / (ms * 1e-3),
            "gs_2d_topk_weights_workload": f"k = 4 on the 300k-surfel 800x800 view, R = {int(point_list.numel())}"}


def training_forward_ms(dev, scene, cam, reps: int = 30):
    """The blend forward as the reference's training loop calls it (network.py:706-709): `accum_max_count` always, plus
    `accum_weights_p` / `accum_weights_count` for its 'simp' render type, next to the plain forward of the headline."""
    from fast_sp_gs_amd._C import get_C_function as f
    W, H, P = cam.W, cam.H, scene.P
    m2, colors, tm, no, depths, radii, tt = f('gs_2d_preprocess_forward')(
        W, H, 3, False, scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs, None, cam.Tw2v,
        cam.Tv2c, cam.campos, None, None, None)
    ranges, point_list = f('GS_prepare')(W, H, m2, depths, radii, tt, False)
    amc = torch.zeros(P, dtype=torch.int32, device=dev)
    awp, awc = torch.zeros(P, device=dev), torch.zeros(P, dtype=torch.int32, device=dev)
    fwd = f('GS_2D_render_forward')
    out = {}
    for name, side in (("plain", (None, None, None)), ("max_count", (amc, None, None)), ("all_three", (amc, awp, awc))):
        run = lambda: fwd(W, H, m2, colors, no, tm, point_list, ranges, cam.near, cam.far, False, None, *side)
        for _ in range(3):
            run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        out[f"blend_forward_{name}_ms"] = e0.elapsed_time(e1) / reps
    out["blend_forward_accum_workload"] = ("GS_2D_render_forward on the benchmark view: no side outputs / accum_max_count "
                                           "(every training step of the reference) / all three accum_* ('simp' render type)")
    return out


def fast_path_rate(dev, scene, cam, gi, steps: int = 20, warmup: int = 3):
    """The "fast" variant (adjugate intersection, fused corner-test binning) on the benchmark scene, forward + backward,
    with the blend backward's per-surfel sums through ordered per-instance records (default) and through atomics."""
    from fast_sp_gs_amd._C import _ops
    from fast_sp_gs_amd.renderer import fast_render_step
    ge = torch.zeros(8, cam.H, cam.W, device=dev)
    go = -gi.sum(0)
    rates = []
    for ordered in (True, False):
        for _ in range(warmup):
            fast_render_step(scene, cam, gi, ge, go, ordered_sums=ordered)
        torch.cuda.synchronize()
        gc.collect()
        gc.disable()
        t0 = time.perf_counter()
        for _ in range(steps):
            fast_render_step(scene, cam, gi, ge, go, ordered_sums=ordered)
        torch.cuda.synchronize()
        rates.append(steps / (time.perf_counter() - t0))
        gc.enable()
    # the two backward decompositions on that view with the per-splat channel set: one block per tile walking its list
    # back to front (the default behind both operator forms) against the reference's second algorithm, one lane per list
    # entry with the pixels passed from lane to lane from the forward's bucket snapshots (gs_2d_fast_redner.cu:563-837)
    bwd_ms = {}
    for name, per_splat_kernel in (("tile", False), ("per_splat", True)):
        call = lambda: fast_render_step(scene, cam, gi, ge, go, per_splat=True, per_splat_kernel=per_splat_kernel)
        call()
        _ops.STAGE_EVENTS, _ops.STAGE_FILTER = events, _ = [], {'gs_2d_fast_render_backward'}
        try:
            for _ in range(10):
                call()
            torch.cuda.synchronize()
        finally:
            _ops.STAGE_EVENTS, _ops.STAGE_FILTER = None, None
        bwd_ms[name] = float(np.mean([a.elapsed_time(b) for _, a, b in events]))
    return rates, bwd_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the fast-path and dynamic-step side measurements")
    ap.add_argument("--counter-run", action="store_true",
                    help="the process runs under a counter collection: every dispatch then carries the profiler's "
                         "serialisation, so the operator with the most launches looks largest; do not stop on that")
    ap.add_argument("--only", choices=["knn_large"], default=None,
                    help="run one side workload alone (for counter collections that must see a single kernel): "
                         "knn_large = K-NN of 3M points against 2048 control points, k = 8, three launches")
    ap.add_argument("--culled-lists", action="store_true",
                    help="time the step on tile lists without the (surfel, tile) instances that no pixel of their tile "
                         "can blend (same images and gradients, shorter lists) instead of the reference's full lists; "
                         "the default run reports that rate as extra_metrics.culled_lists_frames_per_s")
    ap.add_argument("--surfels", type=int, default=300_000)
    ap.add_argument("--size", type=int, default=800)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import _ops, get_C_function
    from fast_sp_gs_amd.renderer import render_step

    dev = torch.device("cuda:0")
    if args.only == "knn_large":
        g = torch.Generator().manual_seed(9)
        pts = (torch.randn(3_000_000, 3, generator=g) * 2).to(dev)
        ctrl = (torch.randn(2048, 3, generator=g) * 2).to(dev)
        knn = get_C_function('knn_topk')
        knn(pts, ctrl, 8)
        torch.cuda.synchronize()
        ms = _timed_ms(lambda: knn(pts, ctrl, 8), reps=2, warm=0)
        print(json.dumps({"knn_large_ms": ms, "queries_per_s": pts.shape[0] / (ms * 1e-3),
                          "workload": "3000000 x 2048, k = 8, D = 3"}))
        return
    scene_h, cam_h = scenes.config2(P=args.surfels, size=args.size)
    scene, cam = scene_h.to(dev), cam_h.to(dev)
    gi = scene_h.extra['grad_image'].to(dev)
    ge = scene_h.extra['grad_extras'].to(dev)
    bg = torch.ones(3, device=dev)  # white background

    def step():
        # the fused per-pixel epilogue runs between the two blend passes, as in training: composite on the background,
        # normals to world space, surf_depth, pseudo surface normal; its backward supplies dL/dextras and the
        # composite's dL/dopacity = -sum_c dL/dimage_c * bg_c to the blend backward
        return render_step(scene, cam, gi, ge, None, background=bg, cull=args.culled_lists)

    # The per-stage events of the timed steps are created and recorded once here, outside the timed region: the runtime
    # grows its event pool in bursts that stall the host for tens of milliseconds.
    _ops.EVENT_POOL[:] = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps * 2 * 12)]
    for e in _ops.EVENT_POOL:
        e.record()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    # Python's cyclic collector is kept out of the timed region (a full collection with torch loaded stalls the host
    # for ~35 ms, 28 steps' worth; nothing in a step creates reference cycles): collect now, switch it back on after.
    gc.collect()
    gc.disable()
    # Inside the timed region only the dominant operator is bracketed by events (on the stream it is launched on): an
    # event is a packet of its own in the device queue, and bracketing all nine operators of a step costs 8 % of the
    # frame rate (18 events x ~4.5 us). The per-stage table comes from a second, fully instrumented pass below.
    _ops.STAGE_EVENTS = events = []
    _ops.STAGE_FILTER = {DOMINANT}
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    dominant_ms = float(np.sum([a.elapsed_time(b) for _, a, b in events])) / args.steps
    _ops.STAGE_FILTER = None
    _ops.STAGE_EVENTS = events = []
    stage_steps = min(args.steps, 20)
    for _ in range(stage_steps):
        out = step()
    torch.cuda.synchronize()
    _ops.STAGE_EVENTS = None
    gc.enable()

    P = scene.P
    Pv = int((out['radii'] > 0).sum())
    R = int(out['point_list'].numel())  # the reference's instance count: every tile of every surfel's rectangle
    R_lists = int((out['ranges'][:, 1] - out['ranges'][:, 0]).sum())  # R, or what the culled binning left in the lists
    HW = cam.W * cam.H
    T = ((cam.W + 15) // 16) * ((cam.H + 15) // 16)
    stage_ms = {}
    for name, a, b in events:
        stage_ms.setdefault(name, []).append(a.elapsed_time(b))
    # per step: an operator that runs in two parts (the binning around the host's wait for the instance count) is timed
    # twice per step and its parts are added
    stage_avg = {k: float(np.sum(v)) / stage_steps for k, v in stage_ms.items()}
    dominant = max(stage_avg, key=stage_avg.get)
    if dominant != DOMINANT and not args.counter_run:
        raise RuntimeError(f"the dominant stage is {dominant}, not {DOMINANT}: bracket that one in the timed region")
    stage_avg[dominant] = dominant_ms  # the figure from the timed region itself
    bytes_dom = algorithmic_bytes(dominant, P, Pv, R, T, HW)
    achieved = bytes_dom / (dominant_ms * 1e-3) / 1e9
    # next to the algorithmic rate (the per-unit byte figure of the reference's scheme over this build's time) the rate
    # of the bytes this build's kernels actually moved, where the committed counter summary holds them
    stages = {}
    for k, v in stage_avg.items():
        stages[k] = {"ms": round(v, 4),
                     "algorithmic_GBps": round(algorithmic_bytes(k, P, Pv, R, T, HW) / (v * 1e-3) / 1e9, 1)}
        moved = measured_traffic(k)
        if moved is not None:
            stages[k]["counter_traffic_bytes"] = moved
            stages[k]["counter_GBps"] = round(moved / (v * 1e-3) / 1e9, 1)

    # top-k queries/s: 200k Gaussian centres against 512 control points, k = 4 (indices bit-exact, squared distances)
    c1 = scenes.config1(n_dirs=8)
    pts, ctrl = c1['points'].to(dev), c1['ctrl'].to(dev)
    knn = get_C_function('knn_topk')
    for _ in range(3):
        knn(pts, ctrl, 4)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        knn(pts, ctrl, 4)
    e1.record()
    torch.cuda.synchronize()
    knn_ms = e0.elapsed_time(e1) / 20

    copy_gbps = copy_probe_gbps(dev)
    extra = {"knn_topk_queries_per_s": pts.shape[0] / (knn_ms * 1e-3), "knn_topk_workload": "200000 x 512, k=4, D=3"}
    extra["standalone_ops"] = standalone_ops(dev, copy_gbps)
    if not args.no_extras and not args.counter_run and not args.culled_lists:
        # the same step on culled tile lists: identical images and gradients from shorter lists (what _GS_2D_Render uses)
        for _ in range(max(args.warmup, 2)):
            culled = render_step(scene, cam, gi, ge, None, background=bg, cull=True)
        torch.cuda.synchronize()
        gc.collect()
        gc.disable()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            culled = render_step(scene, cam, gi, ge, None, background=bg, cull=True)
        torch.cuda.synchronize()
        extra["culled_lists_frames_per_s"] = args.steps / (time.perf_counter() - t0)
        gc.enable()
        extra["culled_lists_instances"] = int((culled['ranges'][:, 1] - culled['ranges'][:, 0]).sum())
        extra["culled_lists_workload"] = ("the benchmark step with GS_prepare(cull=True): instances that no pixel of "
                                          "their tile can blend are left out of the tile lists; images bit-identical, "
                                          "gradients equal to rounding")
        del culled
    if not args.no_extras:
        extra.update(ssim_rate(dev))
        extra.update(simple_knn_ms(dev, scene))
        extra.update(reference_note_blend_ms(dev))
        extra.update(topk_weights_ms(dev, scene, cam))
        extra.update(training_forward_ms(dev, scene, cam))
        extra.update(gs3d_path_rate(dev, scene, cam, gi))
        extra.update(density_control_ms(dev, scene))
        extra.update(large_scene_ms(dev))
        extra["large_scene_culled_lists_views_per_s"] = large_scene_ms(dev, cull=True)["large_scene_views_per_s"]
        (extra["fast_path_frames_per_s"], extra["fast_path_atomic_sums_frames_per_s"]), fast_bwd = fast_path_rate(dev, scene, cam, gi)
        extra["fast_path_workload"] = "same scene through GS_2D_fast_* (corner-test binning keeps fewer instances)"
        extra["fast_backward_tile_kernel_ms"] = fast_bwd["tile"]
        extra["fast_backward_per_splat_kernel_ms"] = fast_bwd["per_splat"]
        extra["fast_backward_workload"] = ("GS_2D_fast_render_backward on that view, per-splat channel set, ordered sums "
                                           "(record clear + kernel + record sum): back-to-front tile kernel / the "
                                           "reference's per-splat decomposition (wavefront = 64 entries)")
        extra["dynamic_step_frames_per_s"] = dynamic_step_rate(dev)
        extra["dynamic_step_workload"] = ("200000 surfels, 512 control points, bf16 MFMA MLP + K-NN(4) + LBS -> render "
                                          "800x800 -> 0.8 L1 + 0.2 D-SSIM (fused kernel) -> backward through LBS / K-NN / MLP "
                                          "(HIP kernels) -> masked Adam on the surfels + Adam on the MLP and control "
                                          "points")

    result = {
        "metric": "fwd+bwd frames/s, 300k surfels @800x800",
        "value": args.steps / dt,
        "unit": "frames/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"static 2DGS fwd+bwd: {P} surfels in the unit ball, {cam.W}x{cam.H}, FoV 40, radius 4, "
                               "SH degree 3, white background, 16x16 tiles, per-tile binning of (tile, depth) keys "
                               + ("(instances that no pixel of their tile can blend are left out of the lists: same "
                                  "images and gradients)" if args.culled_lists else
                                  "(every tile of every surfel's rectangle: the reference's lists, bit for bit)")
                               + ", depth/normal outputs, fused per-pixel epilogue (composite, world normals, "
                               "surf depth / normal) and its backward between the two blend passes",
                   "P": P, "P_visible": Pv, "R": R, "R_in_tile_lists": R_lists, "tiles": T},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": measured_traffic(dominant),
                     "algorithmic_bytes_per_launch": bytes_dom, "valu_issue_frac": measured_valu_issue(dominant), "avg_launch_ms": stage_avg[dominant],
                     "copy_kernel_GBps": round(copy_gbps, 1)},
        "stages": stages,
        "extra_metrics": extra,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(scene_h, cam_h)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
