"""Bit-exact parity of the tile binning (ranges, point list, sorted keys) with the oracle's stable sort, on the GPU's own
preprocess outputs, for every segment-length class of the per-tile sort: short segments (<= 2048 entries, LDS, one
block per tile), long ones (<= 16384, LDS, queued) and very long ones (sorted in global memory), a tile grid too large for the
LDS counters, plus equal depths
(ties must come out in surfel order) and empty tiles."""
import numpy as np
import pytest
import torch

from util import npy

pytestmark = pytest.mark.gpu

CASES = {
    # name: (P, W, H, scale multiplier, duplicate depths)
    "short_segments": (20_000, 320, 200, 1.0, False),
    "long_segments_lds": (9_000, 32, 32, 1.0, False),       # 4 tiles, ~9000 entries each
    "very_long_segments": (40_000, 32, 16, 1.0, False),     # 2 tiles, > 16384 entries each
    "equal_depths": (6_000, 64, 48, 2.0, True),
    "many_tiles": (5_000, 2100, 2100, 20.0, False),         # > 16384 tiles: counters in global memory
}


@pytest.mark.parametrize("name", list(CASES))
def test_binning_bit_exact(name, device, oracle_mod):
    from fast_sp_gs_amd import scenes
    from fast_sp_gs_amd._C import get_C_function
    O = oracle_mod
    P, W, H, mul, dup = CASES[name]
    scene, _ = scenes.config0(P=P, size=max(W, H), seed=21)
    scene.scales = scene.scales * mul
    if W <= 32:  # squeeze everything into the few tiles of a tiny image
        scene.means3D = scene.means3D * 0.05
    if dup:      # a plane parallel to the image plane: thousands of identical depths
        scene.means3D[:, 2] = 0.25
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    d = lambda t: t.to(device).contiguous()
    print(f"[binning {name}] P={P} {W}x{H}", flush=True)
    m2, colors, tm, no, dep, radii, tt = get_C_function('gs_2d_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), None, None, None)
    ranges, pl, keys, offsets = get_C_function('GS_prepare')(W, H, m2, dep, radii, tt, False, return_keys=True,
                                                           return_offsets=True)
    torch.cuda.synchronize()
    r_ranges, r_pl, r_keys = O.prepare(W, H, npy(m2), npy(dep), npy(radii), npy(tt), return_keys=True)
    lens = r_ranges[:, 1] - r_ranges[:, 0]
    print(f"[binning {name}] R={r_pl.size} longest segment {int(lens.max())} empty tiles {int((lens == 0).sum())}",
          flush=True)
    if name == "long_segments_lds":
        assert 2048 < lens.max() <= 16384
    if name == "very_long_segments":
        assert lens.max() > 16384
    if dup:
        assert np.unique(npy(dep)[npy(radii) > 0]).size < (npy(radii) > 0).sum()
    assert np.array_equal(npy(ranges), r_ranges)
    assert np.array_equal(npy(pl), r_pl)
    assert np.array_equal(npy(keys), r_keys)
    assert np.array_equal(npy(offsets)[:P], np.cumsum(npy(tt).astype(np.int64)))


def test_blocking_entry_points_match_the_operator(device):
    """`GS_prepare` runs the binning cut where the host waits (scan_begin / count / scan_end / fill_counted); the blocking
    pair fsgs_gs_prepare_scan + fsgs_gs_prepare_fill, called straight through the C ABI, must give the same lists, and
    the `overlap` hook must see the finished scan."""
    import ctypes
    from fast_sp_gs_amd import lib as L, scenes
    from fast_sp_gs_amd._C import get_C_function
    P, W, H = 20_000, 320, 200
    scene, _ = scenes.config0(P=P, size=W, seed=5)
    cam = scenes.pinhole(W, H, 50.0, torch.tensor([0., 0., 4.]))
    d = lambda t: t.to(device).contiguous()
    print(f"[binning blocking entries] P={P} {W}x{H}", flush=True)
    m2, colors, tm, no, dep, radii, tt = get_C_function('gs_2d_preprocess_forward')(
        W, H, 3, False, d(scene.means3D), d(scene.scales), d(scene.rotations), d(scene.opacities), d(scene.shs), None,
        d(cam.Tw2v), d(cam.Tv2c), d(cam.campos), None, None, None)
    seen = {}
    ranges, pl, offsets, hooked = get_C_function('GS_prepare')(
        W, H, m2, dep, radii, tt, False, return_offsets=True, overlap=lambda off: seen.setdefault('sum', off[P - 1].clone()))
    torch.cuda.synchronize()
    assert int(hooked) == int(tt.sum()) == pl.numel()

    lib = L.load()
    T = ((W + 15) // 16) * ((H + 15) // 16)
    stream = L.current_stream()
    off2 = torch.empty(P, dtype=torch.int64, device=device)
    ws1 = torch.empty(lib.fsgs_gs_prepare_scan_workspace_bytes(P), dtype=torch.uint8, device=device)
    R = ctypes.c_int64(-1)
    L.check(lib.fsgs_gs_prepare_scan(P, L.ptr(tt), L.ptr(off2), L.ptr(ws1), ws1.numel(), ctypes.addressof(R), stream), 'scan')
    assert R.value == pl.numel() and torch.equal(off2, offsets[:P])
    ranges2 = torch.empty((T, 2), dtype=torch.int64, device=device)
    pl2 = torch.empty(R.value, dtype=torch.int32, device=device)
    ws2 = torch.empty(lib.fsgs_gs_prepare_fill_workspace_bytes(R.value), dtype=torch.uint8, device=device)
    bins = torch.empty(lib.fsgs_gs_prepare_bins_bytes(P, W, H), dtype=torch.uint8, device=device)
    bins.fill_(0xff)  # neither buffer needs clearing
    L.check(lib.fsgs_gs_prepare_fill(P, W, H, L.ptr(m2), L.ptr(dep), L.ptr(radii), L.ptr(off2), R.value, L.ptr(ranges2),
                                     L.ptr(pl2), None, L.ptr(bins), bins.numel(), L.ptr(ws2), ws2.numel(), stream), 'fill')
    torch.cuda.synchronize()
    assert torch.equal(ranges2, ranges) and torch.equal(pl2, pl)


@pytest.mark.parametrize("gx,gy,kind", [
    (1, 1, "one"), (7, 5, "random"), (16, 16, "random"), (16, 16, "equal"), (50, 50, "ball"), (50, 50, "empty"),
    (131, 97, "random"), (256, 256, "random"),
])
def test_blend_schedule_is_a_permutation_longest_first(device, gx, gy, kind):
    """The blockIdx -> tile table of the blend kernels (fsgs_debug_tile_order): every tile exactly once, for grids from one
    tile to the 65 536-tile limit, with empty and equal lists; inside each of the 8 interleaved position classes (one
    XCD each) the list lengths fall from round to round of 32 positions (inside a round the tiles are dealt by the load of
    the compute units, in any order), up to the resolution of the length buckets (sixteen per octave)."""
    from fast_sp_gs_amd import lib as L
    T = gx * gy
    rng = np.random.default_rng(gx * 1000 + gy)
    if kind == "random":
        lens = rng.integers(0, 5000, T) * (rng.random(T) < 0.7)
    elif kind == "equal":
        lens = np.full(T, 777)
    elif kind == "empty":
        lens = np.zeros(T, np.int64)
    elif kind == "one":
        lens = np.array([12])
    else:  # chord lengths of a ball centred on the grid, as in the benchmark scene
        ty, tx = np.mgrid[0:gy, 0:gx]
        r2 = ((tx - gx / 2 + 0.5) ** 2 + (ty - gy / 2 + 0.5) ** 2) / (0.36 * gx) ** 2
        lens = (2000 * np.sqrt(np.clip(1 - r2, 0, None))).astype(np.int64).reshape(-1)
    lens = lens.astype(np.int64)
    start = np.concatenate([[0], np.cumsum(lens)[:-1]])
    ranges = torch.from_numpy(np.stack([start, start + lens], 1)).to(device)
    table = torch.full((T,), -1, dtype=torch.int32, device=device)
    print(f"[schedule table] {gx}x{gy} {kind}", flush=True)
    lib = L.load()
    L.check(lib.fsgs_debug_tile_order(gx, gy, L.ptr(ranges), L.ptr(table), L.current_stream()), 'tile_order')
    torch.cuda.synchronize()
    t = npy(table)
    assert np.array_equal(np.sort(t), np.arange(T)), "not a permutation of the tiles"
    ll = lens[t]
    for r in range(8):
        cls = ll[r::8]                       # a region's tiles while it has any; exhausted regions are skipped, so the
        if cls.size < 64: continue           # classes only line up with the regions at the start: check full rounds there
        rounds = cls[:cls.size // 32 * 32].reshape(-1, 32)[:4]
        lo, hi = rounds.min(1), rounds.max(1)
        # a later round's longest tile is not above an earlier round's shortest by more than a bucket: sixteen equal
        # steps per octave, so at most 1/16 of the length
        assert (hi[1:] <= lo[:-1] * (1 + 1 / 16) + 1).all(), (r, lo, hi)
