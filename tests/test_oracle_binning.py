"""Pins the oracle's tile binning (oracle/gs2d.cpp: prepare_count / prepare_fill / higher_msb / get_rect) by brute
force: for every tile, the surfels whose rectangle covers it, ordered by (depth bits, surfel index); plus the
structural invariants of ranges and the sort-bit count the reference derives for known tile counts."""
import numpy as np
import pytest


def _inputs(P, W, H, seed):
    rng = np.random.default_rng(seed)
    means2D = np.ascontiguousarray(rng.uniform(-40, [W + 40, H + 40], size=(P, 2)).astype(np.float32))
    radii = rng.integers(0, 60, size=P).astype(np.int32)
    radii[rng.random(P) < 0.2] = 0
    depths = rng.uniform(0.2, 10, size=P).astype(np.float32)
    depths[::7] = depths[min(3, P - 1)]  # equal depths: order must fall back to the surfel index
    gx, gy = (W + 15) // 16, (H + 15) // 16
    tt = np.zeros(P, np.int32)
    rects = []
    for i in range(P):
        r = np.float32(radii[i])
        px, py = means2D[i]
        x0 = min(gx, max(0, int(np.float32(px - r) / np.float32(16))))
        y0 = min(gy, max(0, int(np.float32(py - r) / np.float32(16))))
        x1 = min(gx, max(0, int(np.float32(np.float32(np.float32(px + r) + np.float32(16)) - np.float32(1)) / np.float32(16))))
        y1 = min(gy, max(0, int(np.float32(np.float32(np.float32(py + r) + np.float32(16)) - np.float32(1)) / np.float32(16))))
        rects.append((x0, y0, x1, y1))
        tt[i] = (x1 - x0) * (y1 - y0) if radii[i] > 0 else 0
    radii[tt == 0] = 0
    return means2D, depths, radii, tt, rects, gx, gy


@pytest.mark.parametrize("P,W,H,seed", [(500, 200, 120, 0), (64, 511, 127, 1), (1, 16, 16, 2), (2000, 64, 64, 3)])
def test_lists_match_brute_force(oracle_mod, P, W, H, seed):
    means2D, depths, radii, tt, rects, gx, gy = _inputs(P, W, H, seed)
    ranges, pl, keys = oracle_mod.prepare(W, H, means2D, depths, radii, tt, return_keys=True)
    assert pl.size == tt.sum()
    bits = depths.view(np.uint32)
    cursor = 0
    for t in range(gx * gy):
        ty, tx = divmod(t, gx)
        members = [i for i in range(P) if radii[i] > 0 and rects[i][0] <= tx < rects[i][2] and rects[i][1] <= ty < rects[i][3]]
        members.sort(key=lambda i: (int(bits[i]), i))
        if not members:
            assert tuple(ranges[t]) == (0, 0)
            continue
        assert tuple(ranges[t]) == (cursor, cursor + len(members))  # contiguous, ascending tile order
        assert list(pl[cursor:cursor + len(members)]) == members
        assert all(int(k) >> 32 == t for k in keys[cursor:cursor + len(members)])
        assert all((int(k) & 0xffffffff) == int(bits[i]) for k, i in zip(keys[cursor:cursor + len(members)], members))
        cursor += len(members)
    assert cursor == pl.size


def test_empty(oracle_mod):
    z = np.zeros
    ranges, pl = oracle_mod.prepare(64, 64, z((5, 2), np.float32), z(5, np.float32), z(5, np.int32), z(5, np.int32))
    assert pl.size == 0 and not ranges.any()
    ranges, pl = oracle_mod.prepare(64, 64, z((0, 2), np.float32), z(0, np.float32), z(0, np.int32), z(0, np.int32))
    assert pl.size == 0 and ranges.shape == (16, 2)


def test_sort_bit_count(oracle_mod):
    f = oracle_mod.lib().oracle_higher_msb
    # tile counts of the benchmark images: 256x256 -> 256 tiles, 800x800 -> 2500, 1352x1014 -> 5440
    assert [f(256), f(2500), f(5440)] == [9, 12, 13]
    for n in (1, 2, 3, 4, 7, 8, 255, 257, 65535, 65536):
        assert f(n) == n.bit_length()
