"""Observation pipeline of the oracle: exact rational area pool, grayscale, frame stack."""

from __future__ import annotations

from fractions import Fraction

import numpy as np


def _axis_overlaps(source: int, output: int, coordinate: int):
    """Source pixels overlapped by output pixel `coordinate`, with overlap lengths on the common grid."""

    start, end = coordinate * source, (coordinate + 1) * source
    taps = []
    for s in range(source):
        overlap = min(end, (s + 1) * output) - max(start, s * output)
        if overlap > 0:
            taps.append((s, overlap))
    return taps


def _exact_gray(indexed_240, playpal, oy, ox):
    rows = _axis_overlaps(240, 84, oy)
    cols = _axis_overlaps(320, 84, ox)
    pooled = []
    for c in range(3):
        total = Fraction(0)
        for sy, wy in rows:
            for sx, wx in cols:
                total += Fraction(wy * wx * int(playpal[indexed_240[sy, sx], c]), 240 * 320)
        pooled.append(int(total + Fraction(1, 2)))  # floor(x + 0.5), x >= 0
    return (pooled[0] * 77 + pooled[1] * 150 + pooled[2] * 29 + 128) >> 8


def test_area_footprints_match_reference_invariants():
    # tests/test_rendering.py:55-70: rows sum to one, <=4 vertical and <=5 horizontal taps
    for oy in range(84):
        taps = _axis_overlaps(240, 84, oy)
        assert sum(w for _s, w in taps) == 240 and len(taps) <= 4
    for ox in range(84):
        taps = _axis_overlaps(320, 84, ox)
        assert sum(w for _s, w in taps) == 320 and len(taps) <= 5


def test_observe_equals_exact_rational_pool_on_random_images(oracle):
    rng = np.random.default_rng(20260813)
    indexed = rng.integers(0, 256, (2, 240, 320), dtype=np.uint8)
    playpal = rng.integers(0, 256, (256, 3), dtype=np.uint8)
    obs, _ = oracle.observe(indexed, playpal)
    pixels = [(0, 0), (83, 83), (0, 83), (83, 0)] + [tuple(rng.integers(0, 84, 2)) for _ in range(300)]
    for lane in range(2):
        for oy, ox in pixels:
            assert obs[lane, oy, ox] == _exact_gray(indexed[lane], playpal, int(oy), int(ox))


def test_view_only_source_treats_status_bar_as_black(oracle):
    rng = np.random.default_rng(5)
    view = rng.integers(0, 256, (1, 208, 320), dtype=np.uint8)
    playpal = rng.integers(1, 256, (256, 3), dtype=np.uint8)  # palette entry 0 is NOT black
    obs_view, _ = oracle.observe(view, playpal)
    black_palette = playpal.copy()
    full = np.concatenate((view, np.zeros((1, 32, 320), dtype=np.uint8)), axis=1)
    black_palette[0] = 0
    # a 240-row frame whose bottom rows use a truly black entry gives the same observation
    remap = view.copy()
    assert not (view == 0).all()
    obs_full, _ = oracle.observe(np.where(full == 0, 0, full), black_palette)
    mask = np.ones((84, 84), dtype=bool)
    # rows that only see view pixels with index != 0 are comparable directly
    uses_zero = np.zeros((84, 84), dtype=bool)
    for oy in range(84):
        for sy, _w in _axis_overlaps(240, 84, oy):
            if sy < 208 and (view[0, sy] == 0).any():
                uses_zero[oy, :] = True
    mask &= ~uses_zero
    assert np.array_equal(obs_view[0][mask], obs_full[0][mask])
    assert (obs_view[0, 73:] == 0).all()  # output rows fully inside the masked status bar
    del remap


def test_constant_frame_closed_form(oracle):
    # every view pixel = one colour -> observation = its gray above the bar, 0 below, blend at the seam
    playpal = np.zeros((256, 3), dtype=np.uint8)
    playpal[192] = (192, 192, 192)
    view = np.full((1, 208, 320), 192, dtype=np.uint8)
    obs, _ = oracle.observe(view, playpal)
    gray = (192 * 77 + 192 * 150 + 192 * 29 + 128) >> 8
    assert (obs[0, :72] == gray).all()
    # output row 72 covers source rows 205.71..208.57: 208-205.714 = 2.2857 of 2.857 rows are lit
    seam = int(Fraction(192 * (208 * 84 - 72 * 240), 240) + Fraction(1, 2))
    assert (obs[0, 72] == ((seam * 256 + 128) >> 8)).all()
    assert (obs[0, 73:] == 0).all()


def test_stack_roll_and_reset_fill(oracle):
    rng = np.random.default_rng(9)
    playpal = rng.integers(0, 256, (256, 3), dtype=np.uint8)
    frames = rng.integers(0, 256, (3, 4, 84, 84), dtype=np.uint8)
    indexed = rng.integers(0, 256, (3, 208, 320), dtype=np.uint8)
    mask = np.asarray([0, 1, 0], dtype=np.uint8)
    obs, stacked = oracle.observe(indexed, playpal, frames=frames, reset_mask=mask)
    # engine.py:9545-9548: roll by -1 on dim 1, newest last
    for lane in (0, 2):
        assert np.array_equal(stacked[lane, :3], frames[lane, 1:])
        assert np.array_equal(stacked[lane, 3], obs[lane])
    # engine.py:2443-2450: reset lanes hold four copies
    for k in range(4):
        assert np.array_equal(stacked[1, k], obs[1])
