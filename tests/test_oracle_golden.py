"""The CPU oracle against golden vectors written by the reference's own Torch path."""

from __future__ import annotations

import numpy as np
import pytest

from conftest import fixture_names, fixture_overlays, lane_inputs, load_fixture

# Cases whose oracle run takes more than a few seconds on the CPU are trimmed to a lane subset.
LANE_LIMIT = {"config3_subset": 1, "config4_subset": 1}


@pytest.mark.parametrize("name", fixture_names())
def test_indexed_frame_bit_exact_and_observation_within_one(oracle, name):
    meta, data, _smap, tables = load_fixture(name)
    lanes = min(meta["lanes"], LANE_LIMIT.get(name, meta["lanes"]))
    overlays = fixture_overlays(meta)
    oracle.set_overlays(overlays)
    try:
        result = oracle.render(tables, lane_inputs(data), data["cosine_correction"], lane_range=(0, lanes))
    finally:
        oracle.set_overlays(None)
    assert np.array_equal(result["indexed"][:lanes], data["indexed"][:lanes])
    # rows 208..239: empty status bar without status bar patches (engine.py:15232-15267 with a zero HUD
    # atlas), the drawn bar with them
    assert bool(result["indexed"][:lanes, 208:].any()) == (overlays is not None)
    # The reference CPU path pools in float32 matmuls; the oracle uses the exact integer
    # form of the reference's GPU branch. Tolerance from tests/test_rendering.py:138-139.
    delta = np.abs(result["obs"][:lanes].astype(np.int32) - data["obs"][:lanes].astype(np.int32))
    assert delta.max() <= 1
    assert delta.mean() < 0.01


STAGE_CASES = ("tiny_stages", "small_midtex_sprites", "pinched_pillars", "split_linedefs")


@pytest.mark.parametrize("name", STAGE_CASES)
def test_every_stage_matches_reference_intermediates(oracle, name):
    _meta, data, _smap, tables = load_fixture(name)
    if "st_geometry" not in data:
        pytest.skip("fixture carries no stage taps")
    result = oracle.render(tables, lane_inputs(data), data["cosine_correction"], lane_range=(0, 1), debug_lane=0)
    taps = result["debug"]
    assert result["sector"][0] == data["st_sector"][0]

    def same(ours, ref):
        ours = np.asarray(ours)
        ref = np.asarray(ref)
        if ours.dtype.kind == "f":
            return bool(np.all((ours == ref) | (np.isnan(ours) & np.isnan(ref))))
        return bool(np.array_equal(ours, ref))

    assert same(taps["geometry"], data["st_geometry"])
    assert same(taps["distances"], data["st_distances"])
    assert same(taps["along"], data["st_along"])
    assert same(taps["geometric"].astype(bool), data["st_geometric"])
    assert same(taps["projected"].astype(bool), data["st_projected"])
    assert same(taps["left_edge"].astype(bool), data["st_left_edge"])
    assert same(taps["visibility"], data["st_visibility"])
    assert same(taps["horizontal_offset"], data["st_hoff"])
    assert same(taps["vertical_step"], data["st_vstep"])
    assert same(taps["flats_frame"], data["st_flats"])
    assert same(taps["surface_depth"], data["st_surface_depth"])
    assert same(taps["scene_surface_depth"], data["st_scene_surface_depth"])
    assert same(taps["walls_frame"], data["st_walls"])
    assert same(taps["scene_depth"], data["st_scene_depth"])
    assert same(taps["sprite_clip_depth"], data["st_clip_depth"])
    assert same(taps["sprite_clip_wall"], data["st_clip_wall"])


def test_sprites_are_actually_drawn_in_the_sprite_fixtures(oracle):
    _meta, data, _smap, tables = load_fixture("small_midtex_sprites")
    result = oracle.render(tables, lane_inputs(data), data["cosine_correction"], lane_range=(0, 1), debug_lane=0)
    changed = int((result["debug"]["walls_frame"] != result["indexed"][0, :208]).sum())
    assert changed > 200, "sprite layer changed too few pixels for the parity check to mean anything"


def test_rgb_expansion_matches_reference(oracle):
    _meta, data, _smap, tables = load_fixture("tiny_stages")
    result = oracle.render(tables, lane_inputs(data), data["cosine_correction"], lane_range=(0, 1), want_rgb=True)
    assert np.array_equal(result["rgb"][0], data["rgb_lane0"])


def test_screen_flashes_blend_the_palette_per_lane(oracle):
    """render_screen_flashes (engine.py:15381-15398): RGB24 bit-exact, lane 0 (both counters zero) unblended."""

    _meta, data, _smap, tables = load_fixture("screen_flashes")
    result = oracle.render(tables, lane_inputs(data), data["cosine_correction"], want_rgb=True)
    assert np.array_equal(result["rgb"], data["rgb_all"])
    playpal = tables["playpal"].reshape(256, 3)
    assert np.array_equal(result["rgb"][0], playpal[result["indexed"][0]])
    assert not np.array_equal(result["rgb"][2], playpal[result["indexed"][2]])


def test_scene_depth_under_the_decals_matches_the_reference(oracle):
    """Decals are drawn where |scene depth - decal distance| <= 1e-3 (engine.py:13930-13933), so the depth
    buffer itself has to be the reference's, bit for bit, on every kind of pixel."""

    _meta, data, _smap, tables = load_fixture("decals")
    for lane in (0, 3, 7):
        taps = oracle.render(tables, lane_inputs(data), data["cosine_correction"], lane_range=(lane, lane + 1), debug_lane=lane)["debug"]
        ours, ref = np.asarray(taps["scene_depth"]), data["ref_scene_depth"][lane]
        assert np.array_equal(ours, ref)
        assert np.isfinite(ref).mean() > 0.9


def test_observation_with_the_status_bar_pooled_matches_the_reference(oracle):
    """An environment made with obs_crop=None pools all 240 rows (env.py:441, engine.py:15440)."""

    meta, data, _smap, tables = load_fixture("overlays")
    oracle.set_overlays(fixture_overlays(meta))
    try:
        result = oracle.render(tables, lane_inputs(data), data["cosine_correction"], obs_source_rows=240)
        masked = oracle.render(tables, lane_inputs(data), data["cosine_correction"])
    finally:
        oracle.set_overlays(None)
    delta = np.abs(result["obs"].astype(np.int32) - data["obs_with_hud"].astype(np.int32))
    assert delta.max() <= 1 and delta.mean() < 0.01   # tolerance: tests/test_rendering.py:138-139
    assert (data["obs_with_hud"][:, 74:] != data["obs"][:, 74:]).mean() > 0.5   # the bar really shows in the last rows
    assert np.array_equal(result["obs"][:, :72], masked["obs"][:, :72])   # rows that pool view rows only are unchanged
