"""Host-side overlay inputs (weapon psprite words, status bar words) against the reference's own selections."""

from __future__ import annotations

import numpy as np
import torch

from conftest import fixture_overlays, load_fixture

WEAPON_ARGUMENTS = (
    "active_weapon", "weapon_state_cooldown", "weapon_fire_count", "weapon_ready_tics", "weapon_lower_cooldown",
    "weapon_raise_cooldown", "pending_weapon", "episode_time", "player_bob_fixed", "player_dead",
)
HUD_ARGUMENTS = (
    "active_weapon", "weapon_ammo_slot", "hud_ready_ammo", "health", "armor", "weapons", "hud_ammo_counts",
    "mugshot_face_index", "mugshot_grin_tics", "mugshot_pain_tics", "mugshot_ouch", "mugshot_pain_direction",
    "attack_held_tics",
)


def _engine(data, names):
    return {name: torch.as_tensor(data[f"engine_{name}"]) for name in names}


def test_fine_sine_table_known_values():
    from gradoom_amd import overlay_inputs

    table = overlay_inputs.fine_sine_fixed()
    # engine.py:318-319 and the symmetry R_InitTables gives the table
    assert table.shape == (8192,) and table[0] == 0 and table[2048] == 65536 and table[6144] == -65536
    assert np.array_equal(table[4096:], -table[:4096])
    assert table[1024] == int(np.trunc(np.sin(np.pi / 4) * 65536))


def test_weapon_words_match_reference_selection():
    from gradoom_amd import overlay_inputs

    meta, data, _smap, _tables = load_fixture("overlays")
    overlays = fixture_overlays(meta)
    words = overlay_inputs.weapon_state(
        **_engine(data, WEAPON_ARGUMENTS), weapon_frame_ids=torch.as_tensor(overlays["weapon_frame_ids"]),
        weapon_flash_ids=torch.as_tensor(overlays["weapon_flash_ids"]), fine_sine=torch.as_tensor(overlay_inputs.fine_sine_fixed()),
    ).numpy()
    assert words.dtype == np.int64 and words.shape == (meta["lanes"], 5)
    assert np.array_equal(words[:, 0], data["ref_weapon_frame_id"])      # engine.py:14949-14967
    assert np.array_equal(words[:, 1], data["ref_weapon_flash_id"])
    assert np.array_equal(words[:, 4], 1 - data["engine_player_dead"].astype(np.int64))
    assert np.array_equal(words, data["weapon_state"])
    # closed forms on hand-picked lanes: a lowering weapon moves 6 map pixels per tic and does not bob
    lowering = data["engine_pending_weapon"] >= 0
    assert lowering.any()
    tics = np.maximum(np.clip(16 - data["engine_weapon_lower_cooldown"], 0, 16), np.clip(14 - (data["engine_episode_time"] - 1), 0, 14))
    assert np.array_equal(words[lowering, 3], tics[lowering].astype(np.int64) * 6 * 65536)
    assert not words[lowering, 2].any()
    # the fixture must also hold bobbing lanes and lanes with a muzzle flash
    assert (words[:, 2] != 0).any() and (words[:, 1] >= 0).any() and (words[:, 1] < 0).any()


def test_status_bar_words_match_reference_face_selection():
    from gradoom_amd import overlay_inputs

    meta, data, _smap, _tables = load_fixture("overlays")
    words = overlay_inputs.hud_state(**_engine(data, HUD_ARGUMENTS)).numpy()
    assert words.dtype == np.int32 and words.shape == (meta["lanes"], 9)
    assert np.array_equal(words[:, 3], data["ref_face_patch"])           # engine.py:15209-15230
    assert np.array_equal(words, data["hud_state"])
    health = np.clip(data["engine_health"], 0, 999).astype(np.int64)     # int() truncates
    assert np.array_equal(words[:, 1], health)
    assert (words[health <= 0, 3] == 69).all() and (health <= 0).any()
    owned = words[:, 4]
    for k in range(5):
        assert np.array_equal((owned >> k) & 1, (data["engine_weapons"][:, k + 1] != 0).astype(np.int64))
    assert len(set(words[:, 3].tolist())) > 3                            # several face states are exercised


def test_decal_packing_keeps_every_slot_in_paint_order():
    # engine.py:13756-13829: live impacts in the order they were made (serial), whatever slots they sit in; the packing
    # has a fixed shape (free slots last, alive word zero) so that nothing has to wait for the device to size it
    from gradoom_amd import overlay_inputs

    rng = np.random.default_rng(5)
    lanes, slots, walls = 6, 9, 12
    serial = rng.permutation(lanes * slots).reshape(lanes, slots).astype(np.int64)
    serial[rng.random((lanes, slots)) < 0.5] = -1
    serial[2] = -1                                   # a lane without decals
    wall = rng.integers(0, walls, (lanes, slots))
    along = rng.random((lanes, slots)).astype(np.float32)
    impact_z = rng.random((lanes, slots)).astype(np.float32) * 100
    style = rng.integers(0, 40, (lanes, slots))
    portal_walls = rng.integers(-500, 500, (walls, 4)).astype(np.float32)
    table = overlay_inputs.fine_sine_fixed()
    state, geom = overlay_inputs.decal_inputs(*(torch.as_tensor(v) for v in (serial, wall, along, impact_z, style, portal_walls)), table)
    assert state.shape == (lanes, slots, 3) and state.dtype == torch.int32
    assert geom.shape == (lanes, slots, 4) and geom.dtype == torch.float32
    for lane in range(lanes):
        live = [slot for slot in np.argsort(serial[lane], kind="stable") if serial[lane, slot] >= 0]
        assert state[lane, :, 2].tolist() == [1] * len(live) + [0] * (slots - len(live))
        for position, slot in enumerate(live):
            assert int(state[lane, position, 0]) == wall[lane, slot] and int(state[lane, position, 1]) == style[lane, slot]
            assert float(geom[lane, position, 0]) == along[lane, slot] and float(geom[lane, position, 1]) == impact_z[lane, slot]
            x1, y1, x2, y2 = portal_walls[wall[lane, slot]]
            sign = 1.0 if style[lane, slot] // 20 == 0 else -1.0       # the seg runs backwards on sidedef 1
            direction = np.arctan2(np.float32(sign * (y2 - y1)), np.float32(sign * (x2 - x1)))
            # the direction goes through the 8192-entry fine-angle table: within one table step of the true cosine / sine
            assert abs(float(geom[lane, position, 2]) - np.cos(direction)) < 2e-3 and abs(float(geom[lane, position, 3]) - np.sin(direction)) < 2e-3
    assert overlay_inputs.decal_inputs(*(torch.as_tensor(v[:, :0]) for v in (serial, wall, along, impact_z, style)), torch.as_tensor(portal_walls), table) is None
