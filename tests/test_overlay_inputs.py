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
