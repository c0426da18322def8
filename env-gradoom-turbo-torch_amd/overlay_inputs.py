"""Host-side inputs of the overlay layers: the per-lane words ``gd_lanes_desc.weapon_state`` and
``gd_lanes_desc.hud_state`` worked out from the engine's gameplay tensors.

Both are a few integer Torch ops per lane on whatever device the tensors live on (no host sync);
the kernels then only composite patches.  Every function takes tensors named like the reference
engine's attributes and cites the lines it mirrors.
"""

from __future__ import annotations

import math

import numpy as np
import torch

FIXED_UNIT = 65536
FINE_ANGLES = 8192
WEAPON_LOWER_TICS = 16          # engine.py:111
WEAPON_SPAWN_RAISE_TICS = 14    # engine.py:114
MUGSHOT_RAMPAGE_DELAY = 70      # engine.py:175


def fine_sine_fixed() -> np.ndarray:
    """ZDoom's 16.16 ``finesine`` table (``engine.py:309-321``)."""

    quarter = FINE_ANGLES // 4
    table = np.empty(FINE_ANGLES, dtype=np.int64)
    phase = np.arange(quarter, dtype=np.float64) * (2.0 * math.pi / FINE_ANGLES)
    first_quarter = np.trunc(np.sin(phase) * FIXED_UNIT).astype(np.int64)
    table[:quarter] = first_quarter
    table[quarter : 2 * quarter] = first_quarter[::-1]
    table[2 * quarter :] = -table[: 2 * quarter]
    table[quarter] = FIXED_UNIT
    table[3 * quarter] = -FIXED_UNIT
    return table


def weapon_state(
    *,
    active_weapon: torch.Tensor,
    weapon_state_cooldown: torch.Tensor,
    weapon_fire_count: torch.Tensor,
    weapon_ready_tics: torch.Tensor,
    weapon_lower_cooldown: torch.Tensor,
    weapon_raise_cooldown: torch.Tensor,
    pending_weapon: torch.Tensor,
    episode_time: torch.Tensor,
    player_bob_fixed: torch.Tensor,
    player_dead: torch.Tensor,
    weapon_frame_ids: torch.Tensor,
    weapon_flash_ids: torch.Tensor,
    fine_sine: torch.Tensor,
) -> torch.Tensor:
    """``int64 [N,5]``: patch id, flash patch id, horizontal and vertical offset (16.16), visible.

    ``_native_weapon_frame_selection`` (``engine.py:14949-14967``) and the offsets of
    ``_native_render_weapon`` (``engine.py:15051-15092``).  ``weapon_frame_ids`` / ``weapon_flash_ids``
    are the map's ``[8, 2, cooldowns]`` tables, ``fine_sine`` the table of :func:`fine_sine_fixed`.
    """

    weapon = active_weapon.to(torch.int64).clamp(0, 7)
    cooldown = weapon_state_cooldown.to(torch.int64).clamp(0, weapon_frame_ids.shape[2] - 1)
    parity = torch.remainder(weapon_fire_count, 2).to(torch.int64)
    idle_chainsaw = (weapon == 1) & (cooldown == 0)
    idle_phase = torch.remainder(torch.clamp_min(weapon_ready_tics - 1, 0) // 4, 2).to(torch.int64)
    parity = torch.where(idle_chainsaw, idle_phase, parity)
    frame_id = weapon_frame_ids[weapon, parity, cooldown].to(torch.int64)
    flash_id = weapon_flash_ids[weapon, parity, cooldown].to(torch.int64)

    lower_vertical_tics = torch.clamp(WEAPON_LOWER_TICS - weapon_lower_cooldown, 0, WEAPON_LOWER_TICS)
    vertical_tics = torch.where(pending_weapon >= 0, lower_vertical_tics, weapon_raise_cooldown)
    spawn_raise_tics = torch.clamp(WEAPON_SPAWN_RAISE_TICS - (episode_time - 1), 0, WEAPON_SPAWN_RAISE_TICS)
    vertical_tics = torch.maximum(vertical_tics, spawn_raise_tics)
    ready = (weapon_state_cooldown <= 0) & (weapon_raise_cooldown <= 0) & (pending_weapon < 0)
    bob_angle = (episode_time.to(torch.int64) * 128) & (FINE_ANGLES - 1)
    bob = player_bob_fixed.to(torch.int64)
    bob_x_fixed = (bob * fine_sine[(bob_angle + FINE_ANGLES // 4) & (FINE_ANGLES - 1)]) >> 16
    bob_y_fixed = (bob * fine_sine[bob_angle & (FINE_ANGLES // 2 - 1)]) >> 16
    bob_x_fixed = torch.where(ready, bob_x_fixed, torch.zeros_like(bob_x_fixed))
    bob_y_fixed = torch.where(ready, bob_y_fixed, torch.zeros_like(bob_y_fixed))
    vertical_offset_fixed = vertical_tics.to(torch.int64) * 6 * FIXED_UNIT + bob_y_fixed
    visible = (~player_dead).to(torch.int64)
    return torch.stack((frame_id, flash_id, bob_x_fixed, vertical_offset_fixed, visible), dim=1).contiguous()


def mugshot_patch(
    *,
    health: torch.Tensor,
    mugshot_face_index: torch.Tensor,
    mugshot_grin_tics: torch.Tensor,
    mugshot_pain_tics: torch.Tensor,
    mugshot_ouch: torch.Tensor,
    mugshot_pain_direction: torch.Tensor,
    attack_held_tics: torch.Tensor,
) -> torch.Tensor:
    """Face patch id per lane (``_native_mugshot_patch_index``, ``engine.py:15209-15230``); ``health`` already an integer."""

    health = health.to(torch.int64)
    # Python's floor division of (100 - health) by 20, clamped to 0..4
    pain = torch.clamp(torch.div(100 - health, 20, rounding_mode="floor"), 0, 4)
    face = 13 + pain * 3 + mugshot_face_index.to(torch.int64)
    rampage = attack_held_tics >= MUGSHOT_RAMPAGE_DELAY
    face = torch.where(rampage, 49 + pain, face)
    direction_base = torch.tensor((44, 49, 54), dtype=torch.int64, device=health.device)[mugshot_pain_direction.to(torch.int64)]
    pained = torch.where(mugshot_ouch, 59 + pain, direction_base + pain)
    face = torch.where(mugshot_pain_tics > 0, pained, face)
    face = torch.where(mugshot_grin_tics > 0, 64 + pain, face)
    return torch.where(health <= 0, torch.full_like(face, 69), face)


def hud_state(
    *,
    active_weapon: torch.Tensor,
    weapon_ammo_slot: torch.Tensor,
    hud_ready_ammo: torch.Tensor,
    health: torch.Tensor,
    armor: torch.Tensor,
    weapons: torch.Tensor,
    hud_ammo_counts: torch.Tensor,
    mugshot_face_index: torch.Tensor,
    mugshot_grin_tics: torch.Tensor,
    mugshot_pain_tics: torch.Tensor,
    mugshot_ouch: torch.Tensor,
    mugshot_pain_direction: torch.Tensor,
    attack_held_tics: torch.Tensor,
) -> torch.Tensor:
    """``int32 [N,9]``: ready ammo, health, armor, face patch, owned-weapon bits, four ammo counts.

    The numbers ``_native_render_hud`` reads with ``int(tensor.item())`` per lane
    (``engine.py:15240-15262``): ``int()`` truncates the float tensors toward zero.
    """

    ammo_slot = weapon_ammo_slot[active_weapon.to(torch.int64)]
    ammo = torch.where(ammo_slot < 0, torch.zeros_like(hud_ready_ammo), hud_ready_ammo).to(torch.int64)
    health_int = health.clamp(0, 999).to(torch.int64)
    armor_int = armor.clamp(0, 999).to(torch.int64)
    face = mugshot_patch(
        health=health_int, mugshot_face_index=mugshot_face_index, mugshot_grin_tics=mugshot_grin_tics,
        mugshot_pain_tics=mugshot_pain_tics, mugshot_ouch=mugshot_ouch, mugshot_pain_direction=mugshot_pain_direction,
        attack_held_tics=attack_held_tics,
    )
    owned = torch.zeros_like(face)
    for weapon_index in range(5):  # bool(self.weapons[lane, weapon_index + 1])
        owned |= (weapons[:, weapon_index + 1] != 0).to(torch.int64) << weapon_index
    counts = hud_ammo_counts.to(torch.int64)
    columns = (ammo, health_int, armor_int, face, owned, counts[:, 0], counts[:, 1], counts[:, 2], counts[:, 3])
    return torch.stack(columns, dim=1).to(torch.int32).contiguous()


def screen_blend(bonus_count: torch.Tensor, damage_count: torch.Tensor, damage_to_alpha: torch.Tensor) -> torch.Tensor:
    """f32 [N,2]: the pickup and damage alphas of ``_native_indexed_to_rgb`` (engine.py:15385-15394).

    ``damage_to_alpha`` is the engine's 114-entry ``_damage_to_alpha`` table.  Lanes carrying this
    tensor get PLAYPAL mixed with gold and then red before the RGB24 frame and the observation.
    """

    bonus = torch.minimum(bonus_count.to(torch.float32) * 8.0, torch.full_like(bonus_count, 128.0, dtype=torch.float32))
    flash = damage_to_alpha.to(torch.float32)[damage_count.clamp(0, 113).to(torch.int64)]
    return torch.stack((bonus / 255.0, flash / 255.0), dim=1).contiguous()


def decal_inputs(serial, wall, along, impact_z, style, portal_walls, fine_sine_fixed):
    """Pack the wall decals of every lane in paint order (engine.py:13756-13829).

    ``serial, wall, along, impact_z, style`` are the engine's ``hitscan_decal_*`` tensors ``[N, slots]``
    (serial < 0 = free slot), ``portal_walls`` the map's ``[W,4]`` linedefs and ``fine_sine_fixed`` the
    8192-entry fine sine table (``fine_sine_fixed()``).  Returns ``(decal_state i32 [N,D,3], decal_geom
    f32 [N,D,4])`` with D the largest number of live decals in a lane, or ``None`` when no lane has one.
    Older impacts come first so that a later chip shades an earlier one at the same texels.
    """

    active_slots = torch.nonzero(torch.any(serial >= 0, dim=0)).flatten()
    if not active_slots.numel():
        return None
    serial = serial[:, active_slots].to(torch.int64)
    active = serial >= 0
    layers = int(torch.amax(torch.sum(active, dim=1)).item())
    order = torch.argsort(torch.where(active, serial, torch.full_like(serial, torch.iinfo(torch.int32).max)), dim=1)
    order = order[:, :layers]
    pick = lambda tensor: tensor[:, active_slots].gather(1, order)  # noqa: E731
    alive = active.gather(1, order)
    wall_index = pick(wall).to(torch.int64).clamp(0, portal_walls.shape[0] - 1)
    style_index = pick(style).to(torch.int64)
    side = style_index // 20
    segment = portal_walls[wall_index]
    vector = segment[..., 2:] - segment[..., :2]
    # the seg runs backwards on sidedef 1; its direction goes through the fine-angle table
    oriented = torch.where((side == 0)[..., None], vector, -vector)
    angle = torch.atan2(oriented[..., 1], oriented[..., 0])
    fine = torch.floor(torch.remainder(angle, 2.0 * math.pi) * (8192 / (2.0 * math.pi))).to(torch.int64) & 8191
    table = torch.as_tensor(fine_sine_fixed, dtype=torch.int64).to(serial.device)
    sine = table[fine].to(torch.float32) / 65536
    cosine = table[(fine + 2048) & 8191].to(torch.float32) / 65536
    state = torch.stack((wall_index, style_index, alive.to(torch.int64)), dim=-1).to(torch.int32).contiguous()
    geom = torch.stack((pick(along).to(torch.float32), pick(impact_z).to(torch.float32), cosine, sine), dim=-1).contiguous()
    return state, geom
