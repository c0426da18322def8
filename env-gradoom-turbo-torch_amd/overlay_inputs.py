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


_WEAPON_INPUTS = (
    "active_weapon", "weapon_state_cooldown", "weapon_fire_count", "weapon_ready_tics", "weapon_lower_cooldown",
    "weapon_raise_cooldown", "pending_weapon", "episode_time", "player_bob_fixed",
)


def weapon_state(*, weapon_frame_ids: torch.Tensor, weapon_flash_ids: torch.Tensor, fine_sine: torch.Tensor,
                 weapon_flash_lights: torch.Tensor | None = None, want_flash_light: bool = False, **engine: torch.Tensor):
    """``int64 [N,5]``: patch id, flash patch id, horizontal and vertical offset (16.16), visible.

    The per-lane half of the reference's weapon layer: ``_native_weapon_frame_selection``
    (``engine.py:14949-14967``) and the raise / lower / bob offsets of ``_native_render_weapon``
    (``engine.py:15051-15092``).  ``engine`` holds the gameplay tensors by the engine's attribute names
    (``active_weapon`` = ``_active_weapon()``, ``player_bob_fixed`` = ``_player_bob_fixed``, ``player_dead`` bool);
    ``weapon_frame_ids`` / ``weapon_flash_ids`` / ``weapon_flash_lights`` are the map's ``[8, 2, cooldowns]`` tables,
    ``fine_sine`` the table of :func:`fine_sine_fixed`.  With ``want_flash_light`` the muzzle flash's extra light level
    comes back as well (``int64 [N]``).

    Tensors on a ROCm device are read where they are by one kernel (``gd_pack_weapon``): no host synchronisation.
    Host tensors (tests, fixture scripts) take the NumPy restatement below.
    """

    if engine["episode_time"].device.type == "cuda":
        return _weapon_state_device(engine, weapon_frame_ids, weapon_flash_ids, weapon_flash_lights, fine_sine, want_flash_light)
    host = {name: np.asarray(value.cpu()).astype(np.int64) for name, value in engine.items() if name in _WEAPON_INPUTS}
    words, light = _weapon_words_host(
        host, np.asarray(engine["player_dead"].cpu()).astype(bool), np.asarray(weapon_frame_ids.cpu()).astype(np.int64),
        np.asarray(weapon_flash_ids.cpu()).astype(np.int64),
        None if weapon_flash_lights is None else np.asarray(weapon_flash_lights.cpu()).astype(np.int64), np.asarray(fine_sine.cpu()).astype(np.int64),
    )
    words = torch.as_tensor(words)
    return (words, torch.as_tensor(light)) if want_flash_light else words


def _weapon_state_device(engine, frame_ids, flash_ids, flash_lights, fine_sine, want_flash_light):
    import ctypes as C

    from . import _abi, _lib

    device = engine["episode_time"].device
    count = int(engine["episode_time"].shape[0])
    desc = _abi.WeaponDesc()
    desc.lane_count = count
    desc.cooldown_slots = int(frame_ids.shape[2])
    keep = []

    def pointer(tensor, dtype):
        if tensor.device != device:
            raise TypeError("every weapon tensor must live on the engine's device")
        tensor = tensor.to(dtype).contiguous()   # a no-op for tensors that already are
        keep.append(tensor)
        return tensor.data_ptr()

    for name in _WEAPON_INPUTS:
        setattr(desc, name, pointer(engine[name], torch.int64))
    desc.player_dead = pointer(engine["player_dead"], torch.uint8)
    desc.weapon_frame_ids = pointer(frame_ids, torch.int64)
    desc.weapon_flash_ids = pointer(flash_ids, torch.int64)
    desc.fine_sine = pointer(fine_sine, torch.int64)
    words = torch.empty((count, 5), dtype=torch.int64, device=device)
    desc.weapon_state = words.data_ptr()
    light = None
    if want_flash_light:
        if flash_lights is None:
            raise ValueError("want_flash_light needs weapon_flash_lights")
        desc.weapon_flash_lights = pointer(flash_lights, torch.int64)
        light = torch.empty((count,), dtype=torch.int64, device=device)
        desc.flash_light = light.data_ptr()
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        _lib.check(_lib.library().gd_pack_weapon(C.byref(desc), C.c_void_p(stream)))
    del keep
    return (words, light) if want_flash_light else words


def _weapon_words_host(state: dict, dead: np.ndarray, frame_table: np.ndarray, flash_table: np.ndarray, light_table, sine: np.ndarray):
    """The words of :func:`weapon_state` for host arrays, as the kernel computes them (test infrastructure)."""

    tics = state["episode_time"]
    slot = np.clip(state["active_weapon"], 0, 7)
    step = np.clip(state["weapon_state_cooldown"], 0, frame_table.shape[2] - 1)
    phase = np.mod(state["weapon_fire_count"], 2)
    idling_saw = (slot == 1) & (step == 0)             # the chainsaw's idle frames alternate every four tics
    phase[idling_saw] = (np.maximum(state["weapon_ready_tics"][idling_saw] - 1, 0) // 4) % 2
    words = np.zeros((len(tics), 5), dtype=np.int64)
    words[:, 0] = frame_table[slot, phase, step]
    words[:, 1] = flash_table[slot, phase, step]
    switching = state["pending_weapon"] >= 0
    drop = np.where(switching, np.clip(WEAPON_LOWER_TICS - state["weapon_lower_cooldown"], 0, WEAPON_LOWER_TICS), state["weapon_raise_cooldown"])
    drop = np.maximum(drop, np.clip(WEAPON_SPAWN_RAISE_TICS + 1 - tics, 0, WEAPON_SPAWN_RAISE_TICS))
    steady = (state["weapon_state_cooldown"] <= 0) & (state["weapon_raise_cooldown"] <= 0) & ~switching
    swing = (tics * 128) % FINE_ANGLES
    bob = state["player_bob_fixed"]
    words[:, 2] = np.where(steady, (bob * sine[(swing + FINE_ANGLES // 4) % FINE_ANGLES]) >> 16, 0)
    words[:, 3] = drop * (6 * FIXED_UNIT) + np.where(steady, (bob * sine[swing % (FINE_ANGLES // 2)]) >> 16, 0)
    words[:, 4] = ~dead
    light = None if light_table is None else light_table[slot, phase, step]
    return words, light


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
    direction_base = 44 + 5 * mugshot_pain_direction.to(torch.int64)   # 44, 49, 54 for directions 0, 1, 2 (no table: a device constant would be copied from the host every call)
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
    8192-entry fine sine table (``fine_sine_fixed()``).  Returns ``(decal_state i32 [N,slots,3], decal_geom
    f32 [N,slots,4])``, or ``None`` when the engine keeps no decal slots.  The shape is fixed: every slot is packed,
    live ones first and older impacts before newer ones (a later chip shades an earlier one at the same texels), free
    slots last with their ``alive`` word zero, which the decal kernel skips.  Nothing here waits for the device.
    """

    if serial.shape[1] == 0:
        return None
    serial = serial.to(torch.int64)
    active = serial >= 0
    order = torch.argsort(torch.where(active, serial, torch.full_like(serial, torch.iinfo(torch.int32).max)), dim=1, stable=True)
    pick = lambda tensor: tensor.gather(1, order)  # noqa: E731
    alive = pick(active)
    wall_index = pick(wall).to(torch.int64).clamp(0, portal_walls.shape[0] - 1)
    style_index = pick(style).to(torch.int64)
    side = torch.div(style_index, 20, rounding_mode="floor")
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
