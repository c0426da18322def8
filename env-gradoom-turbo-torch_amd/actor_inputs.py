"""Gameplay state -> the renderer's packed billboard list, without leaving the device.

The reference builds the list inside ``_native_render_sprites`` (``engine.py:14328-14682``): one kind of
actor after another (monsters, the other players' start dolls, corpses, projectiles, explosions,
teleport fog, bullet puffs, map items, drops), each trimmed to the slots some lane uses with
``nonzero`` - a host synchronisation per kind and a list whose width changes from frame to frame.
``pack_actors`` keeps every slot of every kind, in the same order, and marks unused ones dead: a dead
slot draws nothing and ties between equally distant sprites are broken by list order, which trimming
does not change, so the picture is the same while the shapes are fixed and nothing waits for the host.

Only Torch ops on the engine's own tensors are used (the float32 ``atan2`` that picks a sprite rotation
among them), so the result is the reference's own on whatever device the engine lives.
"""

from __future__ import annotations

import ctypes as C
import math

import numpy as np
import torch

OPAQUE, TRANSLUCENT = -1, -2

# What pack_actors reads: attributes of the engine and of its ``map`` (names as in the reference).
ENGINE_FIELDS = (
    "x", "y", "enemy_x", "enemy_y", "enemy_z", "enemy_alive", "enemy_type", "enemy_angle", "enemy_animation_tics",
    "enemy_target_slot", "enemy_attack_phase", "enemy_cooldown", "enemy_pain_tics", "enemy_death_tics", "enemy_death_type",
    "enemy_death_elapsed", "enemy_death_extreme", "player_dead", "projectile_x", "projectile_y", "projectile_z",
    "projectile_alive", "projectile_type", "projectile_age", "projectile_velocity_x", "projectile_velocity_y",
    "projectile_impact_type", "projectile_impact_tics", "enemy_projectile_x", "enemy_projectile_y", "enemy_projectile_z",
    "enemy_projectile_alive", "enemy_projectile_age", "enemy_projectile_velocity_x", "enemy_projectile_velocity_y",
    "enemy_projectile_impact_tics", "teleport_fog_x", "teleport_fog_y", "teleport_fog_z", "teleport_fog_tics",
    "hitscan_puff_x", "hitscan_puff_y", "hitscan_puff_z", "hitscan_puff_tics", "drop_x", "drop_y", "drop_z", "drop_type",
    "drop_spawned", "item_available", "item_animation_initial_tics", "episode_time", "_enemy_walk_frame_tics",
    "_enemy_idle_frame_tics", "_enemy_attack_recovery", "_player_start_z", "_item_z",
)
MAP_FIELDS = (
    "enemy_walk_sprite_ids", "enemy_attack_sprite_ids", "enemy_pain_sprite_ids", "enemy_death_sprite_ids",
    "enemy_death_frame_durations", "enemy_death_frame_counts", "enemy_xdeath_sprite_ids", "enemy_xdeath_frame_durations",
    "enemy_xdeath_frame_counts", "projectile_explosion_total_tics", "projectile_explosion_frame_durations",
    "projectile_explosion_frame_counts", "raw_projectile_explosion_sprite_ids", "raw_projectile_flight_sprite_ids",
    "raw_teleport_fog_sprite_ids", "raw_bullet_puff_sprite_ids", "raw_static_sprite_ids", "raw_item_animation_sprite_ids",
    "item_raw_visual_types", "item_types", "item_spawns", "player_starts",
)


def _rotation(viewer_angle: torch.Tensor, actor_angle: torch.Tensor) -> torch.Tensor:
    """Doom's clockwise 1..8 sprite rotation as 0..7 (``engine.py:13994-14009``)."""

    turn = torch.remainder(viewer_angle - actor_angle + math.pi / 8, 2 * math.pi)
    return torch.remainder(torch.floor(turn / (math.pi / 4)).to(torch.int64), 8)


def _seen_from(engine, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    return torch.atan2(engine.y[:, None] - y, engine.x[:, None] - x)


def _frame_after(elapsed: torch.Tensor, durations: torch.Tensor, counts: torch.Tensor) -> torch.Tensor:
    """Index of the animation frame showing after ``elapsed`` tics, held on the last one."""

    ends = torch.cumsum(durations, dim=-1)
    return torch.minimum(torch.sum(elapsed[..., None] >= ends, dim=-1), counts - 1)


def monster_patches(engine) -> torch.Tensor:
    """Patch of every monster slot: walk / idle, attack or pain frame seen from the camera
    (``engine.py:14011-14077``)."""

    m = engine.map
    kind = engine.enemy_type.clamp(0, 5)
    facing = _rotation(_seen_from(engine, engine.enemy_x, engine.enemy_y), engine.enemy_angle)
    tics = engine.enemy_animation_tics
    walking = torch.remainder(tics // engine._enemy_walk_frame_tics[kind], 4).to(torch.int64)
    idling = torch.remainder(tics // engine._enemy_idle_frame_tics[kind], 2).to(torch.int64)
    idling = idling.masked_fill(kind == 2, 0)                       # the marine stands on one frame
    walking = torch.where(engine.enemy_target_slot < -1, idling, walking)
    phase, cooldown = engine.enemy_attack_phase, engine.enemy_cooldown
    hitscanner = (kind == 0) | (kind == 1)
    melee = (kind == 4) | (kind == 5)
    recovering = (cooldown > (engine._enemy_attack_recovery[kind] // 2)).to(torch.int64)
    attacking = torch.zeros_like(kind)
    attacking = torch.where(hitscanner & (phase == 2), recovering, attacking)
    attacking = torch.where(melee & (phase == 1), (cooldown <= 8).to(torch.int64), attacking)
    attacking = attacking.masked_fill(melee & (phase == 2), 2)
    attacking = attacking.masked_fill((kind == 3) & ((phase == 4) | (phase == 2)), 1)
    attacking = attacking.masked_fill((kind == 3) & (phase == 3), 2)
    moving = torch.where(phase > 0, m.enemy_attack_sprite_ids[kind, attacking, facing], m.enemy_walk_sprite_ids[kind, walking, facing])
    return torch.where(engine.enemy_pain_tics > 0, m.enemy_pain_sprite_ids[kind, facing], moving)


def monster_bright(engine) -> torch.Tensor:
    """Muzzle-flash frames are full bright (``engine.py:14125-14136``)."""

    kind = engine.enemy_type.clamp(0, 5)
    phase = engine.enemy_attack_phase
    shotgun = (kind == 1) & (phase == 2) & (engine.enemy_cooldown > (engine._enemy_attack_recovery[kind] // 2))
    chaingun = (kind == 3) & ((phase == 2) | (phase == 3))
    return shotgun | chaingun


def corpse_patches(engine) -> torch.Tensor:
    """Death or gib animation frame of every monster slot (``engine.py:14079-14106``)."""

    m = engine.map
    kind = engine.enemy_death_type.clamp(0, 5)
    elapsed = engine.enemy_death_elapsed.to(torch.int64)
    plain = m.enemy_death_sprite_ids[kind, _frame_after(elapsed, m.enemy_death_frame_durations[kind], m.enemy_death_frame_counts[kind])]
    gibbed = m.enemy_xdeath_sprite_ids[kind, _frame_after(elapsed, m.enemy_xdeath_frame_durations[kind], m.enemy_xdeath_frame_counts[kind])]
    return torch.where(engine.enemy_death_extreme, gibbed, plain)


def explosion_patches(engine, kind: torch.Tensor, remaining: torch.Tensor) -> torch.Tensor:
    """Explosion frame of a projectile that hit something (``engine.py:14108-14123``)."""

    m = engine.map
    kind = kind.clamp(0, 2)
    elapsed = m.projectile_explosion_total_tics[kind] - remaining.to(torch.int64)
    frame = _frame_after(elapsed, m.projectile_explosion_frame_durations[kind], m.projectile_explosion_frame_counts[kind])
    return m.raw_projectile_explosion_sprite_ids[kind, frame]


def item_patches(engine) -> tuple[torch.Tensor, torch.Tensor]:
    """Patch and full-bright flag of every map item; bonuses and armours animate (``engine.py:14258-14317``)."""

    m = engine.map
    lanes = engine.x.shape[0]
    still = m.item_raw_visual_types[None, :].expand(lanes, -1)
    kinds = m.item_types[None, :]
    frames = m.raw_item_animation_sprite_ids
    elapsed = engine.episode_time[:, None] + (6 - engine.item_animation_initial_tics)
    phase = torch.remainder(elapsed // 6, 6)                        # A B C D C B, six tics each; A is the still patch
    back_and_forth = 2 - torch.abs(phase - 3)                       # -1 0 1 2 1 0
    health = torch.where(back_and_forth < 0, still, frames[back_and_forth.clamp_min(0)])
    armor = torch.where(back_and_forth < 0, still, frames[back_and_forth.clamp_min(0) + 3])
    patch = torch.where(kinds == 2014, health, still)
    patch = torch.where(kinds == 2015, armor, patch)
    green = (kinds == 2018) & (torch.remainder(elapsed, 13) >= 6)
    blue = (kinds == 2019) & (torch.remainder(elapsed, 12) >= 6)
    patch = torch.where(green, frames[6], patch)
    patch = torch.where(blue, frames[7], patch)
    return patch, green | blue


def pack_actors(engine, limit: int = 512) -> dict[str, torch.Tensor]:
    """Fixed-shape ``sprite_*`` inputs of ``gd_lanes_desc`` from a ``TorchDeathmatchEngine``-like object.

    Returns ``sprite_x/y/z`` f32, ``sprite_id`` i32, ``sprite_alive`` / ``sprite_fullbright`` u8 and
    ``sprite_style`` i8, all ``[N, A]`` with A the sum of every kind's slot count.  The renderer takes at
    most 512 slots per lane: a longer list is cut to ``limit`` after moving each lane's live slots to the
    front in their original order (a stable sort on the device), which loses nothing unless a lane shows
    more than ``limit`` actors at once.
    """

    m = engine.map
    lanes = engine.x.shape[0]
    device = engine.x.device
    kinds: list[tuple] = []      # x, y, z, patch, alive, bright, style

    def full(like: torch.Tensor, value: int) -> torch.Tensor:
        return torch.full(like.shape, value, dtype=torch.int64, device=device)

    # monsters
    kinds.append((engine.enemy_x, engine.enemy_y, engine.enemy_z, monster_patches(engine), engine.enemy_alive,
                  monster_bright(engine), full(engine.enemy_x, OPAQUE)))
    # the other players' start spots show a marine while the player lives (engine.py:14345-14379)
    dolls = m.player_starts[:-1]
    if len(dolls):
        x = dolls[None, :, 0].expand(lanes, -1)
        y = dolls[None, :, 1].expand(lanes, -1)
        facing = _rotation(_seen_from(engine, x, y), torch.deg2rad(dolls[None, :, 2]).expand(lanes, -1))
        kinds.append((x, y, engine._player_start_z[:-1][None, :].expand(lanes, -1), m.enemy_walk_sprite_ids[2, 0, facing],
                      (~engine.player_dead)[:, None].expand(-1, len(dolls)), torch.zeros_like(facing, dtype=torch.bool),
                      full(facing, OPAQUE)))
    # corpses
    dying = engine.enemy_death_tics > 0
    kinds.append((engine.enemy_x, engine.enemy_y, engine.enemy_z, corpse_patches(engine), dying, torch.zeros_like(dying),
                  full(engine.enemy_x, OPAQUE)))
    # the player's rockets and plasma balls in flight (engine.py:14410-14460): plasma blends additively
    shot = engine.projectile_type.clamp(0, 1)
    facing = _rotation(_seen_from(engine, engine.projectile_x, engine.projectile_y),
                       torch.atan2(engine.projectile_velocity_y, engine.projectile_velocity_x))
    frame = torch.where(shot == 1, torch.remainder(engine.projectile_age // 6, 2).to(torch.int64), torch.zeros_like(shot))
    kinds.append((engine.projectile_x, engine.projectile_y, engine.projectile_z, m.raw_projectile_flight_sprite_ids[shot, frame, facing],
                  engine.projectile_alive, engine.projectile_alive, torch.where(shot == 1, 0, OPAQUE)))
    # monster fireballs in flight (engine.py:14462-14510)
    facing = _rotation(_seen_from(engine, engine.enemy_projectile_x, engine.enemy_projectile_y),
                       torch.atan2(engine.enemy_projectile_velocity_y, engine.enemy_projectile_velocity_x))
    frame = torch.remainder(engine.enemy_projectile_age // 4, 2).to(torch.int64)
    kinds.append((engine.enemy_projectile_x, engine.enemy_projectile_y, engine.enemy_projectile_z,
                  m.raw_projectile_flight_sprite_ids[2, frame, facing], engine.enemy_projectile_alive, engine.enemy_projectile_alive,
                  full(frame, 1)))
    # explosions of both (engine.py:14512-14573)
    bursting = engine.projectile_impact_tics > 0
    kinds.append((engine.projectile_x, engine.projectile_y, engine.projectile_z,
                  explosion_patches(engine, engine.projectile_impact_type, engine.projectile_impact_tics), bursting, bursting,
                  torch.where(engine.projectile_impact_type == 1, 0, OPAQUE)))
    bursting = engine.enemy_projectile_impact_tics > 0
    fireball = full(engine.enemy_projectile_x, 2)
    kinds.append((engine.enemy_projectile_x, engine.enemy_projectile_y, engine.enemy_projectile_z,
                  explosion_patches(engine, fireball, engine.enemy_projectile_impact_tics), bursting, bursting,
                  full(engine.enemy_projectile_x, 1)))
    # teleport fog: twelve frames of six tics out of 72 (engine.py:14577-14595)
    tics = engine.teleport_fog_tics
    frame = torch.clamp((72 - tics.to(torch.int64)) // 6, max=11)
    kinds.append((engine.teleport_fog_x, engine.teleport_fog_y, engine.teleport_fog_z, m.raw_teleport_fog_sprite_ids[frame], tics > 0,
                  tics > 0, full(frame, 1)))
    # bullet puffs: four frames of four tics, the first one bright, all translucent (engine.py:14597-14630)
    tics = engine.hitscan_puff_tics
    frame = (3 - torch.clamp((tics.to(torch.int64) - 1) // 4, 0, 3))
    kinds.append((engine.hitscan_puff_x, engine.hitscan_puff_y, engine.hitscan_puff_z, m.raw_bullet_puff_sprite_ids[frame], tics > 0,
                  frame == 0, full(frame, TRANSLUCENT)))
    # map items
    if len(m.item_types):
        patch, bright = item_patches(engine)
        kinds.append((m.item_spawns[None, :, 0].expand(lanes, -1), m.item_spawns[None, :, 1].expand(lanes, -1),
                      engine._item_z[None, :].expand(lanes, -1), patch, engine.item_available, bright, full(patch, OPAQUE)))
    # what monsters drop (engine.py:14657-14682)
    static = m.raw_static_sprite_ids
    patch = static[12].expand_as(engine.drop_type)
    patch = torch.where(engine.drop_type == 2007, static[6], patch)
    patch = torch.where(engine.drop_type == 2002, static[14], patch)
    lying = (engine.drop_type >= 0) & engine.drop_spawned
    kinds.append((engine.drop_x, engine.drop_y, engine.drop_z, patch, lying, torch.zeros_like(lying), full(patch, OPAQUE)))

    def column(k: int, dtype) -> torch.Tensor:
        return torch.cat([kind[k].to(dtype) for kind in kinds], dim=1).contiguous()

    packed = dict(
        sprite_x=column(0, torch.float32), sprite_y=column(1, torch.float32), sprite_z=column(2, torch.float32),
        sprite_id=column(3, torch.int32), sprite_alive=column(4, torch.uint8), sprite_fullbright=column(5, torch.uint8),
        sprite_style=column(6, torch.int8),
    )
    return compact_actors(packed, limit) if limit else packed


def compact_actors(packed: dict[str, torch.Tensor], limit: int) -> dict[str, torch.Tensor]:
    """Cut a packed list to ``limit`` slots per lane, live slots first and in their original order."""

    if packed["sprite_alive"].shape[1] <= limit:
        return packed
    front = torch.argsort(1 - packed["sprite_alive"].to(torch.int16), dim=1, stable=True)[:, :limit]
    return {key: value.gather(1, front).contiguous() for key, value in packed.items()}


_TORCH_OF = {np.float32: torch.float32, np.uint8: torch.uint8, np.int64: torch.int64, np.int32: torch.int32, np.int8: torch.int8}


def pack_actors_fused(engine, limit: int = 512) -> dict[str, torch.Tensor]:
    """``pack_actors`` as one HIP kernel (``gd_pack_actors``): same list, same order, same dtypes.

    The four sprite rotations still come from the reference's float32 Torch ops (``atan2``); everything
    else - frame selection, patch lookup, flags, the concatenation - happens in one launch that reads the
    engine's tensors where they are.  Needs the engine on a ROCm device and the library built.
    """

    from . import _abi, _lib

    m = engine.map
    device = engine.x.device
    if device.type != "cuda":
        raise RuntimeError("pack_actors_fused needs the engine's tensors on the GPU")
    lanes = int(engine.x.shape[0])
    dolls = m.player_starts[:-1]
    rotations = dict(
        enemy_rotation=_rotation(_seen_from(engine, engine.enemy_x, engine.enemy_y), engine.enemy_angle),
        projectile_rotation=_rotation(_seen_from(engine, engine.projectile_x, engine.projectile_y),
                                      torch.atan2(engine.projectile_velocity_y, engine.projectile_velocity_x)),
        enemy_projectile_rotation=_rotation(_seen_from(engine, engine.enemy_projectile_x, engine.enemy_projectile_y),
                                            torch.atan2(engine.enemy_projectile_velocity_y, engine.enemy_projectile_velocity_x)),
    )
    if len(dolls):
        doll_x = dolls[None, :, 0].expand(lanes, -1)
        doll_y = dolls[None, :, 1].expand(lanes, -1)
        rotations["doll_rotation"] = _rotation(_seen_from(engine, doll_x, doll_y), torch.deg2rad(dolls[None, :, 2]).expand(lanes, -1))
    derived = dict(
        doll_x=dolls[:, 0], doll_y=dolls[:, 1], doll_z=engine._player_start_z[:-1],
        item_x=m.item_spawns[:, 0], item_y=m.item_spawns[:, 1], item_z=engine._item_z,
        enemy_walk_frame_tics=engine._enemy_walk_frame_tics, enemy_idle_frame_tics=engine._enemy_idle_frame_tics,
        enemy_attack_recovery=engine._enemy_attack_recovery,
    )
    desc = _abi.ActorDesc()
    desc.lane_count = lanes
    desc.enemy_slots = int(engine.enemy_x.shape[1])
    desc.doll_count = int(len(dolls))
    desc.player_projectile_slots = int(engine.projectile_x.shape[1])
    desc.enemy_projectile_slots = int(engine.enemy_projectile_x.shape[1])
    desc.fog_slots = int(engine.teleport_fog_x.shape[1])
    desc.puff_slots = int(engine.hitscan_puff_x.shape[1])
    desc.item_count = int(len(m.item_types))
    desc.drop_slots = int(engine.drop_x.shape[1])
    desc.attack_frames = int(m.enemy_attack_sprite_ids.shape[1])
    desc.death_frames = int(m.enemy_death_sprite_ids.shape[1])
    desc.xdeath_frames = int(m.enemy_xdeath_sprite_ids.shape[1])
    desc.explosion_frames = int(m.raw_projectile_explosion_sprite_ids.shape[1])
    if int(m.raw_static_sprite_ids.shape[0]) < 15:
        raise ValueError("raw_static_sprite_ids needs at least 15 entries")
    keep = []
    for name, dtype in _abi.ACTOR_ARRAYS:
        if name in rotations:
            value = rotations[name].to(torch.uint8)
        elif name in derived:
            value = derived[name]
        elif hasattr(engine, name):
            value = getattr(engine, name)
        else:
            value = getattr(m, name)
        wanted = _TORCH_OF[dtype]
        if value.dtype == torch.bool and wanted == torch.uint8:
            value = value.view(torch.uint8) if value.is_contiguous() else value.contiguous().view(torch.uint8)
        if value.dtype != wanted:
            raise TypeError(f"{name} must be {wanted}, got {value.dtype}")
        if value.device != device:
            raise TypeError(f"{name} must live on {device}")
        value = value.contiguous()
        keep.append(value)
        setattr(desc, name, value.data_ptr() if value.numel() else None)
    width = (2 * desc.enemy_slots + desc.doll_count + 2 * desc.player_projectile_slots + 2 * desc.enemy_projectile_slots
             + desc.fog_slots + desc.puff_slots + desc.item_count + desc.drop_slots)
    packed = {}
    for name, dtype in _abi.ACTOR_OUTPUTS:
        packed[name] = torch.empty((lanes, width), dtype=_TORCH_OF[dtype], device=device)
        setattr(desc, name, packed[name].data_ptr())
    stream = torch.cuda.current_stream(device).cuda_stream
    _lib.check(_lib.library().gd_pack_actors(C.byref(desc), C.c_void_p(stream)))
    del keep
    return compact_actors(packed, limit) if limit else packed
