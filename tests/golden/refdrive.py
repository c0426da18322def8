"""Drive the reference's Torch CPU render path on synthetic maps (build container only).

The reference package cannot be imported as ``gradoom`` here because its
``__init__``/``env`` modules need ``gymnasium``; the render path itself lives in
``gradoom.engine`` + ``gradoom.scenario`` which only need torch/numpy.  This
module registers an empty parent package whose ``__path__`` points at the
reference sources and imports just those two modules.  It is used only by
``make_golden.py`` to write fixtures; nothing on the GPU box imports it.
"""

from __future__ import annotations

import importlib
import os
import sys
import types

import numpy as np
import torch

REFERENCE_SRC = os.environ.get("GRADOOM_REFERENCE_SRC", "/root/reference/src/gradoom")


def load_reference():
    if "gradoom.engine" in sys.modules:
        return sys.modules["gradoom.engine"], sys.modules["gradoom.scenario"]
    if not os.path.isdir(REFERENCE_SRC):
        raise RuntimeError(f"reference sources not found at {REFERENCE_SRC}")
    parent = types.ModuleType("gradoom")
    parent.__path__ = [REFERENCE_SRC]
    sys.modules["gradoom"] = parent
    scenario = importlib.import_module("gradoom.scenario")
    engine = importlib.import_module("gradoom.engine")
    return engine, scenario


def actor_tables(smap, seed: int) -> dict:
    """Seeded patch-id and animation tables for every kind of actor, plus map items and player starts
    (``scenario.py:346-378``); the ids only need to name existing patches."""

    rng = np.random.default_rng(seed)
    patches = len(smap.sprite_widths)
    ids = lambda *shape: rng.integers(0, patches, shape).astype(np.int32)  # noqa: E731
    death_frames = 6
    death_counts = rng.integers(3, death_frames + 1, 6).astype(np.int32)
    xdeath_counts = rng.integers(3, death_frames + 1, 6).astype(np.int32)
    durations = lambda counts: np.where(np.arange(death_frames)[None, :] < counts[:, None], rng.integers(3, 9, (6, death_frames)), 0).astype(np.int32)  # noqa: E731
    death_durations, xdeath_durations = durations(death_counts), durations(xdeath_counts)
    sectors = rng.permutation(len(smap.sector_quads))
    centre = lambda s, du, dv: (1 - du) * (1 - dv) * smap.sector_quads[s][0] + du * (1 - dv) * smap.sector_quads[s][1] + (1 - du) * dv * smap.sector_quads[s][2] + du * dv * smap.sector_quads[s][3]  # noqa: E731
    starts = [(*np.round(centre(int(s), 0.5, 0.5)), float(rng.integers(0, 8) * 45)) for s in sectors[:4]]
    item_count = 24
    item_kinds = rng.choice(np.array([2011, 2012, 2014, 2015, 2018, 2019, 2007, 2048, 2001, 2002]), item_count)
    spots = [(*np.round(centre(int(sectors[k % len(sectors)]), rng.uniform(0.2, 0.8), rng.uniform(0.2, 0.8))), 0.0) for k in range(item_count)]
    return dict(
        enemy_walk_sprite_ids=ids(6, 4, 8), enemy_attack_sprite_ids=ids(6, 3, 8), enemy_pain_sprite_ids=ids(6, 8),
        enemy_death_sprite_ids=ids(6, death_frames), enemy_death_frame_counts=death_counts, enemy_death_frame_durations=death_durations,
        enemy_xdeath_sprite_ids=ids(6, death_frames), enemy_xdeath_frame_counts=xdeath_counts, enemy_xdeath_frame_durations=xdeath_durations,
        raw_projectile_flight_sprite_ids=ids(3, 2, 8), raw_projectile_explosion_sprite_ids=ids(3, 5),
        raw_teleport_fog_sprite_ids=ids(12), raw_bullet_puff_sprite_ids=ids(4), raw_static_sprite_ids=ids(32),
        raw_item_animation_sprite_ids=ids(8),
        player_starts=np.asarray(starts, dtype=np.float32), item_spawns=np.asarray(spots, dtype=np.float32),
        item_types=item_kinds.astype(np.int32),
    )


def to_compiled_scenario(smap, *, flash_lights: bool = False, overlays: dict | None = None, actors: int = 0):
    """Wrap a SynthMap in the reference's CompiledScenario (``scenario.py:302-401``)."""

    _engine, scenario = load_reference()
    wall_count = len(smap.wall_segments)
    sprite_count = len(smap.sprite_widths)
    # enemy types 0..5 x 4 walk frames x 8 rotations address up to 192 patches
    # (engine.py:14073); drops use raw_static_sprite_ids[12] (engine.py:14657-14660).
    enemy_walk = (np.arange(6 * 4 * 8, dtype=np.int32) % sprite_count).reshape(6, 4, 8)
    raw_static = (np.arange(32, dtype=np.int32) * 5 + 3) % sprite_count
    kwargs = {}
    if flash_lights:
        lights = np.zeros((8, 2, 52), dtype=np.int64)
        lights[:, :, 1] = 1
        lights[:, :, 2] = 2
        kwargs["native_weapon_flash_lights"] = lights
    if smap.projectile_additive_luts is not None:
        # styled sprites: blend tables and the patches of the effects that use them (scenario.py:361-369)
        kwargs.update(
            projectile_additive_luts=smap.projectile_additive_luts, sprite_translucent_lut=smap.sprite_translucent_lut,
            raw_projectile_flight_sprite_ids=((np.arange(3 * 2 * 8, dtype=np.int32) * 7 + 1) % sprite_count).reshape(3, 2, 8),
            raw_teleport_fog_sprite_ids=(np.arange(12, dtype=np.int32) * 3 + 2) % sprite_count,
            raw_bullet_puff_sprite_ids=(np.arange(4, dtype=np.int32) * 11 + 5) % sprite_count,
        )
    if overlays is not None:
        # raw psprite and status bar patches (scenario.py:382-397)
        kwargs.update(
            native_weapon_patch_atlas=overlays["weapon_atlas"], native_weapon_patch_opaque=overlays["weapon_opaque"].astype(bool),
            native_weapon_patch_widths=overlays["weapon_w"], native_weapon_patch_heights=overlays["weapon_h"],
            native_weapon_patch_left_offsets=overlays["weapon_left"], native_weapon_patch_top_offsets=overlays["weapon_top"],
            native_weapon_frame_ids=overlays["weapon_frame_ids"], native_weapon_flash_ids=overlays["weapon_flash_ids"],
            native_weapon_flash_lights=overlays["weapon_flash_lights"],
            hud_patch_names=tuple(f"H{i}" for i in range(len(overlays["hud_w"]))),
            hud_patch_atlas=overlays["hud_atlas"], hud_patch_opaque=overlays["hud_opaque"].astype(bool),
            hud_patch_widths=overlays["hud_w"], hud_patch_heights=overlays["hud_h"],
            hud_patch_left_offsets=overlays["hud_left"], hud_patch_top_offsets=overlays["hud_top"],
        )
        if overlays.get("decal_atlas") is not None:
            kwargs.update(
                bullet_decal_atlas=overlays["decal_atlas"], bullet_decal_heights=overlays["decal_h"],
                bullet_decal_left_offsets=overlays["decal_left"], bullet_decal_top_offsets=overlays["decal_top"],
                bullet_decal_opacity_lut=overlays["decal_opacity_lut"], bullet_decal_black_lut=overlays["decal_black_lut"],
            )
    fields = dict(
        player_starts=np.asarray([(float(smap.vertices[0, 0]), float(smap.vertices[0, 1]), 0.0)], dtype=np.float32),
        item_spawns=np.empty((0, 3), dtype=np.float32),
        item_types=np.empty((0,), dtype=np.int32),
        enemy_walk_sprite_ids=enemy_walk,
        raw_static_sprite_ids=raw_static,
    )
    if actors:
        fields.update(actor_tables(smap, actors))
    fields.update(kwargs)
    return scenario.CompiledScenario(
        scenario_sha256="s" * 64,
        iwad_sha256="i" * 64,
        namespace="zdoom",
        vertices=smap.vertices,
        wall_segments=smap.wall_segments,
        blocking_segments=smap.blocking_segments.copy(),
        blocking_wall_indices=smap.blocking_wall_indices,
        wall_texture_ids=np.zeros(wall_count, dtype=np.int32),
        wall_texture_offsets=np.zeros((wall_count, 2), dtype=np.float32),
        wall_side_texture_ids=smap.wall_side_texture_ids,
        wall_side_texture_offsets=smap.wall_side_texture_offsets,
        wall_sectors=smap.wall_sectors,
        sector_edge_mask=smap.sector_edge_mask,
        sector_heights=smap.sector_heights,
        sector_lights=smap.sector_lights,
        sector_floor_texture_ids=smap.sector_floor_texture_ids,
        sector_ceiling_texture_ids=smap.sector_ceiling_texture_ids,
        playpal=smap.playpal,
        texture_names=tuple(f"T{i}" for i in range(len(smap.texture_widths))),
        texture_atlas=smap.texture_atlas,
        texture_widths=smap.texture_widths,
        texture_heights=smap.texture_heights,
        sprite_names=tuple(f"S{i}" for i in range(sprite_count)),
        sprite_atlas=smap.sprite_atlas,
        sprite_opaque=smap.sprite_opaque,
        sprite_widths=smap.sprite_widths,
        sprite_heights=smap.sprite_heights,
        sprite_left_offsets=smap.sprite_left_offsets,
        sprite_top_offsets=smap.sprite_top_offsets,
        weapon_sprite_names=tuple(f"W{i}" for i in range(8)),
        weapon_screen_values=np.zeros((8, 84, 84), dtype=np.float32),
        weapon_screen_alpha=np.zeros((8, 84, 84), dtype=np.float32),
        colormap=smap.colormap,
        wall_projection_fragments_fixed=smap.wall_projection_fragments_fixed,
        wall_projection_fragment_mask=smap.wall_projection_fragment_mask,
        **fields,
    )


def make_engine(smap, lanes: int, *, flash_lights: bool = False, overlays: dict | None = None, screen_flashes: bool = False,
                actors: int = 0):
    engine_module, _scenario = load_reference()
    compiled = to_compiled_scenario(smap, flash_lights=flash_lights, overlays=overlays, actors=actors)
    return engine_module.TorchDeathmatchEngine(
        compiled, lanes, device=torch.device("cpu"), render_screen_flashes=screen_flashes
    )


def set_poses(engine, poses) -> None:
    """Overwrite the per-lane camera like the reference's own tests do (tests/test_rendering.py:388-393)."""

    engine_module, _ = load_reference()
    bam = torch.as_tensor(poses.angle_bam, dtype=torch.int64)
    engine._angle_bam.copy_(bam)
    engine.angle.copy_(bam.to(torch.float32) * engine_module._BAM_TO_RADIANS)
    engine.x.copy_(torch.as_tensor(poses.x))
    engine.y.copy_(torch.as_tensor(poses.y))
    engine._x_fixed.copy_(torch.round(engine.x * 65536).to(torch.int64))
    engine._y_fixed.copy_(torch.round(engine.y * 65536).to(torch.int64))
    engine._pitch_bam.copy_(torch.as_tensor(poses.pitch_bam, dtype=torch.int64))
    engine.view_z.copy_(torch.as_tensor(poses.view_z))
    # flash_light = native_weapon_flash_lights[weapon, parity, cooldown] (engine.py:14949-14967)
    engine.weapon_state_cooldown.copy_(
        torch.as_tensor(poses.flash_light).to(engine.weapon_state_cooldown.dtype)
    )


def set_sprites(engine, sprites, seed: int, effects=None):
    """Place billboards through the enemy and drop slots (engine.py:14328-14343, 14657-14682).

    Slots [0, 64) of ``sprites`` go to enemy slots, [64, 128) to drop slots.  The
    patch id an enemy shows depends on its type, walk frame and viewing rotation
    (engine.py:14011-14077); this function randomises those and then asks the
    reference which patch, fullbright flag and packed order result, returning the
    packed per-lane list the renderer consumes (engine.py:14684 onward).
    """

    count = sprites.x.shape[1]
    lanes = sprites.x.shape[0]
    enemy_count = min(count, engine.enemy_slots)
    drop_count = min(max(count - enemy_count, 0), engine.enemy_slots)
    generator = torch.Generator().manual_seed(seed)
    if enemy_count:
        sl = slice(0, enemy_count)
        engine.enemy_x[:, sl] = torch.as_tensor(sprites.x[:, :enemy_count])
        engine.enemy_y[:, sl] = torch.as_tensor(sprites.y[:, :enemy_count])
        engine.enemy_z[:, sl] = torch.as_tensor(sprites.z[:, :enemy_count])
        engine.enemy_alive[:, sl] = torch.as_tensor(sprites.alive[:, :enemy_count])
        engine.enemy_type[:, sl] = torch.randint(0, 6, (lanes, enemy_count), generator=generator)
        engine.enemy_angle[:, sl] = torch.rand((lanes, enemy_count), generator=generator) * 6.25
        engine.enemy_animation_tics[:, sl] = torch.randint(
            0, 64, (lanes, enemy_count), generator=generator
        ).to(engine.enemy_animation_tics.dtype)
        # type 3 in attack phase 2/3 is a BRIGHT state (engine.py:14125-14136)
        bright = torch.as_tensor(sprites.fullbright[:, :enemy_count])
        engine.enemy_type[:, sl] = torch.where(bright, torch.full_like(engine.enemy_type[:, sl], 3), engine.enemy_type[:, sl])
        engine.enemy_attack_phase[:, sl] = torch.where(
            bright, torch.full_like(engine.enemy_attack_phase[:, sl], 3), torch.zeros_like(engine.enemy_attack_phase[:, sl])
        )
    if drop_count:
        src = slice(enemy_count, enemy_count + drop_count)
        sl = slice(0, drop_count)
        engine.drop_x[:, sl] = torch.as_tensor(sprites.x[:, src])
        engine.drop_y[:, sl] = torch.as_tensor(sprites.y[:, src])
        engine.drop_z[:, sl] = torch.as_tensor(sprites.z[:, src])
        engine.drop_type[:, sl] = torch.where(torch.as_tensor(sprites.alive[:, src]), 2001, -1)
        engine.drop_spawned[:, sl] = True
    if effects is not None:
        set_effect_sprites(engine, effects, seed + 1)
    return packed_sprites(engine)


def set_decals(engine, smap, seed: int, per_lane: int = 40):
    """Bullet chips where rays from each camera meet the nearest linedef (engine.py:1868-1885 state).

    Most chips face the camera, some sit on the far side; two share a spot so that the newer shades
    the older; slots and serials are shuffled so that paint order differs from slot order.
    """

    rng = np.random.default_rng(seed)
    lanes = engine.num_envs
    segments = smap.wall_segments.astype(np.float64)
    slots = engine.hitscan_decal_slots
    for lane in range(lanes):
        px, py, angle = float(engine.x[lane]), float(engine.y[lane]), float(engine.angle[lane])
        view_z = float(engine.view_z[lane])
        chips = []
        for _ in range(per_lane):
            theta = angle + rng.uniform(-0.7, 0.7)
            dx, dy = np.cos(theta), np.sin(theta)
            sx, sy = segments[:, 2] - segments[:, 0], segments[:, 3] - segments[:, 1]
            ox, oy = segments[:, 0] - px, segments[:, 1] - py
            den = dx * sy - dy * sx
            safe = np.where(np.abs(den) < 1e-9, 1.0, den)
            dist = (ox * sy - oy * sx) / safe
            along = (ox * dy - oy * dx) / safe
            hit = (np.abs(den) >= 1e-9) & (dist > 1.0) & (along >= 0.05) & (along <= 0.95)
            if not hit.any():
                continue
            w = int(np.argmin(np.where(hit, dist, np.inf)))
            cross = sx[w] * (py - segments[w, 1]) - sy[w] * (px - segments[w, 0])
            side = 1 if cross > 0 else 0
            if smap.wall_sectors[w, 1] < 0:
                side = 0 if rng.random() < 0.9 else 1 - side * 0  # one-sided linedefs only have side 0
            elif rng.random() < 0.15:
                side = 1 - side
            style = int(rng.integers(0, 5)) + 5 * int(rng.integers(0, 2)) + 10 * int(rng.integers(0, 2)) + 20 * side
            chips.append((w, float(along[w]), view_z + float(rng.uniform(-35.0, 45.0)), style))
        if chips:
            w, a, z, style = chips[0]
            chips.append((w, a + 0.004, z + 1.5, (style // 20) * 20 + int(rng.integers(0, 20))))
        chosen = rng.choice(slots, size=len(chips), replace=False)
        serials = rng.permutation(len(chips)) + int(rng.integers(0, 1000))
        for (w, a, z, style), slot, serial in zip(chips, chosen, serials):
            engine.hitscan_decal_wall[lane, slot] = w
            engine.hitscan_decal_along[lane, slot] = a
            engine.hitscan_decal_z[lane, slot] = z
            engine.hitscan_decal_style[lane, slot] = style
            engine.hitscan_decal_serial[lane, slot] = int(serial)


def set_actor_state(engine, smap, seed: int):
    """Randomise every kind of actor the sprite pass shows (state tensors of ``engine.py:1745-1925``)."""

    from gradoom_amd import synthmap

    generator = torch.Generator().manual_seed(seed)
    lanes = engine.num_envs

    def rand(low, high, shape, like):
        return torch.randint(low, high, shape, generator=generator).to(like.dtype)

    def place(count, offset):
        spots = synthmap.generate_sprites(smap, lanes, count, seed + offset)
        return (torch.as_tensor(v) for v in (spots.x, spots.y, spots.z, spots.alive))

    # monsters: alive, dying or absent
    n = engine.enemy_slots
    x, y, z, used = place(n, 1)
    engine.enemy_x[:], engine.enemy_y[:], engine.enemy_z[:] = x, y, z
    dying = used & (torch.rand((lanes, n), generator=generator) < 0.3)
    engine.enemy_alive[:] = used & ~dying
    engine.enemy_type[:] = rand(0, 6, (lanes, n), engine.enemy_type)
    engine.enemy_angle[:] = torch.rand((lanes, n), generator=generator) * 6.25
    engine.enemy_animation_tics[:] = rand(0, 200, (lanes, n), engine.enemy_animation_tics)
    engine.enemy_target_slot[:] = rand(-2, 4, (lanes, n), engine.enemy_target_slot)
    engine.enemy_attack_phase[:] = rand(0, 5, (lanes, n), engine.enemy_attack_phase)
    engine.enemy_cooldown[:] = rand(0, 40, (lanes, n), engine.enemy_cooldown)
    engine.enemy_pain_tics[:] = torch.where(torch.rand((lanes, n), generator=generator) < 0.2, 3, 0).to(engine.enemy_pain_tics.dtype)
    engine.enemy_death_tics[:] = torch.where(dying, 9, 0).to(engine.enemy_death_tics.dtype)
    engine.enemy_death_type[:] = rand(0, 6, (lanes, n), engine.enemy_death_type)
    engine.enemy_death_elapsed[:] = rand(0, 60, (lanes, n), engine.enemy_death_elapsed)
    engine.enemy_death_extreme[:] = torch.rand((lanes, n), generator=generator) < 0.4
    engine.player_dead[:] = torch.rand((lanes,), generator=generator) < 0.25
    # the player's projectiles: flying or exploding
    n = engine.player_projectile_slots
    x, y, z, used = place(n, 2)
    engine.projectile_x[:], engine.projectile_y[:], engine.projectile_z[:] = x, y, z
    bursting = used & (torch.rand((lanes, n), generator=generator) < 0.4)
    engine.projectile_alive[:] = used & ~bursting
    engine.projectile_type[:] = rand(0, 2, (lanes, n), engine.projectile_type)
    engine.projectile_age[:] = rand(0, 40, (lanes, n), engine.projectile_age)
    engine.projectile_velocity_x[:] = torch.rand((lanes, n), generator=generator) * 20 - 10
    engine.projectile_velocity_y[:] = torch.rand((lanes, n), generator=generator) * 20 - 10
    engine.projectile_impact_type[:] = rand(0, 2, (lanes, n), engine.projectile_impact_type)
    engine.projectile_impact_tics[:] = torch.where(bursting, rand(1, 18, (lanes, n), engine.projectile_impact_tics), 0).to(engine.projectile_impact_tics.dtype)
    # monster fireballs
    n = engine.enemy_projectile_slots
    x, y, z, used = place(n, 3)
    engine.enemy_projectile_x[:], engine.enemy_projectile_y[:], engine.enemy_projectile_z[:] = x, y, z
    bursting = used & (torch.rand((lanes, n), generator=generator) < 0.4)
    engine.enemy_projectile_alive[:] = used & ~bursting
    engine.enemy_projectile_age[:] = rand(0, 40, (lanes, n), engine.enemy_projectile_age)
    engine.enemy_projectile_velocity_x[:] = torch.rand((lanes, n), generator=generator) * 20 - 10
    engine.enemy_projectile_velocity_y[:] = torch.rand((lanes, n), generator=generator) * 20 - 10
    engine.enemy_projectile_impact_tics[:] = torch.where(bursting, rand(1, 18, (lanes, n), engine.enemy_projectile_impact_tics), 0).to(engine.enemy_projectile_impact_tics.dtype)
    # teleport fog, bullet puffs, drops
    n = engine.enemy_slots
    x, y, z, used = place(n, 4)
    engine.teleport_fog_x[:], engine.teleport_fog_y[:], engine.teleport_fog_z[:] = x, y, z
    engine.teleport_fog_tics[:] = torch.where(used, rand(1, 73, (lanes, n), engine.teleport_fog_tics), 0).to(engine.teleport_fog_tics.dtype)
    n = engine.hitscan_puff_slots
    x, y, z, used = place(n, 5)
    engine.hitscan_puff_x[:], engine.hitscan_puff_y[:], engine.hitscan_puff_z[:] = x, y, z
    engine.hitscan_puff_tics[:] = torch.where(used, rand(1, 17, (lanes, n), engine.hitscan_puff_tics), 0).to(engine.hitscan_puff_tics.dtype)
    n = engine.enemy_slots
    x, y, z, used = place(n, 6)
    engine.drop_x[:], engine.drop_y[:], engine.drop_z[:] = x, y, z
    kinds = torch.tensor((2001, 2002, 2007, 2048))[torch.randint(0, 4, (lanes, n), generator=generator)]
    engine.drop_type[:] = torch.where(used, kinds, -1)
    engine.drop_spawned[:] = torch.rand((lanes, n), generator=generator) < 0.8
    # map items
    items = len(engine.map.item_types)
    engine.item_available[:] = torch.rand((lanes, items), generator=generator) < 0.7
    engine.item_animation_initial_tics[:] = rand(1, 7, (lanes, items), engine.item_animation_initial_tics)
    engine.episode_time[:] = rand(0, 500, (lanes,), engine.episode_time)


def set_effect_sprites(engine, sprites, seed: int):
    """Place styled billboards: plasma balls and rockets in flight (additive table 0 / opaque,
    engine.py:14410-14460), teleport fog (additive table 1, engine.py:14577-14595) and bullet puffs
    (translucent, engine.py:14597-14630).  A third of ``sprites`` goes to each kind."""

    lanes, count = sprites.x.shape
    third = count // 3
    generator = torch.Generator().manual_seed(seed)
    x, y, z = (torch.as_tensor(v) for v in (sprites.x, sprites.y, sprites.z))
    alive = torch.as_tensor(sprites.alive)
    flight = slice(0, min(third, engine.player_projectile_slots))
    n = flight.stop
    engine.projectile_x[:, :n], engine.projectile_y[:, :n], engine.projectile_z[:, :n] = x[:, flight], y[:, flight], z[:, flight]
    engine.projectile_alive[:, :n] = alive[:, flight]
    engine.projectile_type[:, :n] = torch.randint(0, 2, (lanes, n), generator=generator)
    engine.projectile_age[:, :n] = torch.randint(0, 40, (lanes, n), generator=generator).to(engine.projectile_age.dtype)
    engine.projectile_velocity_x[:, :n] = torch.rand((lanes, n), generator=generator) * 20 - 10
    engine.projectile_velocity_y[:, :n] = torch.rand((lanes, n), generator=generator) * 20 - 10
    fog = slice(third, third + min(third, engine.enemy_slots))
    n = fog.stop - fog.start
    engine.teleport_fog_x[:, :n], engine.teleport_fog_y[:, :n], engine.teleport_fog_z[:, :n] = x[:, fog], y[:, fog], z[:, fog]
    tics = torch.randint(1, 73, (lanes, n), generator=generator)
    engine.teleport_fog_tics[:, :n] = torch.where(alive[:, fog], tics, torch.zeros_like(tics)).to(engine.teleport_fog_tics.dtype)
    puff = slice(2 * third, 2 * third + min(count - 2 * third, engine.hitscan_puff_slots))
    n = puff.stop - puff.start
    engine.hitscan_puff_x[:, :n], engine.hitscan_puff_y[:, :n], engine.hitscan_puff_z[:, :n] = x[:, puff], y[:, puff], z[:, puff]
    tics = torch.randint(1, 17, (lanes, n), generator=generator)
    engine.hitscan_puff_tics[:, :n] = torch.where(alive[:, puff], tics, torch.zeros_like(tics)).to(engine.hitscan_puff_tics.dtype)


def packed_sprites(engine):
    """Replay the reference's slot trimming and concatenation order (engine.py:14328-14682) for the kinds
    this driver places: enemies, player projectiles in flight, teleport fog, bullet puffs and drops."""

    engine_module, _scenario = load_reference()

    enemy_sprite = engine._native_enemy_sprite_ids()
    enemy_slots = torch.nonzero(torch.any(engine.enemy_alive, dim=0)).flatten()
    enemy_type = engine.enemy_type[:, enemy_slots].clamp(0, 5)
    fullbright = engine._native_enemy_fullbright(
        enemy_type,
        engine.enemy_attack_phase[:, enemy_slots],
        engine.enemy_cooldown[:, enemy_slots],
        engine._enemy_attack_recovery[enemy_type],
    )
    drop_visible = (engine.drop_type >= 0) & engine.drop_spawned
    static = engine.map.raw_static_sprite_ids
    drop_sprite = static[12].expand_as(engine.drop_type)
    drop_sprite = torch.where(engine.drop_type == 2007, static[6], drop_sprite)
    drop_sprite = torch.where(engine.drop_type == 2002, static[14], drop_sprite)
    drop_slots = torch.nonzero(torch.any(drop_visible, dim=0)).flatten()
    opaque = lambda like: torch.full_like(like, -1, dtype=torch.int64)  # noqa: E731
    kinds = [  # x, y, z, patch, alive, fullbright, style
        (engine.enemy_x[:, enemy_slots], engine.enemy_y[:, enemy_slots], engine.enemy_z[:, enemy_slots],
         enemy_sprite[:, enemy_slots], engine.enemy_alive[:, enemy_slots], fullbright, opaque(enemy_sprite[:, enemy_slots])),
    ]
    # player projectiles in flight (engine.py:14410-14460)
    flight_type = engine.projectile_type.clamp(0, 1)
    rotation = engine._doom_sprite_rotation(
        torch.atan2(engine.y[:, None] - engine.projectile_y, engine.x[:, None] - engine.projectile_x),
        torch.atan2(engine.projectile_velocity_y, engine.projectile_velocity_x),
    )
    flight_frame = torch.where(flight_type == 1, torch.remainder(engine.projectile_age // 6, 2).to(torch.int64), torch.zeros_like(flight_type))
    flight_sprite = engine.map.raw_projectile_flight_sprite_ids[flight_type, flight_frame, rotation]
    slots = torch.nonzero(torch.any(engine.projectile_alive, dim=0)).flatten()
    if slots.numel():
        alive = engine.projectile_alive[:, slots]
        kinds.append((engine.projectile_x[:, slots], engine.projectile_y[:, slots], engine.projectile_z[:, slots],
                      flight_sprite[:, slots], alive, alive,
                      torch.where(flight_type[:, slots] == 1, torch.zeros_like(flight_type[:, slots]), opaque(flight_type[:, slots]))))
    # teleport fog (engine.py:14577-14595)
    slots = torch.nonzero(torch.any(engine.teleport_fog_tics > 0, dim=0)).flatten()
    if slots.numel():
        tics = engine.teleport_fog_tics[:, slots]
        frame = torch.clamp((engine_module._TELEPORT_FOG_TOTAL_TICS - tics.to(torch.int64)) // 6, max=11)
        patch = engine.map.raw_teleport_fog_sprite_ids[frame]
        kinds.append((engine.teleport_fog_x[:, slots], engine.teleport_fog_y[:, slots], engine.teleport_fog_z[:, slots],
                      patch, tics > 0, tics > 0, torch.ones_like(patch, dtype=torch.int64)))
    # bullet puffs (engine.py:14597-14630)
    slots = torch.nonzero(torch.any(engine.hitscan_puff_tics > 0, dim=0)).flatten()
    if slots.numel():
        tics = engine.hitscan_puff_tics[:, slots]
        step = engine_module._BULLET_PUFF_FRAME_TICS
        frame = torch.where(tics > 3 * step, 0, torch.where(tics > 2 * step, 1, torch.where(tics > step, 2, 3))).to(torch.int64)
        patch = engine.map.raw_bullet_puff_sprite_ids[frame]
        kinds.append((engine.hitscan_puff_x[:, slots], engine.hitscan_puff_y[:, slots], engine.hitscan_puff_z[:, slots],
                      patch, tics > 0, frame == 0, torch.full_like(patch, -2, dtype=torch.int64)))
    if drop_slots.numel():
        kinds.append((engine.drop_x[:, drop_slots], engine.drop_y[:, drop_slots], engine.drop_z[:, drop_slots],
                      drop_sprite[:, drop_slots], drop_visible[:, drop_slots], torch.zeros_like(drop_visible[:, drop_slots]),
                      opaque(drop_sprite[:, drop_slots])))
    columns = [torch.cat([kind[k] for kind in kinds], dim=1) for k in range(7)]
    return dict(
        sprite_x=columns[0].numpy(), sprite_y=columns[1].numpy(), sprite_z=columns[2].numpy(),
        sprite_id=columns[3].numpy().astype(np.int32), sprite_alive=columns[4].numpy(),
        sprite_fullbright=columns[5].numpy(), sprite_style=columns[6].numpy().astype(np.int8),
    )


def set_overlay_state(engine, seed: int) -> None:
    """Randomise the gameplay tensors the weapon and status bar layers read (engine.py:14949-15267)."""

    n = engine.num_envs
    g = torch.Generator().manual_seed(seed)

    def integers(low, high, dtype):
        return torch.randint(low, high, (n,), generator=g).to(dtype)

    cooldowns = engine.map.native_weapon_frame_ids.shape[2]
    engine.selected_weapon.copy_(integers(0, engine._slot_base_weapon.shape[0], torch.int64))
    engine.selected_weapon_variant.copy_(integers(0, 2, torch.bool))
    engine.weapon_state_cooldown.copy_(integers(0, cooldowns + 1, torch.int32))
    engine.weapon_state_cooldown[::3] = 0
    engine.weapon_fire_count.copy_(integers(0, 9, torch.int32))
    engine.weapon_ready_tics.copy_(integers(0, 40, torch.int32))
    engine.weapon_raise_cooldown.copy_(integers(0, 8, torch.int32))
    engine.weapon_raise_cooldown[::2] = 0
    engine.weapon_lower_cooldown.copy_(integers(0, 20, torch.int32))
    engine.pending_weapon.copy_(torch.where(torch.rand(n, generator=g) < 0.3, integers(0, 7, torch.int64), torch.full((n,), -1)))
    engine.episode_time.copy_(integers(1, 400, torch.int32))
    engine.episode_time[0] = 3   # spawn raise still running
    engine._player_bob_fixed.copy_(integers(0, 16 * 65536, torch.int64))
    engine.health.copy_(integers(-20, 201, torch.float32) + 0.5)
    engine.health[1] = 0.0
    engine.player_dead.copy_(engine.health <= 0)
    engine.armor.copy_(integers(0, 250, torch.float32) + 0.25)
    engine.hud_ready_ammo.copy_(integers(0, 1100, torch.float32))
    engine.weapons.copy_((torch.rand((n, engine.weapons.shape[1]), generator=g) < 0.5).to(engine.weapons.dtype))
    engine.hud_ammo_counts.copy_(torch.randint(0, 400, (n, 4), generator=g).to(engine.hud_ammo_counts.dtype))
    engine.mugshot_face_index.copy_(integers(0, 3, torch.int64))
    engine.mugshot_grin_tics.copy_(torch.where(torch.rand(n, generator=g) < 0.2, integers(1, 9, torch.int32), torch.zeros(n, dtype=torch.int32)))
    engine.mugshot_pain_tics.copy_(torch.where(torch.rand(n, generator=g) < 0.4, integers(1, 9, torch.int32), torch.zeros(n, dtype=torch.int32)))
    engine.mugshot_ouch.copy_(integers(0, 2, torch.bool))
    engine.mugshot_pain_direction.copy_(integers(0, 3, torch.int64))
    engine.attack_held_tics.copy_(torch.where(torch.rand(n, generator=g) < 0.3, integers(70, 100, torch.int32), integers(0, 70, torch.int32)))


def overlay_engine_tensors(engine) -> dict:
    """The engine tensors ``overlay_inputs.weapon_state`` / ``hud_state`` take, by their argument names."""

    return dict(
        active_weapon=engine._active_weapon(), weapon_state_cooldown=engine.weapon_state_cooldown,
        weapon_fire_count=engine.weapon_fire_count, weapon_ready_tics=engine.weapon_ready_tics,
        weapon_lower_cooldown=engine.weapon_lower_cooldown, weapon_raise_cooldown=engine.weapon_raise_cooldown,
        pending_weapon=engine.pending_weapon, episode_time=engine.episode_time, player_bob_fixed=engine._player_bob_fixed,
        player_dead=engine.player_dead, weapon_ammo_slot=engine._weapon_ammo_slot, hud_ready_ammo=engine.hud_ready_ammo,
        health=engine.health, armor=engine.armor, weapons=engine.weapons, hud_ammo_counts=engine.hud_ammo_counts,
        mugshot_face_index=engine.mugshot_face_index, mugshot_grin_tics=engine.mugshot_grin_tics,
        mugshot_pain_tics=engine.mugshot_pain_tics, mugshot_ouch=engine.mugshot_ouch,
        mugshot_pain_direction=engine.mugshot_pain_direction, attack_held_tics=engine.attack_held_tics,
    )
