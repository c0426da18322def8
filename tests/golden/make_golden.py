"""Write golden vectors from the reference's own Torch CPU render path (build container only).

Usage:  python tests/golden/make_golden.py [--only NAME ...] [--time]

For each case below a seeded synthetic map and pose set is built with
``synthmap``, rendered by the reference (``/root/reference/src/gradoom/engine.py``,
imported through ``refdrive``), and the inputs + outputs are stored as
``tests/golden/fixtures/<name>.npz``:

* lane inputs exactly as ``gd_lanes_desc`` wants them (including the Torch
  float32 ray tables and sprite depths, so nothing on the GPU box needs the
  reference or a particular Torch CPU build);
* ``indexed``  uint8 [N,240,320]  ``_render_native_indexed_frame(include_hud=True)`` (engine.py:15338)
* ``obs``      uint8 [N,84,84]    ``render_reference_frame()`` CPU float path (engine.py:15436)
* for ``stages`` cases, lane 0 intermediates of every pipeline stage
  (geometry, intersections, PrepWall, flats, depth / sprite-clip buffers).

The map itself is regenerated from its seed at test time; ``map_sha256`` guards
against generator drift.
"""

from __future__ import annotations

import argparse
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))

import __graft_entry__ as entry  # noqa: E402

entry.load_package()
from gradoom_amd import hostmath, overlay_inputs, synthmap  # noqa: E402

import refdrive  # noqa: E402
from make_golden_meta import fragment_digest, map_digest  # noqa: E402

FIXTURES = os.path.join(HERE, "fixtures")

# name -> generator arguments. Every case is a distinct (map seed, pose seed).
CASES = {
    "tiny_stages": dict(map_seed=7, grid=(4, 3), sectors=10, linedefs=48, lanes=4, pose_seed=1, stages=True),
    "small_pitch": dict(map_seed=11, grid=(4, 3), sectors=10, linedefs=60, lanes=8, pose_seed=1, pitch=True),
    "small_flash": dict(map_seed=12, grid=(5, 4), sectors=17, linedefs=100, lanes=8, pose_seed=1, flash=True),
    "small_midtex_sprites": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=8, pose_seed=1, sprites=128, flash=True,
        pitch=True, midtex=0.2, stages=True,
    ),
    "config1": dict(map_seed=1001, grid=(9, 6), sectors=48, linedefs=320, lanes=16, pose_seed=1),
    "config1_pitch_flash": dict(
        map_seed=1001, grid=(9, 6), sectors=48, linedefs=320, lanes=8, pose_seed=2, pitch=True, flash=True
    ),
    "config1_midtex": dict(map_seed=2001, grid=(9, 6), sectors=48, linedefs=320, lanes=8, pose_seed=3, midtex=0.2),
    "brick_islands": dict(
        map_seed=61, grid=(5, 4), sectors=18, linedefs=170, lanes=8, pose_seed=1, layout="brick", islands=6, midtex=0.2
    ),
    "grid_islands_sprites": dict(
        map_seed=62, grid=(6, 5), sectors=26, linedefs=200, lanes=8, pose_seed=1, islands=10, pitch=True, flash=True,
        sprites=32,
    ),
    "brick_islands_320": dict(
        map_seed=63, grid=(8, 6), sectors=44, linedefs=360, lanes=12, pose_seed=2, layout="brick", islands=16, midtex=0.15
    ),
    # weapon psprite + muzzle flash over the view and the status bar in rows 208..239, from seeded
    # synthetic patches (synthmap.generate_overlays) and randomised gameplay tensors
    "overlays": dict(
        map_seed=12, grid=(5, 4), sectors=17, linedefs=100, lanes=12, pose_seed=4, pitch=True, sprites=16, overlays=71
    ),
    # Single-column events found by searching seeded maps and poses with the oracle's rule counters: the
    # equal-depth solid replacement, the solid bridge, the sector bridge and the tied-strip rule fire on
    # the picked (pose seed, lane) pairs; the other lanes are close-to-wall poses of the same maps.
    "rare_rules_brick26": dict(
        map_seed=3001, grid=(6, 5), sectors=26, linedefs=260, lanes=6, layout="brick", islands=10, midtex=0.1,
        picks=[(1, 14), (5, 1), (8, 8), (1, 0), (5, 0), (8, 0)], pose_seed=1,
    ),
    "rare_rules_brick18": dict(
        map_seed=3023, grid=(5, 4), sectors=18, linedefs=170, lanes=4, layout="brick", islands=6, midtex=0.1,
        picks=[(3, 10), (3, 0), (3, 1), (3, 2)], pose_seed=3,
    ),
    "grazing_brick26": dict(
        map_seed=3001, grid=(6, 5), sectors=26, linedefs=260, lanes=8, layout="brick", islands=10, midtex=0.1,
        picks=[(1, 10), (3, 1), (1, 0), (1, 1), (1, 2), (3, 0), (3, 2), (3, 3)], margin=0.02, pose_seed=1, pitch=True,
    ),
    # Two void pillars touching at a corner put four same-sector one-sided linedefs on one vertex: the
    # reference drops its direct endpoint-neighbour tables and searches the neighbour slots instead.
    "pinched_pillars": dict(
        map_seed=41, grid=(4, 3), sectors=10, linedefs=120, lanes=8, pose_seed=1, islands=2, pillars=4, midtex=0.1,
        pitch=True, flash=True, stages=True,
    ),
    # A fifth of the linedefs carry two or three BSP projection fragments (scenario.py:420-454): OWallMost and
    # the wallscan light then work from the fragment that owns the column.
    "split_linedefs": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=8, pose_seed=2, sprites=32, pitch=True, flash=True,
        midtex=0.2, split_seed=5, stages=True,
    ),
    "split_linedefs_grazing": dict(
        map_seed=3001, grid=(6, 5), sectors=26, linedefs=260, lanes=6, layout="brick", islands=10, midtex=0.1,
        pose_seed=7, margin=0.02, split_seed=9,
    ),
    # Styled billboards among opaque ones: plasma balls (additive table 0), teleport fog (additive table 1) and
    # bullet puffs (translucent table) blend over whatever lies under them through seeded random tables.
    "styled_sprites": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=8, pose_seed=3, sprites=48, effects=60, blend_seed=13,
        pitch=True, flash=True, midtex=0.2,
    ),
    # render_screen_flashes: PLAYPAL mixed with gold (pickups) and red (damage) per lane before the RGB24 frame
    # and the observation (engine.py:15381-15398)
    "screen_flashes": dict(
        map_seed=12, grid=(5, 4), sectors=17, linedefs=100, lanes=4, pose_seed=6, sprites=16, screen_flashes=29
    ),
    # Bullet chip decals on the linedefs the cameras look at (engine.py:13747-13991), under sprites, the weapon
    # and the status bar; the reference's scene depth buffer and its picture right after the decal pass ride along.
    "decals": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=8, pose_seed=5, sprites=24, pitch=True, flash=True,
        midtex=0.2, overlays=83, decals=17,
    ),
    # Every kind of actor the sprite pass shows (monsters in all their states, start dolls, corpses, projectiles and
    # explosions of both sides, teleport fog, bullet puffs, animated map items, drops) from randomised gameplay
    # tensors; the list the renderer gets is actor_inputs.pack_actors(engine), 556 fixed slots per lane.
    "actors": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=8, pose_seed=7, pitch=True, flash=True, midtex=0.1,
        blend_seed=19, actors=31,
    ),
    # Inputs beyond the generator's defaults (heights in multiples of 8, 64x128 wall textures, eyes 41 above the floor):
    # heights uniform over whole map units with ceilings 64..256 above their floors, so that neighbours may miss each
    # other vertically altogether and every sector is a plane level of its own;
    "uniform_heights": dict(
        map_seed=1001, grid=(9, 6), sectors=48, linedefs=320, lanes=10, pose_seed=4, pitch=True, flash=True, sprites=24,
        midtex=0.15, variant=dict(seed=5, heights="uniform"), eye="any",
    ),
    # the same on a map with more plane levels than any table of the renderer holds (96 sectors)
    "uniform_heights_96": dict(
        map_seed=1002, grid=(12, 9), sectors=96, linedefs=800, lanes=6, pose_seed=3, sprites=16, midtex=0.1,
        variant=dict(seed=6, heights="uniform"), eye="any",
    ),
    # closed doors (ceiling at the floor) and crawl spaces 8..24 units high among ordinary rooms
    "doors": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=12, pose_seed=8, pitch=True, flash=True, sprites=24,
        midtex=0.2, variant=dict(seed=7, heights="doors"),
    ),
    "doors_brick": dict(
        map_seed=3001, grid=(6, 5), sectors=26, linedefs=260, lanes=10, pose_seed=9, layout="brick", islands=10, midtex=0.1,
        variant=dict(seed=8, heights="doors"), margin=0.05, eye="any",
    ),
    # wall textures of every power-of-two size from 8 to 256 either way, flats 64 or 128 rows
    "mixed_textures": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=10, pose_seed=10, pitch=True, midtex=0.2,
        variant=dict(seed=9, textures="mixed"), eye="any",
    ),
    # and sizes that are no powers of two, as WAD textures have (24, 72, 96, 100, 136, 160, 200)
    "npot_textures": dict(
        map_seed=22, grid=(6, 5), sectors=26, linedefs=160, lanes=10, pose_seed=11, pitch=True, flash=True, midtex=0.25,
        sprites=8, variant=dict(seed=10, textures="npot"),
    ),
    # config1's cameras again after every sector light changed: what gd_renderer_set_sector_lights must produce
    "config1_relit": dict(map_seed=1001, grid=(9, 6), sectors=48, linedefs=320, lanes=16, pose_seed=1, variant=dict(seed=11, lights=True)),
    "config2_subset": dict(map_seed=1002, grid=(12, 9), sectors=96, linedefs=800, lanes=4, pose_seed=1, sprites=32),
    "config3_subset": dict(
        map_seed=1003, grid=(15, 15), sectors=200, linedefs=2000, lanes=2, pose_seed=1, sprites=64, flash=True
    ),
    "config4_subset": dict(
        map_seed=1004, grid=(21, 21), sectors=400, linedefs=4000, lanes=2, pose_seed=1, sprites=128, midtex=0.15
    ),
    # the headline map with the benchmark's height distribution (floors U{0..255}, ceilings U{64..256} above: a plane
    # level per sector, about 750 in all), the variant seed bench.py and the full-size GPU tests use
    "config4_uniform_subset": dict(
        map_seed=1004, grid=(21, 21), sectors=400, linedefs=4000, lanes=2, pose_seed=2, sprites=128, midtex=0.15, flash=True,
        variant=dict(seed=5, heights="uniform"),
    ),
    # Sectors with the ceiling BELOW the floor, which no map of the reference holds: three seeds of the random-map tests
    # (tests/random_cases.py), each the first found to show one way such a sector differs from an ordinary one.  Seen from a
    # neighbour its wall tiers share rows (the four-column group's shade applies once either tier's common bottom is passed);
    "inverted_shared_tier_rows": dict(recipe=dict(seed=70017, inverted=True, variants=False), lanes=16),
    # seen from inside, the ceiling's and the floor's plane rows overlap;
    "inverted_plane_rows_overlap": dict(recipe=dict(seed=80127, inverted=True, variants=True, eye_any=True), lanes=16),
    # behind a window that a zero-height sector closed, its ceiling clip passes the floor clip and the silhouette over the
    # rows between decides whether a billboard behind shows.
    "inverted_clip_past_window": dict(recipe=dict(seed=503259, mixed=True, variants=True, eye_any=True), lanes=16),
    # An 80-sector corridor seen end on: up to 85 linedefs in one column ray, more than a column of the HIP path keeps in
    # its own list (the reference's dense loops have no list to overflow).
    "corridor_80": dict(recipe=dict(kind="corridor", sectors=80), lanes=6),
    # Cameras in the void beside the map: hardly a pixel that a wall pass claims, most flat rays unresolved.
    "cameras_outside": dict(recipe=dict(kind="outside"), lanes=8),
    # Seed 50078 of the random-map tests, lanes 7 and 14: a column loses its sector, picks a linedef beyond a projected solid
    # and takes that path's clips, which close the window over rows that no drawseg painted or claimed.
    "portal_path_clip_closes_window": dict(recipe=dict(seed=50078), lanes=16),
    # Billboards in awkward places: at the eye, a step from it, on vertices and linedefs, far outside the map, lifted or
    # sunk.  No two at exactly the same depth: among those the reference's order is torch.topk's, which is not defined.
    "awkward_billboards": dict(recipe=dict(kind="awkward_billboards", seed=1200007, ties=False), lanes=16),
    # Seed 7045 of reference_sweep.py's layers kind: a bullet chip on a wall eight units from the eye whose texel row
    # boundary falls on a screen row, (y - top) / vertical_scale a rounding step from a whole number in lane 3.  The
    # reference's `96.0 / distance` is a Python number over a tensor, which Torch evaluates as reciprocal(distance) * 96.
    "decal_row_on_a_rounding_step": dict(recipe=dict(seed=7045, mixed=True, variants=True, eye_any=True, inverted=False), lanes=8,
                                         overlays=46, decals=62, effects=24),
}


def build_case(name: str, cfg: dict, do_time: bool) -> dict:
    recipe_parts = None
    if cfg.get("recipe"):
        # map, poses and billboards as tests/random_cases.py builds them (heights edited by hand, maybe a variant, split
        # linedefs or blend tables on top); the billboards' patches are then whatever the reference's actors show
        import random_cases

        recipe_parts = random_cases.build_parts(cfg["recipe"], cfg["lanes"])
        smap = recipe_parts[0]
        cfg = dict(cfg, flash=True, sectors=len(smap.sector_heights), linedefs=len(smap.wall_segments))
    else:
        smap = synthmap.generate_map(
            cfg["map_seed"], grid=cfg["grid"], sectors=cfg["sectors"], linedefs=cfg["linedefs"], midtex=cfg.get("midtex", 0.0),
            layout=cfg.get("layout", "grid"), islands=cfg.get("islands", 0), pillars=cfg.get("pillars", 0),
        )
    base_digest = map_digest(smap)
    if cfg.get("variant"):
        smap = synthmap.with_variant(smap, **cfg["variant"])
    if cfg.get("split_seed"):
        smap = synthmap.split_linedefs(smap, cfg["split_seed"])
    if cfg.get("blend_seed"):
        smap = synthmap.with_blend_tables(smap, cfg["blend_seed"])
    lanes = cfg["lanes"]
    started = time.time()
    overlays = synthmap.generate_overlays(cfg["overlays"]) if cfg.get("overlays") else None
    engine = refdrive.make_engine(
        smap, lanes, flash_lights=cfg.get("flash", False), overlays=overlays, screen_flashes=bool(cfg.get("screen_flashes")),
        actors=cfg.get("actors", 0),
    )
    ctor_seconds = time.time() - started
    if recipe_parts is not None:
        poses = recipe_parts[1]
    else:
        picks = cfg.get("picks") or [(cfg["pose_seed"], lane) for lane in range(lanes)]
        assert len(picks) == lanes
        poses = synthmap.generate_picked_poses(
            smap, picks, pitch=cfg.get("pitch", False), flash=cfg.get("flash", False), margin=cfg.get("margin", 0.15),
            eye=cfg.get("eye", "standing"),
        )
    refdrive.set_poses(engine, poses)
    offsets = hostmath.native_ray_offsets("cpu")
    assert torch.equal(offsets, engine._native_ray_offsets)
    ray_cos, ray_sin = hostmath.ray_tables(engine.angle, offsets)
    data = dict(
        x=engine.x.numpy().copy(), y=engine.y.numpy().copy(), angle=engine.angle.numpy().copy(),
        view_z=engine.view_z.numpy().copy(), x_fixed=engine._x_fixed.numpy().copy(),
        y_fixed=engine._y_fixed.numpy().copy(), angle_bam=engine._angle_bam.numpy().copy(),
        pitch_bam=engine._pitch_bam.numpy().copy(), flash_light=np.asarray(poses.flash_light, dtype=np.int64),
        ray_cos=ray_cos.numpy(), ray_sin=ray_sin.numpy(),
        cosine_correction=hostmath.cosine_correction("cpu").numpy(),
    )
    if cfg.get("actors"):
        # every kind of actor from randomised gameplay tensors, packed at full width by actor_inputs.pack_actors
        from gradoom_amd import actor_inputs

        refdrive.set_actor_state(engine, smap, cfg["actors"])
        packed = {key: value.numpy() for key, value in actor_inputs.pack_actors(engine).items()}
        data.update(packed)
        # the tensors the packing read, so that it can be re-run without the reference
        for field in actor_inputs.ENGINE_FIELDS:
            data[f"actor_engine_{field}"] = getattr(engine, field).numpy().copy()
        for field in actor_inputs.MAP_FIELDS:
            data[f"actor_map_{field}"] = getattr(engine.map, field).numpy().copy()
        data["sprite_depth"] = hostmath.sprite_depth(
            engine.x, engine.y, engine.angle, torch.as_tensor(packed["sprite_x"]), torch.as_tensor(packed["sprite_y"])
        ).numpy()
    if recipe_parts is not None and not cfg.get("actors"):
        effects = synthmap.generate_sprites(smap, lanes, cfg["effects"], cfg["recipe"].get("seed", 1) + 50) if cfg.get("effects") else None
        packed = refdrive.set_sprites(engine, recipe_parts[2], cfg["recipe"].get("seed", 1), effects)
        data.update(packed)
        data["sprite_depth"] = hostmath.sprite_depth(
            engine.x, engine.y, engine.angle, torch.as_tensor(packed["sprite_x"]), torch.as_tensor(packed["sprite_y"])
        ).numpy()
    elif cfg.get("sprites", 0):
        sprites = synthmap.generate_sprites(smap, lanes, cfg["sprites"], cfg["pose_seed"])
        effects = synthmap.generate_sprites(smap, lanes, cfg["effects"], cfg["pose_seed"] + 50) if cfg.get("effects") else None
        packed = refdrive.set_sprites(engine, sprites, cfg["pose_seed"], effects)
        data.update(packed)
        data["sprite_depth"] = hostmath.sprite_depth(
            engine.x, engine.y, engine.angle, torch.as_tensor(packed["sprite_x"]), torch.as_tensor(packed["sprite_y"])
        ).numpy()
    if overlays is not None:
        refdrive.set_overlay_state(engine, cfg["overlays"])
        tensors = refdrive.overlay_engine_tensors(engine)
        weapon_arguments = (
            "active_weapon", "weapon_state_cooldown", "weapon_fire_count", "weapon_ready_tics", "weapon_lower_cooldown",
            "weapon_raise_cooldown", "pending_weapon", "episode_time", "player_bob_fixed", "player_dead",
        )
        hud_arguments = (
            "active_weapon", "weapon_ammo_slot", "hud_ready_ammo", "health", "armor", "weapons", "hud_ammo_counts",
            "mugshot_face_index", "mugshot_grin_tics", "mugshot_pain_tics", "mugshot_ouch", "mugshot_pain_direction",
            "attack_held_tics",
        )
        data["weapon_state"] = overlay_inputs.weapon_state(
            **{k: tensors[k] for k in weapon_arguments}, weapon_frame_ids=torch.as_tensor(overlays["weapon_frame_ids"]),
            weapon_flash_ids=torch.as_tensor(overlays["weapon_flash_ids"]), fine_sine=torch.as_tensor(overlay_inputs.fine_sine_fixed()),
        ).numpy()
        data["hud_state"] = overlay_inputs.hud_state(**{k: tensors[k] for k in hud_arguments}).numpy()
        # the muzzle flash lights the scene: extralight of engine.py:14949-14967
        data["flash_light"] = engine._native_weapon_frame_selection()[2].numpy().astype(np.int64)
        assert np.array_equal(overlay_inputs.fine_sine_fixed(), engine._fine_sine_fixed.numpy())
        for key, value in tensors.items():
            data[f"engine_{key}"] = value.numpy().copy()
        # the reference's own per-lane selections, to pin overlay_inputs independently of the frames
        frame_id, flash_id, _light = engine._native_weapon_frame_selection()
        data["ref_weapon_frame_id"] = frame_id.numpy().astype(np.int64)
        data["ref_weapon_flash_id"] = flash_id.numpy().astype(np.int64)
        # the observation of an environment made with obs_crop=None: the status bar is pooled, not masked
        # (env.py:441, engine.py:15440)
        engine.mask_hud = False
        with torch.no_grad():
            data["obs_with_hud"] = engine.render_reference_frame().numpy()
        engine.mask_hud = True
        data["ref_face_patch"] = np.asarray(
            [engine._native_mugshot_patch_index(lane, int(engine.health[lane].clamp(0, 999).item())) for lane in range(lanes)],
            dtype=np.int64,
        )
    if cfg.get("decals"):
        refdrive.set_decals(engine, smap, cfg["decals"])
        packed_decals = overlay_inputs.decal_inputs(
            engine.hitscan_decal_serial, engine.hitscan_decal_wall, engine.hitscan_decal_along, engine.hitscan_decal_z,
            engine.hitscan_decal_style, engine.map.portal_walls, overlay_inputs.fine_sine_fixed(),
        )
        data["decal_state"], data["decal_geom"] = (value.numpy() for value in packed_decals)
        with torch.no_grad():
            background = engine._render_native_background()
            data["ref_scene_depth"] = background[1].numpy()
            data["ref_decal_frame"] = engine._native_render_hitscan_decals(background[0], engine.view_z, background[1]).numpy()
            data["ref_background_frame"] = background[0].numpy()
    if cfg.get("screen_flashes"):
        # pickup and damage counters as gameplay leaves them; lane 0 keeps both at zero (blend = identity)
        generator = torch.Generator().manual_seed(cfg["screen_flashes"])
        engine.bonus_count[:] = torch.randint(0, 24, (lanes,), generator=generator).to(engine.bonus_count.dtype)
        engine.damage_count[:] = torch.randint(0, 130, (lanes,), generator=generator).to(engine.damage_count.dtype)
        engine.bonus_count[0] = 0
        engine.damage_count[0] = 0
        engine.damage_count[1] = 0
        data["screen_blend"] = overlay_inputs.screen_blend(engine.bonus_count, engine.damage_count, engine._damage_to_alpha).numpy()
        with torch.no_grad():
            data["rgb_all"] = engine.render_native_frame(include_hud=True).numpy()
    started = time.time()
    with torch.no_grad():
        indexed = engine._render_native_indexed_frame(include_hud=True)
        obs = engine.render_reference_frame()
        rgb_lane0 = engine.render_native_frame(include_hud=True)[0]
    render_seconds = time.time() - started
    data["indexed"] = indexed.numpy()
    data["obs"] = obs.numpy()
    data["rgb_lane0"] = rgb_lane0.numpy()
    if cfg.get("stages", False):
        with torch.no_grad():
            geometry = engine._native_wall_projection_geometry()
            inter = engine._native_portal_intersections(geometry)
            hoff, vstep = engine._native_wall_texture_mapping()
            sector = engine._current_sector()
            flats, surface, scene_surface = engine._native_render_flats(sector, engine.view_z)
            walls, scene_depth, clip_depth, clip_wall = engine._native_render_portal_walls(
                flats, engine.view_z, surface, scene_surface
            )
        data.update(
            st_sector=sector.numpy().astype(np.int32),
            st_geometry=torch.stack(geometry, dim=-1)[0].numpy(),
            st_distances=inter[0][0].numpy(), st_along=inter[1][0].numpy(), st_geometric=inter[2][0].numpy(),
            st_projected=inter[3][0].numpy(), st_left_edge=inter[4][0].numpy(), st_visibility=inter[5][0].numpy(),
            st_hoff=hoff[0].numpy(), st_vstep=vstep[0].numpy(), st_flats=flats[0].numpy(),
            st_surface_depth=surface[0].numpy(), st_scene_surface_depth=scene_surface[0].numpy(),
            st_walls=walls[0].numpy(), st_scene_depth=scene_depth[0].numpy(), st_clip_depth=clip_depth[0].numpy(),
            st_clip_wall=clip_wall[0].numpy().astype(np.int32),
        )
        # derived map tables (engine.py:721-849, 1527-1634)
        dmap = engine.map
        data.update(
            ref_wall_lengths=dmap.portal_wall_lengths.numpy(),
            ref_endpoint_neighbors=dmap.portal_endpoint_neighbors.numpy(),
            ref_endpoint_neighbor_starts=dmap.portal_endpoint_neighbor_starts.numpy(),
            ref_endpoint_neighbor_ends=dmap.portal_endpoint_neighbor_ends.numpy(),
            ref_solid_bridge_start_indices=dmap.portal_endpoint_solid_bridge_start_indices.numpy(),
            ref_solid_bridge_start_mask=dmap.portal_endpoint_solid_bridge_start_mask.numpy(),
            ref_solid_bridge_end_indices=dmap.portal_endpoint_solid_bridge_end_indices.numpy(),
            ref_solid_bridge_end_mask=dmap.portal_endpoint_solid_bridge_end_mask.numpy(),
            ref_direct_neighbors=np.asarray(engine._native_direct_endpoint_neighbors is not None),
            ref_same_pair=engine._native_same_portal_sector_pairs.numpy(),
            ref_opposing=engine._native_opposing_portal_pairs.numpy(),
            ref_portal_bridge_index=engine._native_projected_portal_bridge_indices.numpy(),
            ref_portal_bridge_mask=engine._native_projected_portal_bridge_mask.numpy(),
            ref_sector_bridge_index=engine._native_projected_sector_bridge_indices.numpy(),
            ref_sector_bridge_mask=engine._native_projected_sector_bridge_mask.numpy(),
            ref_walls_fixed=torch.round(dmap.portal_walls * 65536).to(torch.int64).numpy(),
            ref_blocking_wall_indices=engine._native_blocking_wall_indices.numpy(),
            ref_sector_lights=dmap.sector_lights.numpy(),
        )
    timing = None
    if do_time:
        # The CPU-baseline protocol: full indexed frame + observation + stack update per lane.
        torch.set_num_threads(os.cpu_count())
        samples = []
        for _ in range(3):
            started = time.time()
            with torch.no_grad():
                engine._finish_observation(engine.render_reference_frame())
            samples.append(lanes / (time.time() - started))
        timing = float(np.median(samples))
    meta = dict(cfg)
    meta["map_sha256"] = base_digest
    if cfg.get("variant"):
        meta["variant_sha256"] = map_digest(smap)
    if cfg.get("split_seed"):
        meta["fragment_sha256"] = fragment_digest(smap)
    data["meta"] = np.asarray(repr(meta))
    print(
        f"{name}: W={cfg['linedefs']} S={cfg['sectors']} lanes={lanes} ctor {ctor_seconds:.1f}s render {render_seconds:.1f}s"
        + (f" reference CPU {timing:.3f} lane-frames/s on {os.cpu_count()} cores" if timing else ""),
        flush=True,
    )
    return data


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--only", nargs="*", default=None)
    parser.add_argument("--time", action="store_true")
    args = parser.parse_args()
    os.makedirs(FIXTURES, exist_ok=True)
    for name, cfg in CASES.items():
        if args.only and name not in args.only:
            continue
        data = build_case(name, cfg, args.time)
        np.savez_compressed(os.path.join(FIXTURES, f"{name}.npz"), **data)


if __name__ == "__main__":
    main()
