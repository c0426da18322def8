"""ctypes mirror of ``include/gradoom_amd.h`` (struct layouts and field order must match)."""

from __future__ import annotations

import ctypes as C

import numpy as np

SCREEN_WIDTH = 320
VIEW_HEIGHT = 208
SCREEN_HEIGHT = 240
OBS_SIZE = 84
FRAME_STACK = 4

STACK_STEP = 0
STACK_RESET = 1
LAYOUT_CHW = 0
LAYOUT_HWC = 1

GD_OK = 0
STATIC_SCRATCH_MIB = 64  # gd_render_static: the fixed per-GPU working memory
STATIC_MAX_LANES = 65536
GD_E_ARG = -1
GD_E_HIP = -2
GD_E_UNSUPPORTED = -3

ABI_VERSION = 4  # GD_ABI_VERSION

_P = C.c_void_p


class _Sized(C.Structure):
    """A descriptor whose first field carries its own size (checked by every entry point)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.struct_size = C.sizeof(self)


MAP_SCALARS = (
    "wall_count",
    "sector_count",
    "vertex_count",
    "texture_count",
    "tex_max_h",
    "tex_max_w",
    "sprite_count",
    "spr_max_h",
    "spr_max_w",
    "blocking_count",
    "neighbor_slots",
    "direct_neighbors",
    "floor_level_count",
    "ceil_level_count",
    "grid_nx",
    "grid_ny",
    "fine_nx",
    "fine_ny",
    "fragment_slots",
    "split_count",
)
MAP_FLOATS = ("grid_min_x", "grid_min_y", "grid_cell", "fine_cell")

# (field, numpy dtype) in header order
MAP_ARRAYS = (
    ("walls", np.float32),
    ("walls_fixed", np.int32),
    ("wall_sectors", np.int32),
    ("wall_vertex", np.int32),
    ("side_tex", np.int32),
    ("side_off", np.float32),
    ("wall_len", np.float32),
    ("endpoint_neighbors", np.int32),
    ("endpoint_neighbor_starts", np.uint8),
    ("endpoint_neighbor_ends", np.uint8),
    ("direct_neighbor_table", np.int32),
    ("solid_bridge_start_ofs", np.int32),
    ("solid_bridge_start_idx", np.int32),
    ("solid_bridge_end_ofs", np.int32),
    ("solid_bridge_end_idx", np.int32),
    ("vertex_wall_ofs", np.int32),
    ("vertex_wall_idx", np.int32),
    ("sector_wall_ofs", np.int32),
    ("sector_wall_idx", np.int32),
    ("sector_edge_ofs", np.int32),
    ("sector_edge_idx", np.int32),
    ("blocking_walls", np.int32),
    ("wall_split_slot", np.int32),
    ("split_fragments_fixed", np.int32),
    ("split_fragment_mask", np.uint8),
    ("grid_cell_ofs", np.int32),
    ("grid_item_sector", np.int32),
    ("grid_item_edge_ofs", np.int32),
    ("grid_item_edges", np.int32),
    ("fine_sector", np.uint32),
    ("floor_levels", np.float32),
    ("ceil_levels", np.float32),
    ("sector_heights", np.float32),
    ("sector_lights", np.float32),
    ("sector_floor_tex", np.int32),
    ("sector_ceil_tex", np.int32),
    ("tex_atlas", np.uint8),
    ("tex_w", np.int32),
    ("tex_h", np.int32),
    ("playpal", np.uint8),
    ("colormap", np.uint8),
    ("spr_atlas", np.uint8),
    ("spr_opaque", np.uint8),
    ("spr_post_top", np.uint8),
    ("spr_w", np.int32),
    ("spr_h", np.int32),
    ("spr_left", np.int32),
    ("spr_top", np.int32),
    ("additive_luts", np.uint8),
    ("translucent_lut", np.uint8),
)

LANE_ARRAYS = (
    ("x", np.float32),
    ("y", np.float32),
    ("angle", np.float32),
    ("view_z", np.float32),
    ("x_fixed", np.int64),
    ("y_fixed", np.int64),
    ("angle_bam", np.int64),
    ("pitch_bam", np.int64),
    ("flash_light", np.int64),
    ("ray_cos", np.float32),
    ("ray_sin", np.float32),
    ("sprite_x", np.float32),
    ("sprite_y", np.float32),
    ("sprite_z", np.float32),
    ("sprite_depth", np.float32),
    ("sprite_id", np.int32),
    ("sprite_alive", np.uint8),
    ("sprite_fullbright", np.uint8),
    ("weapon_state", np.int64),
    ("hud_state", np.int32),
    ("decal_state", np.int32),
    ("decal_geom", np.float32),
    ("screen_blend", np.float32),
    ("sprite_style", np.int8),
)

OUT_FIELDS = ("indexed", "obs", "frames", "reset_mask", "rgb", "final_frames")


class MapDesc(_Sized):
    _fields_ = (
        [("struct_size", C.c_uint32)]
        + [(name, C.c_int32) for name in MAP_SCALARS]
        + [(name, C.c_float) for name in MAP_FLOATS]
        + [(name, _P) for name, _ in MAP_ARRAYS]
    )


class LanesDesc(_Sized):
    _fields_ = [("struct_size", C.c_uint32), ("lane_count", C.c_int32), ("sprite_slots", C.c_int32), ("decal_slots", C.c_int32)] + [
        (name, _P) for name, _ in LANE_ARRAYS
    ]


OVERLAY_SCALARS = ("weapon_patch_count", "weapon_max_h", "weapon_max_w", "hud_patch_count", "hud_max_h", "hud_max_w")
OVERLAY_ARRAYS = (
    ("weapon_atlas", np.uint8),
    ("weapon_opaque", np.uint8),
    ("weapon_w", np.int32),
    ("weapon_h", np.int32),
    ("weapon_left", np.int32),
    ("weapon_top", np.int32),
    ("hud_atlas", np.uint8),
    ("hud_opaque", np.uint8),
    ("hud_w", np.int32),
    ("hud_h", np.int32),
    ("hud_left", np.int32),
    ("hud_top", np.int32),
)


DECAL_SCALARS = ("decal_variant_count", "decal_max_h", "decal_max_w", "decal_black_rows")
DECAL_ARRAYS = (
    ("decal_atlas", np.uint8),
    ("decal_h", np.int32),
    ("decal_left", np.int32),
    ("decal_top", np.int32),
    ("decal_opacity_lut", np.uint8),
    ("decal_black_lut", np.uint8),
)


class OverlayDesc(_Sized):
    _fields_ = (
        [("struct_size", C.c_uint32)]
        + [(name, C.c_int32) for name in OVERLAY_SCALARS] + [(name, _P) for name, _ in OVERLAY_ARRAYS]
        + [(name, C.c_int32) for name in DECAL_SCALARS] + [(name, _P) for name, _ in DECAL_ARRAYS]
    )


def host_overlay_desc(overlays: dict) -> tuple[OverlayDesc, list]:
    """OverlayDesc of HOST pointers from a dict of arrays named like ``gd_overlay_desc``'s fields.

    ``weapon_atlas`` / ``hud_atlas`` are ``[patches, max_h, max_w]``; counts and sizes come from them.
    """

    desc = OverlayDesc()
    keep = []
    for prefix in ("weapon", "hud"):
        atlas = np.ascontiguousarray(overlays[f"{prefix}_atlas"], dtype=np.uint8)
        if atlas.ndim != 3:
            raise ValueError(f"{prefix}_atlas must be [patches, height, width]")
        setattr(desc, f"{prefix}_patch_count", atlas.shape[0])
        setattr(desc, f"{prefix}_max_h", atlas.shape[1])
        setattr(desc, f"{prefix}_max_w", atlas.shape[2])
        if np.asarray(overlays[f"{prefix}_opaque"]).shape != atlas.shape:
            raise ValueError(f"{prefix}_opaque must have the shape of {prefix}_atlas")
        for field in ("w", "h", "left", "top"):
            if np.asarray(overlays[f"{prefix}_{field}"]).shape != (atlas.shape[0],):
                raise ValueError(f"{prefix}_{field} must hold one value per patch")
    for name, dtype in OVERLAY_ARRAYS:
        array = np.ascontiguousarray(overlays[name], dtype=dtype)
        keep.append(array)
        setattr(desc, name, array.ctypes.data)
    if overlays.get("decal_atlas") is not None:
        atlas = np.ascontiguousarray(overlays["decal_atlas"], dtype=np.uint8)
        if atlas.ndim != 3 or atlas.shape[0] != 5:
            raise ValueError("decal_atlas must be [5, height, width]")
        black = np.ascontiguousarray(overlays["decal_black_lut"], dtype=np.uint8)
        if np.asarray(overlays["decal_opacity_lut"]).shape != (32, 256) or black.ndim != 2 or black.shape[1] != 256:
            raise ValueError("decal_opacity_lut must be [32,256] and decal_black_lut [rows,256]")
        desc.decal_variant_count, desc.decal_max_h, desc.decal_max_w = atlas.shape
        desc.decal_black_rows = black.shape[0]
        for name, dtype in DECAL_ARRAYS:
            array = np.ascontiguousarray(overlays[name], dtype=dtype)
            if name in ("decal_h", "decal_left", "decal_top") and array.shape != (5,):
                raise ValueError(f"{name} must hold one value per variant")
            keep.append(array)
            setattr(desc, name, array.ctypes.data)
    return desc, keep


class FrameOut(_Sized):
    _fields_ = [("struct_size", C.c_uint32)] + [(name, _P) for name in OUT_FIELDS] + [
        ("stack_mode", C.c_int32), ("obs_source_rows", C.c_int32), ("final_frames_layout", C.c_int32)]


def host_map_desc(tables: dict) -> tuple[MapDesc, list]:
    """Build a MapDesc of HOST pointers from ``mapbuild.build_map_tables`` output.

    Returns the struct and the list of arrays that must stay alive while it is used.
    """

    desc = MapDesc()
    keep = []
    for name in MAP_SCALARS:
        setattr(desc, name, int(tables[name]))
    for name in MAP_FLOATS:
        setattr(desc, name, float(tables[name]))
    for name, dtype in MAP_ARRAYS:
        array = np.ascontiguousarray(tables[name], dtype=dtype)
        keep.append(array)
        setattr(desc, name, array.ctypes.data)
    return desc, keep


ACTOR_SCALARS = (
    "lane_count",
    "enemy_slots",
    "doll_count",
    "player_projectile_slots",
    "enemy_projectile_slots",
    "fog_slots",
    "puff_slots",
    "item_count",
    "drop_slots",
    "attack_frames",
    "death_frames",
    "xdeath_frames",
    "explosion_frames",
)
ACTOR_ARRAYS = (
    ("enemy_x", np.float32),
    ("enemy_y", np.float32),
    ("enemy_z", np.float32),
    ("enemy_alive", np.uint8),
    ("enemy_type", np.int64),
    ("enemy_rotation", np.uint8),
    ("enemy_animation_tics", np.int32),
    ("enemy_target_slot", np.int64),
    ("enemy_attack_phase", np.int32),
    ("enemy_cooldown", np.int32),
    ("enemy_pain_tics", np.int32),
    ("enemy_death_tics", np.int32),
    ("enemy_death_type", np.int64),
    ("enemy_death_elapsed", np.int32),
    ("enemy_death_extreme", np.uint8),
    ("doll_x", np.float32),
    ("doll_y", np.float32),
    ("doll_z", np.float32),
    ("doll_rotation", np.uint8),
    ("player_dead", np.uint8),
    ("projectile_x", np.float32),
    ("projectile_y", np.float32),
    ("projectile_z", np.float32),
    ("projectile_alive", np.uint8),
    ("projectile_type", np.int64),
    ("projectile_age", np.int32),
    ("projectile_rotation", np.uint8),
    ("projectile_impact_type", np.int64),
    ("projectile_impact_tics", np.int32),
    ("enemy_projectile_x", np.float32),
    ("enemy_projectile_y", np.float32),
    ("enemy_projectile_z", np.float32),
    ("enemy_projectile_alive", np.uint8),
    ("enemy_projectile_age", np.int32),
    ("enemy_projectile_rotation", np.uint8),
    ("enemy_projectile_impact_tics", np.int32),
    ("teleport_fog_x", np.float32),
    ("teleport_fog_y", np.float32),
    ("teleport_fog_z", np.float32),
    ("teleport_fog_tics", np.int32),
    ("hitscan_puff_x", np.float32),
    ("hitscan_puff_y", np.float32),
    ("hitscan_puff_z", np.float32),
    ("hitscan_puff_tics", np.int32),
    ("item_x", np.float32),
    ("item_y", np.float32),
    ("item_z", np.float32),
    ("item_types", np.int64),
    ("item_raw_visual_types", np.int64),
    ("item_available", np.uint8),
    ("item_animation_initial_tics", np.int32),
    ("episode_time", np.int32),
    ("drop_x", np.float32),
    ("drop_y", np.float32),
    ("drop_z", np.float32),
    ("drop_type", np.int64),
    ("drop_spawned", np.uint8),
    ("enemy_walk_frame_tics", np.int32),
    ("enemy_idle_frame_tics", np.int32),
    ("enemy_attack_recovery", np.int32),
    ("enemy_walk_sprite_ids", np.int64),
    ("enemy_attack_sprite_ids", np.int64),
    ("enemy_pain_sprite_ids", np.int64),
    ("enemy_death_sprite_ids", np.int64),
    ("enemy_death_frame_durations", np.int64),
    ("enemy_death_frame_counts", np.int64),
    ("enemy_xdeath_sprite_ids", np.int64),
    ("enemy_xdeath_frame_durations", np.int64),
    ("enemy_xdeath_frame_counts", np.int64),
    ("projectile_explosion_total_tics", np.int64),
    ("projectile_explosion_frame_durations", np.int64),
    ("projectile_explosion_frame_counts", np.int64),
    ("raw_projectile_explosion_sprite_ids", np.int64),
    ("raw_projectile_flight_sprite_ids", np.int64),
    ("raw_teleport_fog_sprite_ids", np.int64),
    ("raw_bullet_puff_sprite_ids", np.int64),
    ("raw_static_sprite_ids", np.int64),
    ("raw_item_animation_sprite_ids", np.int64),
)
ACTOR_OUTPUTS = (
    ("sprite_x", np.float32),
    ("sprite_y", np.float32),
    ("sprite_z", np.float32),
    ("sprite_id", np.int32),
    ("sprite_alive", np.uint8),
    ("sprite_fullbright", np.uint8),
    ("sprite_style", np.int8),
)


class ActorDesc(_Sized):
    _fields_ = (
        [("struct_size", C.c_uint32)]
        + [(name, C.c_int32) for name in ACTOR_SCALARS] + [(name, _P) for name, _ in ACTOR_ARRAYS]
        + [(name, _P) for name, _ in ACTOR_OUTPUTS]
    )


WEAPON_INPUTS = (
    "active_weapon", "weapon_state_cooldown", "weapon_fire_count", "weapon_ready_tics", "weapon_lower_cooldown",
    "weapon_raise_cooldown", "pending_weapon", "episode_time", "player_bob_fixed", "player_dead",
)
WEAPON_TABLES = ("weapon_frame_ids", "weapon_flash_ids", "weapon_flash_lights", "fine_sine")


class WeaponDesc(_Sized):
    """``gd_weapon_desc``: the gameplay tensors ``gd_pack_weapon`` reads and the two tensors it writes."""

    _fields_ = (
        [("struct_size", C.c_uint32), ("lane_count", C.c_int32), ("cooldown_slots", C.c_int32)]
        + [(name, _P) for name in WEAPON_INPUTS + WEAPON_TABLES]
        + [("weapon_state", _P), ("flash_light", _P)]
    )
