"""ctypes front end of the CPU oracle (test infrastructure only).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)
import __graft_entry__ as _entry  # noqa: E402

_entry.load_package()
from gradoom_amd import _abi  # noqa: E402

_LIB = None


class Debug(C.Structure):
    _fields_ = [("debug_lane", C.c_int32)] + [
        (name, C.c_void_p)
        for name in (
            "flats_frame",
            "surface_depth",
            "scene_surface_depth",
            "distances",
            "along",
            "geometric",
            "projected",
            "left_edge",
            "geometry",
            "horizontal_offset",
            "vertical_step",
            "visibility",
            "scene_depth",
            "sprite_clip_depth",
            "sprite_clip_wall",
            "sector",
            "walls_frame",
        )
    ]


def library():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "_build", "liboracle.so")
        sources = [os.path.join(_HERE, "gd_oracle.cpp"), os.path.join(_ROOT, "include", "gradoom_amd.h")]
        if not os.path.exists(path) or any(os.path.getmtime(src) > os.path.getmtime(path) for src in sources):
            subprocess.run(["make", "-C", _HERE, "-s"], check=True)
        lib = C.CDLL(path)
        lib.gdo_render.restype = C.c_int
        lib.gdo_observe.restype = C.c_int
        lib.gdo_last_error.restype = C.c_char_p
        _LIB = lib
    return _LIB


_OVERLAY_KEEP = None


def set_overlays(overlays: dict | None) -> None:
    """Weapon and status bar patches for later ``render`` calls (``None`` removes them)."""

    global _OVERLAY_KEEP
    lib = library()
    if overlays is None:
        lib.gdo_set_overlays(None)
        _OVERLAY_KEEP = None
        return
    desc, keep = _abi.host_overlay_desc(overlays)
    lib.gdo_set_overlays(C.byref(desc))
    _OVERLAY_KEEP = (desc, keep)


def fine_tables():
    sine = np.zeros(8192, dtype=np.int64)
    tangent = np.zeros(4096, dtype=np.int64)
    library().gdo_fine_tables(sine.ctypes.data_as(C.c_void_p), tangent.ctypes.data_as(C.c_void_p))
    return sine, tangent


def lanes_desc(lanes: dict):
    """``lanes``: numpy arrays keyed by the fields of gd_lanes_desc (sprites optional)."""

    desc = _abi.LanesDesc()
    keep = []
    count = len(lanes["x"])
    desc.lane_count = count
    sprite_x = lanes.get("sprite_x")
    desc.sprite_slots = 0 if sprite_x is None else int(np.asarray(sprite_x).shape[1])
    decal_state = lanes.get("decal_state")
    desc.decal_slots = 0 if decal_state is None else int(np.asarray(decal_state).shape[1])
    for name, dtype in _abi.LANE_ARRAYS:
        value = lanes.get(name)
        if value is None:
            setattr(desc, name, None)
            continue
        array = np.ascontiguousarray(value, dtype=dtype)
        keep.append(array)
        setattr(desc, name, array.ctypes.data)
    return desc, keep


def render(tables: dict, lanes: dict, cosine_correction, *, lane_range=None, frames=None, reset_mask=None,
           want_rgb=False, debug_lane=None, stack_mode=0, obs_source_rows=208):
    """Render lanes on the CPU. Returns dict(indexed, obs, frames, rgb, debug...)."""

    lib = library()
    map_desc, keep_map = _abi.host_map_desc(tables)
    lane_desc, keep_lanes = lanes_desc(lanes)
    count = lane_desc.lane_count
    begin, end = (0, count) if lane_range is None else lane_range
    indexed = np.zeros((count, 240, 320), dtype=np.uint8)
    obs = np.zeros((count, 84, 84), dtype=np.uint8)
    out = _abi.FrameOut()
    out.indexed = indexed.ctypes.data
    out.obs = obs.ctypes.data
    out.stack_mode = int(stack_mode)
    out.obs_source_rows = int(obs_source_rows)
    result = {"indexed": indexed, "obs": obs}
    if frames is not None:
        frames = np.ascontiguousarray(frames, dtype=np.uint8).copy()
        out.frames = frames.ctypes.data
        result["frames"] = frames
    mask = None
    if reset_mask is not None:
        mask = np.ascontiguousarray(reset_mask, dtype=np.uint8)
        out.reset_mask = mask.ctypes.data
    if want_rgb:
        rgb = np.zeros((count, 240, 320, 3), dtype=np.uint8)
        out.rgb = rgb.ctypes.data
        result["rgb"] = rgb
    correction = np.ascontiguousarray(cosine_correction, dtype=np.float32)
    debug = Debug()
    debug.debug_lane = -1
    sector = np.zeros(count, dtype=np.int32)
    debug.sector = sector.ctypes.data
    result["sector"] = sector
    if debug_lane is not None:
        walls = int(tables["wall_count"])
        debug.debug_lane = int(debug_lane)
        taps = {
            "flats_frame": np.zeros((208, 320), np.uint8),
            "surface_depth": np.zeros((208, 320), np.float32),
            "scene_surface_depth": np.zeros((208, 320), np.float32),
            "distances": np.zeros((320, walls), np.float32),
            "along": np.zeros((320, walls), np.float32),
            "geometric": np.zeros((320, walls), np.uint8),
            "projected": np.zeros((320, walls), np.uint8),
            "left_edge": np.zeros((320, walls), np.uint8),
            "geometry": np.zeros((walls, 4), np.int64),
            "horizontal_offset": np.zeros((320, walls), np.int64),
            "vertical_step": np.zeros((320, walls), np.int64),
            "visibility": np.zeros((320, walls, 2), np.int64),
            "scene_depth": np.zeros((208, 320), np.float32),
            "sprite_clip_depth": np.zeros((208, 320), np.float32),
            "sprite_clip_wall": np.zeros((208, 320), np.int32),
            "walls_frame": np.zeros((208, 320), np.uint8),
        }
        for name, array in taps.items():
            setattr(debug, name, array.ctypes.data)
        result["debug"] = taps
    code = lib.gdo_render(
        C.byref(map_desc), C.byref(lane_desc), C.byref(out), C.c_int32(begin), C.c_int32(end),
        correction.ctypes.data_as(C.c_void_p), C.byref(debug),
    )
    if code != 0:
        raise RuntimeError(f"oracle render failed ({code}): {lib.gdo_last_error().decode()}")
    del keep_map, keep_lanes, mask
    return result


def render_parallel(tables: dict, lanes: dict, cosine_correction, threads: int) -> dict:
    """``render`` (frame and observation only) with the lanes dealt out to ``threads`` host threads."""

    lib = library()
    lib.gdo_render_parallel.restype = C.c_int
    map_desc, keep_map = _abi.host_map_desc(tables)
    lane_desc, keep_lanes = lanes_desc(lanes)
    count = lane_desc.lane_count
    indexed = np.zeros((count, 240, 320), dtype=np.uint8)
    obs = np.zeros((count, 84, 84), dtype=np.uint8)
    frames = np.zeros((count, 4, 84, 84), dtype=np.uint8)
    out = _abi.FrameOut()
    out.indexed, out.obs, out.frames = indexed.ctypes.data, obs.ctypes.data, frames.ctypes.data
    correction = np.ascontiguousarray(cosine_correction, dtype=np.float32)
    code = lib.gdo_render_parallel(
        C.byref(map_desc), C.byref(lane_desc), C.byref(out), C.c_int32(0), C.c_int32(count),
        correction.ctypes.data_as(C.c_void_p), C.c_int32(threads),
    )
    if code != 0:
        raise RuntimeError(f"oracle render failed ({code}): {lib.gdo_last_error().decode()}")
    del keep_map, keep_lanes
    return {"indexed": indexed, "obs": obs, "frames": frames}


def observe(indexed, playpal, *, frames=None, reset_mask=None, stack_mode=0):
    lib = library()
    indexed = np.ascontiguousarray(indexed, dtype=np.uint8)
    count, rows, _ = indexed.shape
    playpal = np.ascontiguousarray(playpal, dtype=np.uint8)
    obs = np.zeros((count, 84, 84), dtype=np.uint8)
    frames_ptr = None
    if frames is not None:
        frames = np.ascontiguousarray(frames, dtype=np.uint8).copy()
        frames_ptr = frames.ctypes.data_as(C.c_void_p)
    mask_ptr = None
    if reset_mask is not None:
        reset_mask = np.ascontiguousarray(reset_mask, dtype=np.uint8)
        mask_ptr = reset_mask.ctypes.data_as(C.c_void_p)
    code = lib.gdo_observe(
        indexed.ctypes.data_as(C.c_void_p), C.c_int32(rows), playpal.ctypes.data_as(C.c_void_p), C.c_int32(count),
        obs.ctypes.data_as(C.c_void_p), frames_ptr, mask_ptr, C.c_int32(stack_mode),
    )
    if code != 0:
        raise RuntimeError(f"oracle observe failed ({code})")
    return obs, frames


def relation_tables(tables: dict) -> dict:
    """Dense [W,W] / [2,W,W] relation tables from the oracle's on-the-fly functions (small maps only)."""

    lib = library()
    map_desc, keep = _abi.host_map_desc(tables)
    walls = int(tables["wall_count"])
    out = dict(
        same_pair=np.zeros((walls, walls), np.uint8), opposing=np.zeros((walls, walls), np.uint8),
        portal_bridge_index=np.zeros((2, walls, walls), np.int64), portal_bridge_mask=np.zeros((2, walls, walls), np.uint8),
        sector_bridge_index=np.zeros((2, walls, walls), np.int64), sector_bridge_mask=np.zeros((2, walls, walls), np.uint8),
    )
    lib.gdo_relation_tables.restype = None
    lib.gdo_relation_tables(
        C.byref(map_desc), *(out[name].ctypes.data_as(C.c_void_p) for name in (
            "same_pair", "opposing", "portal_bridge_index", "portal_bridge_mask", "sector_bridge_index", "sector_bridge_mask")),
    )
    del keep
    return out


COVERAGE_NAMES = (
    "passes", "valid", "equal_depth_solid", "projected_solid", "solid_bridge", "endpoint_owner", "near_projected",
    "topological_owner", "sector_bridge", "opposing_boundary", "excluded_right_edge", "continues_owner_boundary",
    "forward_bridge", "completes_endpoint_bridge", "endpoint_only_portal", "tied_strip", "enters_other", "enters_shared",
    "geometric_path", "portal_bridge", "completes_portal_bridge", "ps_keeps_path", "no_keeps_path", "bottom_tail",
    "masked_column", "masked_extends", "dead_column_revived",
)


def coverage(reset: bool = False) -> dict:
    """How often each ownership rule of the wall traversal fired since the last reset."""

    values = (C.c_longlong * len(COVERAGE_NAMES))()
    count = library().gdo_coverage(values, len(COVERAGE_NAMES), int(reset))
    assert count == len(COVERAGE_NAMES)
    return {name: int(values[i]) for i, name in enumerate(COVERAGE_NAMES)}
