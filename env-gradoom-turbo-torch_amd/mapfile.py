"""Maps on disk: one ``.npz`` file holding the scenario arrays the renderer reads.

The arrays carry the field names of the reference's ``CompiledScenario``
(``/root/reference/src/gradoom/scenario.py:302-401``), after the fallbacks the engine applies when it
copies a scenario to the device (``engine.py:869-912``): ``texture_atlas`` holds palette indices
(``texture_index_atlas`` when the scenario has one), the ``sprite_*`` arrays hold the raw patches
(``raw_sprite_*`` when present).  Nothing in the file is executable: it is written with
``numpy.savez_compressed`` and read with ``allow_pickle=False``.

Schema, version 1 (``S`` sectors, ``W`` linedefs, ``T`` textures, ``P`` sprite patches):

==================================  =========  ====================  =========================================
array                               dtype      shape                 meaning
==================================  =========  ====================  =========================================
``map_schema_version``              int32      ()                    1
``vertices``                        float32    [V, 2]
``wall_segments``                   float32    [W, 4]                x1, y1, x2, y2; front sector on the right
``wall_sectors``                    int32      [W, 2]                front, back (-1: one-sided)
``wall_side_texture_ids``           int32      [W, 2, 3]             middle, bottom, top per side; -1 none
``wall_side_texture_offsets``       float32    [W, 2, 2]
``blocking_wall_indices``           int32      [B]
``sector_edge_mask``                bool       [S, W]                linedefs bounding each sector
``sector_heights``                  float32    [S, 2]                floor, ceiling
``sector_lights``                   float32    [S]
``sector_floor_texture_ids``        int32      [S]
``sector_ceiling_texture_ids``      int32      [S]
``texture_atlas``                   uint8      [T, maxH, maxW]       palette indices
``texture_widths / _heights``       int32      [T]
``playpal``                         uint8      [256, 3]
``colormap``                        uint8      [34, 256]
``sprite_atlas / sprite_opaque``    uint8      [P, maxH, maxW]
``sprite_widths / _heights``        int32      [P]
``sprite_left_offsets / _top_..``   int32      [P]
==================================  =========  ====================  =========================================

Optional: ``wall_projection_fragments_fixed`` int64 ``[W, F, 4]`` with ``wall_projection_fragment_mask`` bool
``[W, F]`` (``scenario.py:400-401``), ``projectile_additive_luts`` uint8 ``[2, 256, 256]`` and
``sprite_translucent_lut`` uint8 ``[256, 256]`` (``scenario.py:367-368``).
"""

from __future__ import annotations

import types

import numpy as np

SCHEMA_VERSION = 1

# name -> (dtype, number of dimensions, trailing shape or None)
REQUIRED = {
    "vertices": (np.float32, 2, (2,)),
    "wall_segments": (np.float32, 2, (4,)),
    "wall_sectors": (np.int32, 2, (2,)),
    "wall_side_texture_ids": (np.int32, 3, (2, 3)),
    "wall_side_texture_offsets": (np.float32, 3, (2, 2)),
    "blocking_wall_indices": (np.int32, 1, None),
    "sector_edge_mask": (np.bool_, 2, None),
    "sector_heights": (np.float32, 2, (2,)),
    "sector_lights": (np.float32, 1, None),
    "sector_floor_texture_ids": (np.int32, 1, None),
    "sector_ceiling_texture_ids": (np.int32, 1, None),
    "texture_atlas": (np.uint8, 3, None),
    "texture_widths": (np.int32, 1, None),
    "texture_heights": (np.int32, 1, None),
    "playpal": (np.uint8, 2, (256, 3)),
    "colormap": (np.uint8, 2, (34, 256)),
    "sprite_atlas": (np.uint8, 3, None),
    "sprite_opaque": (np.uint8, 3, None),
    "sprite_widths": (np.int32, 1, None),
    "sprite_heights": (np.int32, 1, None),
    "sprite_left_offsets": (np.int32, 1, None),
    "sprite_top_offsets": (np.int32, 1, None),
}
OPTIONAL = {
    "wall_projection_fragments_fixed": (np.int64, 3, (4,)),
    "wall_projection_fragment_mask": (np.bool_, 2, None),
    "projectile_additive_luts": (np.uint8, 3, (256, 256)),
    "sprite_translucent_lut": (np.uint8, 2, (256, 256)),
}


def _host(value, dtype=None):
    if value is None:
        return None
    if hasattr(value, "detach"):   # a Torch tensor, on any device
        value = value.detach().cpu().numpy()
    array = np.asarray(value)
    return array if dtype is None else array.astype(dtype, copy=False)


class ScenarioView:
    """A ``CompiledScenario`` seen through the attribute names the map-table builder reads.

    The engine draws from ``texture_index_atlas`` and the ``raw_sprite_*`` patches and falls back to
    ``texture_atlas`` / ``sprite_*`` when a scenario has none, with an identity COLORMAP when it has
    none of its own (``engine.py:869-912``); the view applies the same fallbacks.
    """

    _PLAIN = (
        "vertices", "wall_segments", "wall_sectors", "wall_side_texture_ids", "wall_side_texture_offsets",
        "blocking_wall_indices", "sector_edge_mask", "sector_heights", "sector_lights", "sector_floor_texture_ids",
        "sector_ceiling_texture_ids", "texture_widths", "texture_heights", "playpal", "wall_projection_fragments_fixed",
        "wall_projection_fragment_mask", "projectile_additive_luts", "sprite_translucent_lut",
    )
    _SPRITE = ("atlas", "opaque", "widths", "heights", "left_offsets", "top_offsets")

    def __init__(self, scenario):
        for name in self._PLAIN:
            setattr(self, name, _host(getattr(scenario, name, None)))
        index_atlas = getattr(scenario, "texture_index_atlas", None)
        self.texture_atlas = _host(scenario.texture_atlas if index_atlas is None else index_atlas)
        colormap = getattr(scenario, "colormap", None)
        self.colormap = np.broadcast_to(np.arange(256, dtype=np.uint8), (34, 256)).copy() if colormap is None else _host(colormap)
        for field in self._SPRITE:
            raw = getattr(scenario, f"raw_sprite_{field}", None)
            setattr(self, f"sprite_{field}", _host(getattr(scenario, f"sprite_{field}") if raw is None else raw))
        for name in ("vertices", "wall_segments", "wall_sectors", "sector_heights", "texture_atlas", "playpal"):
            if getattr(self, name) is None:
                raise ValueError(f"scenario has no {name}")

    @property
    def blocking_segments(self):
        return self.wall_segments[self.blocking_wall_indices]


def _checked(name: str, value, spec) -> np.ndarray:
    dtype, ndim, trailing = spec
    array = np.asarray(value)
    if array.ndim != ndim or (trailing is not None and tuple(array.shape[ndim - len(trailing):]) != tuple(trailing)):
        wanted = "x".join(["?"] * (ndim - len(trailing or ())) + [str(n) for n in (trailing or ())])
        raise ValueError(f"{name} must have shape [{wanted}], not {list(array.shape)}")
    converted = array.astype(dtype)
    if np.issubdtype(dtype, np.integer) and not np.array_equal(converted, array):
        raise ValueError(f"{name} does not fit {np.dtype(dtype).name}")
    return np.ascontiguousarray(converted)


def _check_consistency(arrays: dict) -> None:
    walls, sectors = len(arrays["wall_segments"]), len(arrays["sector_heights"])
    for name in ("wall_sectors", "wall_side_texture_ids", "wall_side_texture_offsets"):
        if len(arrays[name]) != walls:
            raise ValueError(f"{name} must hold one row per linedef ({walls})")
    for name in ("sector_lights", "sector_floor_texture_ids", "sector_ceiling_texture_ids"):
        if len(arrays[name]) != sectors:
            raise ValueError(f"{name} must hold one value per sector ({sectors})")
    if arrays["sector_edge_mask"].shape != (sectors, walls):
        raise ValueError(f"sector_edge_mask must have shape [{sectors}, {walls}]")
    textures, patches = len(arrays["texture_atlas"]), len(arrays["sprite_atlas"])
    for name in ("texture_widths", "texture_heights"):
        if len(arrays[name]) != textures:
            raise ValueError(f"{name} must hold one value per texture ({textures})")
    if arrays["sprite_opaque"].shape != arrays["sprite_atlas"].shape:
        raise ValueError("sprite_opaque must have the shape of sprite_atlas")
    for name in ("sprite_widths", "sprite_heights", "sprite_left_offsets", "sprite_top_offsets"):
        if len(arrays[name]) != patches:
            raise ValueError(f"{name} must hold one value per sprite patch ({patches})")
    fragments, mask = arrays.get("wall_projection_fragments_fixed"), arrays.get("wall_projection_fragment_mask")
    if (fragments is None) != (mask is None):
        raise ValueError("wall_projection_fragments_fixed and wall_projection_fragment_mask come together")
    if fragments is not None and (fragments.shape[:2] != mask.shape or len(fragments) != walls):
        raise ValueError("projection fragments must have shape [W, F, 4] and their mask [W, F]")


def scenario_arrays(scenario) -> dict[str, np.ndarray]:
    """The schema's arrays from a ``CompiledScenario``-like object (or a ``SynthMap``), checked and converted."""

    view = ScenarioView(scenario)
    arrays = {}
    for name, spec in REQUIRED.items():
        value = getattr(view, name, None)
        if value is None:
            raise ValueError(f"scenario has no {name}")
        arrays[name] = _checked(name, value, spec)
    for name, spec in OPTIONAL.items():
        value = getattr(view, name, None)
        if value is not None:
            arrays[name] = _checked(name, value, spec)
    _check_consistency(arrays)
    return arrays


def save_map(path: str, scenario) -> None:
    """Write ``scenario`` (``CompiledScenario`` field names) as a version-1 map file."""

    arrays = scenario_arrays(scenario)
    with open(path, "wb") as handle:
        np.savez_compressed(handle, map_schema_version=np.int32(SCHEMA_VERSION), **arrays)


def load_map(path: str):
    """Read a map file into an object ``mapbuild.build_map_tables`` / ``HipRenderer`` take.

    Raises ``ValueError`` for a missing array, a wrong dtype or shape, or another schema version.
    """

    with np.load(path, allow_pickle=False) as stored:
        if "map_schema_version" not in stored.files:
            raise ValueError(f"{path} is not a map file (no map_schema_version)")
        version = int(stored["map_schema_version"])
        if version != SCHEMA_VERSION:
            raise ValueError(f"{path} has map schema version {version}; this package reads version {SCHEMA_VERSION}")
        arrays = {}
        for name, spec in REQUIRED.items():
            if name not in stored.files:
                raise ValueError(f"{path} lacks {name}")
            if stored[name].dtype != np.dtype(spec[0]):
                raise ValueError(f"{name} must be stored as {np.dtype(spec[0]).name}, not {stored[name].dtype.name}")
            arrays[name] = _checked(name, stored[name], spec)
        for name, spec in OPTIONAL.items():
            if name in stored.files:
                if stored[name].dtype != np.dtype(spec[0]):
                    raise ValueError(f"{name} must be stored as {np.dtype(spec[0]).name}, not {stored[name].dtype.name}")
                arrays[name] = _checked(name, stored[name], spec)
    _check_consistency(arrays)
    loaded = types.SimpleNamespace(**{name: arrays.get(name) for name in list(REQUIRED) + list(OPTIONAL)})
    loaded.blocking_segments = loaded.wall_segments[loaded.blocking_wall_indices]
    return loaded
