"""Map digest shared by the fixture writer and the tests (no reference import here)."""

from __future__ import annotations

import hashlib

import numpy as np

DIGEST_FIELDS = (
    "wall_segments", "wall_sectors", "wall_side_texture_ids", "wall_side_texture_offsets", "sector_heights",
    "sector_lights", "sector_floor_texture_ids", "sector_ceiling_texture_ids", "texture_atlas", "playpal",
    "colormap", "sprite_atlas", "sprite_widths", "sprite_heights",
)


def map_digest(smap) -> str:
    digest = hashlib.sha256()
    for name in DIGEST_FIELDS:
        digest.update(np.ascontiguousarray(getattr(smap, name)).tobytes())
    return digest.hexdigest()


def fragment_digest(smap) -> str:
    digest = hashlib.sha256()
    digest.update(np.ascontiguousarray(smap.wall_projection_fragments_fixed, dtype=np.int64).tobytes())
    digest.update(np.ascontiguousarray(smap.wall_projection_fragment_mask, dtype=np.uint8).tobytes())
    return digest.hexdigest()
