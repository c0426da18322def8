"""Seeded random small maps with hand-edited sector heights, shared by the random-map GPU tests, the fixture loader and
the script that writes the reference's golden vectors for some of them (``tests/golden/make_golden.py``)."""

from __future__ import annotations

import numpy as np

SHAPES = (
    ("grid", (4, 3), 10, 60, 0, 0), ("grid", (5, 4), 17, 140, 4, 2), ("brick", (5, 4), 18, 170, 6, 0),
    ("brick", (4, 3), 10, 90, 3, 2), ("grid", (6, 5), 26, 240, 10, 0), ("brick", (6, 5), 26, 260, 10, 3),
    ("grid", (3, 3), 8, 80, 2, 1), ("brick", (3, 3), 8, 100, 2, 0),
)


def closed_door_parts(seed: int, lanes: int, *, inverted: bool = False, variants: bool = True, eye_any: bool = False, mixed: bool = False):
    """A random map of one of SHAPES plus hand-closed doors and crawl spaces on up to four sectors (``inverted``: ceilings
    16 units below their floors instead; ``mixed``: each of the four one of the three kinds), then (``variants``: seven
    times in ten) other heights, texture sizes and lights over the whole map; ``eye_any``: six times in ten the eyes
    stand at any height, not between their sector's floor and ceiling.  Returns (map, poses, sprites, sprite styles)."""
    from gradoom_amd import synthmap

    rng = np.random.default_rng(seed)
    layout, grid, sectors, linedefs, islands, pillars = SHAPES[seed % len(SHAPES)]
    smap = synthmap.generate_map(seed, grid=grid, sectors=sectors, linedefs=linedefs, layout=layout, islands=islands, pillars=pillars,
                                 midtex=float(rng.choice([0.0, 0.1, 0.3])))
    if rng.random() < 0.7:
        heights = np.array(smap.sector_heights, copy=True)
        for sector in rng.choice(len(heights), size=min(4, len(heights)), replace=False):
            kind = int(rng.choice([0, 2]))
            if mixed:
                kind = int(rng.integers(0, 3))
            if inverted or kind == 1:
                heights[sector, 1] = heights[sector, 0] - 16   # a ceiling below its floor
            elif kind == 0:
                heights[sector, 1] = heights[sector, 0]        # a closed door
            else:
                heights[sector, 0] = heights[sector, 1] - 8    # a crawl space
        smap.sector_heights[...] = heights
    if variants and rng.random() < 0.7:
        smap = synthmap.with_variant(smap, seed + 9, heights=[None, "uniform", "doors"][int(rng.integers(0, 3))],
                                     textures=[None, "mixed", "npot"][int(rng.integers(0, 3))], lights=bool(rng.random() < 0.5))
    if rng.random() < 0.4:
        smap = synthmap.split_linedefs(smap, seed + 1)
    if rng.random() < 0.5:
        smap = synthmap.with_blend_tables(smap, seed + 2)
    margin = float(rng.choice([0.005, 0.02, 0.15]))
    eye = {"eye": "any"} if eye_any and rng.random() < 0.6 else {}
    poses = synthmap.generate_poses(smap, lanes, seed + 3, pitch=bool(rng.random() < 0.6), flash=bool(rng.random() < 0.5), margin=margin, **eye)
    if rng.random() < 0.3:
        poses.pitch_bam[:] = rng.integers(-30, 31, lanes) * (182 << 16)
    sprites = synthmap.generate_sprites(smap, lanes, 24, seed + 4)
    styles = rng.choice(np.array([-1, -1, -1, -2, 0, 1], dtype=np.int8), size=sprites.x.shape)
    return smap, poses, sprites, styles


def closed_door_case(seed: int, lanes: int, **options):
    """closed_door_parts as (map, derived tables, lane arrays with styled billboards)."""
    from gradoom_amd import mapbuild
    from gradoom_amd.selfcheck import make_lane_arrays

    smap, poses, sprites, styles = closed_door_parts(seed, lanes, **options)
    arrays = make_lane_arrays(smap, poses, sprites)
    arrays["sprite_style"] = styles
    return smap, mapbuild.build_map_tables(smap), arrays


def corridor_parts(lanes: int, sectors: int = 80):
    """A corridor of `sectors` sectors and cameras in it that look along it, so that every divider lands in the same
    screen columns: more linedefs per column ray than the 64 a column keeps in its own slots.  (map, poses, sprites)"""
    from gradoom_amd import synthmap

    smap = synthmap.generate_map(5, grid=(sectors, 1), sectors=sectors, linedefs=3 * sectors + 1, midtex=0.2)
    poses = synthmap.generate_poses(smap, lanes, 11, pitch=True, flash=True)
    rng = np.random.default_rng(3)
    for lane in range(lanes):
        sector = int(rng.integers(0, 8)) if lane % 2 == 0 else int(rng.integers(sectors - 8, sectors))   # either end, looking at the other
        centre = smap.sector_quads[sector].mean(axis=0)
        poses.x[lane], poses.y[lane] = float(centre[0]) + float(rng.uniform(-20, 20)), float(centre[1]) + float(rng.uniform(-20, 20))
        poses.view_z[lane] = float(smap.sector_heights[sector, 0]) + 41.0
        degrees = (0.0 if lane % 2 == 0 else 180.0) + float(rng.uniform(-12, 12))
        poses.angle_bam[lane] = int(round(degrees / 360.0 * 4294967296.0)) & 0xFFFFFFFF
    sprites = synthmap.generate_sprites(smap, lanes, 24, 12)
    return smap, poses, sprites


def corridor_case(lanes: int, sectors: int = 80):
    """corridor_parts as (map, derived tables, lane arrays)."""
    from gradoom_amd import mapbuild
    from gradoom_amd.selfcheck import make_lane_arrays

    smap, poses, sprites = corridor_parts(lanes, sectors)
    return smap, mapbuild.build_map_tables(smap), make_lane_arrays(smap, poses, sprites)


def outside_parts(lanes: int):
    """Cameras in the void beside a small map, 8 to 200 units off one of its four sides, looking wherever the generator
    turned them: no wall pass claims most of the screen.  (map, poses, sprites)"""
    from gradoom_amd import synthmap

    smap = synthmap.generate_map(7001, grid=(5, 4), sectors=17, linedefs=140, layout="grid", islands=4, pillars=2, midtex=0.1)
    poses = synthmap.generate_poses(smap, lanes, 11, pitch=True)
    segments = np.asarray(smap.wall_segments, dtype=np.float64)
    low = np.array([segments[:, [0, 2]].min(), segments[:, [1, 3]].min()])
    high = np.array([segments[:, [0, 2]].max(), segments[:, [1, 3]].max()])
    rng = np.random.default_rng(5)
    for lane in range(lanes):
        along, away = rng.uniform(0.1, 0.9), rng.uniform(8, 200)
        side = lane % 4
        if side < 2:
            poses.x[lane] = low[0] - away if side == 0 else high[0] + away
            poses.y[lane] = low[1] + along * (high[1] - low[1])
        else:
            poses.x[lane] = low[0] + along * (high[0] - low[0])
            poses.y[lane] = low[1] - away if side == 2 else high[1] + away
    sprites = synthmap.generate_sprites(smap, lanes, 24, 12)
    return smap, poses, sprites


def awkward_billboard_parts(seed: int, lanes: int, ties: bool = True):
    """closed_door_parts with its billboards moved to awkward places: exact depth ties with an earlier slot, at the eye,
    within a few units of it, far outside the map, on a vertex, on a linedef, lifted or sunk.  (map, poses, sprites)

    ``ties=False`` leaves out what puts two billboards at exactly the same depth (a shared spot, a second billboard at the
    eye).  The reference paints the billboards of a column in the order ``torch.topk`` returns them
    (``engine.py:14768-14780``), which among equal depths is whatever that routine's partial sort leaves: its CPU build
    paints five billboards at one spot in slot order in 319 columns of a frame and in another order in the 320th.  The
    oracle and the HIP path paint equal depths in slot order; only cases without ties can be compared with the reference."""
    smap, poses, sprites, _styles = closed_door_parts(seed, lanes, mixed=True, eye_any=True)
    rng = np.random.default_rng(seed * 13 + 5)
    segments = np.asarray(smap.wall_segments, dtype=np.float32)
    vertices = segments.reshape(-1, 2)
    for lane in range(lanes):
        at_the_eye = 0
        for slot in range(sprites.x.shape[1]):
            kind = int(rng.integers(0, 12))
            if kind == 0:
                sprites.z[lane, slot] += np.float32(rng.uniform(-60, 140))
            elif kind == 1 and slot > 0:
                other = int(rng.integers(0, slot))
                moved = bool(rng.random() < 0.5)
                lift = np.float32(rng.integers(-16, 17))
                if ties:
                    sprites.x[lane, slot], sprites.y[lane, slot] = sprites.x[lane, other], sprites.y[lane, other]
                    if moved:
                        sprites.z[lane, slot] = sprites.z[lane, other] + lift
            elif kind == 2:
                if ties or at_the_eye == 0:
                    sprites.x[lane, slot], sprites.y[lane, slot] = poses.x[lane], poses.y[lane]
                at_the_eye += 1
            elif kind == 3:
                angle, reach = float(rng.uniform(0, 6.283)), float(rng.choice([0.01, 0.5, 2.0, 6.0]))
                sprites.x[lane, slot] = poses.x[lane] + np.float32(reach * np.cos(angle))
                sprites.y[lane, slot] = poses.y[lane] + np.float32(reach * np.sin(angle))
            elif kind == 4:
                sprites.x[lane, slot] += np.float32(rng.uniform(-3000, 3000))
                sprites.y[lane, slot] += np.float32(rng.uniform(-3000, 3000))
            elif kind == 5:
                sprites.x[lane, slot], sprites.y[lane, slot] = vertices[int(rng.integers(0, len(vertices)))]
            elif kind == 6:
                wall, along = segments[int(rng.integers(0, len(segments)))], np.float32(rng.random())
                sprites.x[lane, slot] = wall[0] + along * (wall[2] - wall[0])
                sprites.y[lane, slot] = wall[1] + along * (wall[3] - wall[1])
    return smap, poses, sprites


def build_parts(recipe: dict, lanes: int):
    """(map, poses, sprites) of a recipe as the golden fixtures name it: {"kind": "closed_door" (the default) | "awkward_billboards" |
    "corridor" | "outside", ...the builder's own arguments}."""
    recipe = dict(recipe)
    kind = recipe.pop("kind", "closed_door")
    if kind == "closed_door":
        return closed_door_parts(recipe.pop("seed"), lanes, **recipe)[:3]
    if kind == "awkward_billboards":
        return awkward_billboard_parts(recipe.pop("seed"), lanes, **recipe)
    if kind == "corridor":
        return corridor_parts(lanes, **recipe)
    if kind == "outside":
        return outside_parts(lanes, **recipe)
    raise ValueError(f"unknown recipe kind {kind!r}")
