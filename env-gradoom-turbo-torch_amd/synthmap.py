"""Seeded synthetic maps, textures and camera poses for the batched renderer.

The generator emits the subset of the reference's ``CompiledScenario`` schema
that the native render path reads (``/root/reference/src/gradoom/scenario.py:302-401``):
linedef segments with exact shared float32 vertices, per-side texture ids in
(middle, bottom, top) order (``scenario.py:516``), sector heights/lights/flats,
one shared ``[T, maxH, maxW]`` texture atlas with power-of-two sizes, PLAYPAL,
COLORMAP and a raw sprite atlas.  Only NumPy is used so the same arrays can be
fed to the reference (to write golden vectors), to the CPU oracle and to the
HIP path.

Map shape: a jittered grid of quadrilateral cells.  A seeded subset of cells
is void (solid rock); every other cell is one sector.  An edge between two
sectors is a two-sided linedef, an edge between a sector and void/outside is
one-sided, and edges are split at exact dyadic points until the requested
linedef count is reached.  The front sector (``wall_sectors[w, 0]``) lies to
the right of the directed linedef, which is what makes a one-sided wall
front-facing from inside its sector (``engine.py:10777-10780``).
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np

CONFIGS = {
    # name: lanes, grid, sectors, linedefs, sprites/lane, masked-midtex probability
    "config1": dict(lanes=16, grid=(9, 6), sectors=48, linedefs=320, sprites=0, midtex=0.0),
    "config2": dict(lanes=256, grid=(12, 9), sectors=96, linedefs=800, sprites=32, midtex=0.0),
    "config3": dict(lanes=1024, grid=(15, 15), sectors=200, linedefs=2000, sprites=64, midtex=0.0),
    "config4": dict(lanes=4096, grid=(21, 21), sectors=400, linedefs=4000, sprites=128, midtex=0.15),
}

CELL = 256.0
JITTER = 40
MAX_SPLIT_DEPTH = 3


@dataclasses.dataclass
class SynthMap:
    """Host arrays of one synthetic scenario (names follow ``CompiledScenario``)."""

    vertices: np.ndarray  # [V,2] f32
    wall_segments: np.ndarray  # [W,4] f32 (x1,y1,x2,y2)
    wall_sectors: np.ndarray  # [W,2] i32 (front, back or -1)
    wall_side_texture_ids: np.ndarray  # [W,2,3] i32 (middle,bottom,top), -1 none
    wall_side_texture_offsets: np.ndarray  # [W,2,2] f32
    blocking_wall_indices: np.ndarray  # [B] i32
    sector_edge_mask: np.ndarray  # [S,W] bool
    sector_heights: np.ndarray  # [S,2] f32 (floor, ceiling)
    sector_lights: np.ndarray  # [S] i16
    sector_floor_texture_ids: np.ndarray  # [S] i32
    sector_ceiling_texture_ids: np.ndarray  # [S] i32
    texture_atlas: np.ndarray  # [T,maxH,maxW] u8
    texture_widths: np.ndarray  # [T] i32
    texture_heights: np.ndarray  # [T] i32
    playpal: np.ndarray  # [256,3] u8
    colormap: np.ndarray  # [34,256] u8
    sprite_atlas: np.ndarray  # [P,maxH,maxW] u8, index 0 transparent
    sprite_widths: np.ndarray  # [P] i32
    sprite_heights: np.ndarray  # [P] i32
    sprite_left_offsets: np.ndarray  # [P] i32
    sprite_top_offsets: np.ndarray  # [P] i32
    sector_cells: np.ndarray  # [S,2] i32 grid cell of each sector (generator bookkeeping)
    grid_points: np.ndarray  # [gy+1,gx+1,2] f32 jittered grid vertices
    sector_quads: np.ndarray | None = None  # [S,4,2] f64 corners p00,p10,p01,p11 used to place cameras/sprites
    void_boxes: np.ndarray | None = None  # [B,4] f64 x0,y0,x1,y1 of void pillars inside sectors (no camera goes there)
    wall_projection_fragments_fixed: np.ndarray | None = None  # [W,F,4] i64 16.16 BSP fragments (scenario.py:400)
    wall_projection_fragment_mask: np.ndarray | None = None  # [W,F] bool
    projectile_additive_luts: np.ndarray | None = None  # [2,256,256] u8 (scenario.py:367)
    sprite_translucent_lut: np.ndarray | None = None  # [256,256] u8 (scenario.py:368)

    @property
    def blocking_segments(self) -> np.ndarray:
        return self.wall_segments[self.blocking_wall_indices]

    @property
    def sprite_opaque(self) -> np.ndarray:
        return self.sprite_atlas != 0


@dataclasses.dataclass
class Poses:
    """Per-lane camera state, in the reference engine's own tensors' dtypes."""

    x: np.ndarray  # [N] f32
    y: np.ndarray  # [N] f32
    angle_bam: np.ndarray  # [N] i64, unsigned 32-bit BAM
    pitch_bam: np.ndarray  # [N] i64
    view_z: np.ndarray  # [N] f32
    flash_light: np.ndarray  # [N] i64 in {0,1,2}
    sector: np.ndarray  # [N] i32 sector the pose was drawn in (bookkeeping)


@dataclasses.dataclass
class Sprites:
    """Packed per-lane billboard list (the renderer's sprite input)."""

    x: np.ndarray  # [N,A] f32
    y: np.ndarray  # [N,A] f32
    z: np.ndarray  # [N,A] f32
    sprite: np.ndarray  # [N,A] i32 patch id
    alive: np.ndarray  # [N,A] bool
    fullbright: np.ndarray  # [N,A] bool
    style: np.ndarray | None = None  # [N,A] i8: -1 opaque, -2 translucent, >= 0 additive table (engine.py:14343)


def _split_edges(rng, edges, target):
    """Split ``edges`` (list of (p, q, front, back, depth)) at midpoints up to ``target``."""

    edges = list(edges)
    if len(edges) > target:
        raise ValueError(f"grid already has {len(edges)} linedefs, more than the {target} asked for")
    while len(edges) < target:
        order = rng.permutation(len(edges))
        progressed = False
        for index in order:
            if len(edges) >= target:
                break
            p, q, front, back, depth = edges[index]
            if depth >= MAX_SPLIT_DEPTH:
                continue
            mid = ((p[0] + q[0]) / 2.0, (p[1] + q[1]) / 2.0)
            edges[index] = (p, mid, front, back, depth + 1)
            edges.append((mid, q, front, back, depth + 1))
            progressed = True
        if not progressed:
            raise ValueError("cannot reach the requested linedef count at the split depth limit")
    return edges


def generate_map(
    seed: int,
    *,
    grid: tuple[int, int],
    sectors: int,
    linedefs: int,
    midtex: float = 0.0,
    wall_textures: int = 64,
    flats: int = 16,
    sprite_patches: int = 64,
    layout: str = "grid",
    islands: int = 0,
    pillars: int = 0,
) -> SynthMap:
    if layout == "brick":
        return _generate_brick_map(
            seed, grid=grid, sectors=sectors, linedefs=linedefs, midtex=midtex, wall_textures=wall_textures,
            flats=flats, sprite_patches=sprite_patches, islands=islands, pillars=pillars,
        )
    if layout != "grid":
        raise ValueError("layout must be 'grid' or 'brick'")
    rng = np.random.default_rng(seed)
    gx, gy = grid
    if sectors > gx * gy:
        raise ValueError("more sectors than grid cells")
    origin_x = -gx * CELL / 2.0
    origin_y = -gy * CELL / 2.0
    points = np.zeros((gy + 1, gx + 1, 2), dtype=np.float64)
    for j in range(gy + 1):
        for i in range(gx + 1):
            points[j, i, 0] = origin_x + i * CELL + int(rng.integers(-JITTER, JITTER + 1))
            points[j, i, 1] = origin_y + j * CELL + int(rng.integers(-JITTER, JITTER + 1))

    # Choose which cells are void; every other cell becomes a sector in row-major order.
    cell_sector = np.full((gy, gx), -1, dtype=np.int64)
    void = np.zeros(gy * gx, dtype=bool)
    void[rng.permutation(gy * gx)[: gy * gx - sectors]] = True
    sector_cells = []
    for j in range(gy):
        for i in range(gx):
            if not void[j * gx + i]:
                cell_sector[j, i] = len(sector_cells)
                sector_cells.append((i, j))

    def sector_of(i, j):
        if 0 <= i < gx and 0 <= j < gy:
            return int(cell_sector[j, i])
        return -1

    # Cells are counter-clockwise quads, so the interior is on the LEFT of each
    # directed boundary edge; a linedef wants its front sector on the RIGHT,
    # hence every edge is emitted reversed relative to its front cell.
    edges = []

    def add_edge(p, q, left_sector, right_sector):
        # left/right relative to the direction p->q.
        if left_sector < 0 and right_sector < 0:
            return
        if right_sector < 0:
            p, q, left_sector, right_sector = q, p, right_sector, left_sector
        elif left_sector >= 0 and rng.random() < 0.5:
            p, q, left_sector, right_sector = q, p, right_sector, left_sector
        edges.append((tuple(p), tuple(q), right_sector, left_sector, 0))

    for j in range(gy + 1):
        for i in range(gx):
            # horizontal edge from (i,j) to (i+1,j): cell above (j) is on the left, below (j-1) on the right
            add_edge(points[j, i], points[j, i + 1], sector_of(i, j), sector_of(i, j - 1))
    for j in range(gy):
        for i in range(gx + 1):
            # vertical edge from (i,j) to (i,j+1): cell (i-1) is on the left, cell (i) on the right
            add_edge(points[j, i], points[j + 1, i], sector_of(i - 1, j), sector_of(i, j))

    quads = np.zeros((len(sector_cells), 4, 2), dtype=np.float64)
    for index, (i, j) in enumerate(sector_cells):
        quads[index] = (points[j, i], points[j, i + 1], points[j + 1, i], points[j + 1, i + 1])
    return _finish_map(
        rng, edges, sector_cells, points, quads, linedefs=linedefs, midtex=midtex, wall_textures=wall_textures,
        flats=flats, sprite_patches=sprite_patches, islands=islands, pillars=pillars,
    )


def _add_islands(rng, edges, sector_cells, sector_quads, count):
    """Nest an axis-aligned rectangular sector in the middle of `count` cells.

    Opposite sides of an island bound the same sector pair with anti-parallel directions and no
    shared endpoint, the configuration the reference calls opposing portals (``engine.py:1605-1612``).
    """

    hosts = rng.permutation(len(sector_cells))[:count]
    quads = list(sector_quads)
    cells = list(sector_cells)
    for host in hosts:
        centre = np.round(np.mean(sector_quads[host], axis=0))
        half_w = float(rng.integers(3, 7) * 8)
        half_h = float(rng.integers(3, 7) * 8)
        x0, x1, y0, y1 = centre[0] - half_w, centre[0] + half_w, centre[1] - half_h, centre[1] + half_h
        island = len(cells)
        cells.append(tuple(sector_cells[host]))
        quads.append(np.asarray([(x0, y0), (x1, y0), (x0, y1), (x1, y1)], dtype=np.float64))
        # counter-clockwise loop: the island is on the left, so it is the back sector
        corners = [(x0, y0), (x1, y0), (x1, y1), (x0, y1)]
        for k in range(4):
            p, q = corners[k], corners[(k + 1) % 4]
            if rng.random() < 0.5:
                edges.append((p, q, int(host), island, MAX_SPLIT_DEPTH))
            else:
                edges.append((q, p, island, int(host), MAX_SPLIT_DEPTH))
    return edges, cells, np.asarray(quads, dtype=np.float64)


def with_blend_tables(smap: SynthMap, seed: int) -> SynthMap:
    """A copy of the map with seeded random additive / translucent blend tables (scenario.py:367-368)."""

    rng = np.random.default_rng(seed)
    return dataclasses.replace(
        smap,
        projectile_additive_luts=rng.integers(0, 256, (2, 256, 256), dtype=np.uint8),
        sprite_translucent_lut=rng.integers(0, 256, (256, 256), dtype=np.uint8),
    )


def with_variant(smap: SynthMap, seed: int, *, heights: str | None = None, textures: str | None = None, lights: bool = False) -> SynthMap:
    """A copy of the map with other sector heights, texture sizes or sector lights (same geometry, same texture ids).

    ``heights="uniform"``: floors uniform in 0..255, ceilings 64..256 above their floor, whole map units (so
    neighbouring sectors may not overlap vertically at all, and a map has as many plane levels as sectors).
    ``heights="doors"``: the quantised heights of ``generate_map`` with an eighth of the sectors closed (ceiling
    at the floor) and a tenth crawl spaces 8..24 units high.
    ``textures="mixed"``: wall textures of every power-of-two size from 8 to 256 either way, flats 64x64 or 64x128.
    ``textures="npot"``: half the wall textures have sizes that are no powers of two (WAD textures keep their
    native size, ``textures.py:209-218``): columns wrap modulo the width, rows modulo 2^floor(log2(height))
    (``engine.py:12792-12843``).
    ``lights``: other sector light levels.
    """

    rng = np.random.default_rng(seed)
    changes = {}
    count = len(smap.sector_heights)
    if heights == "uniform":
        floors = rng.integers(0, 256, count).astype(np.float32)
        changes["sector_heights"] = np.stack((floors, floors + rng.integers(64, 257, count).astype(np.float32)), axis=1)
    elif heights == "doors":
        sector_heights = smap.sector_heights.copy()
        kind = rng.random(count)
        closed = kind < 0.125
        crawl = (kind >= 0.125) & (kind < 0.225)
        sector_heights[closed, 1] = sector_heights[closed, 0]
        sector_heights[crawl, 1] = sector_heights[crawl, 0] + 8.0 * rng.integers(1, 4, int(crawl.sum()))
        changes["sector_heights"] = sector_heights.astype(np.float32)
    elif heights is not None:
        raise ValueError("heights must be 'uniform' or 'doors'")
    if textures in ("mixed", "npot"):
        total = len(smap.texture_widths)
        walls = int(np.min(np.concatenate((smap.sector_floor_texture_ids, smap.sector_ceiling_texture_ids))))   # flats follow the wall textures
        widths = smap.texture_widths.copy()
        tex_heights = smap.texture_heights.copy()
        widths[:walls] = 1 << rng.integers(3, 9, walls)
        tex_heights[:walls] = 1 << rng.integers(3, 9, walls)
        if textures == "npot":
            odd = rng.random(walls) < 0.5
            widths[:walls][odd] = rng.choice(np.asarray([24, 40, 72, 96, 100, 160, 200]), int(odd.sum()))
            odd = rng.random(walls) < 0.5
            tex_heights[:walls][odd] = rng.choice(np.asarray([24, 72, 96, 100, 136, 160, 200]), int(odd.sum()))
        tex_heights[walls:] = np.where(rng.random(total - walls) < 0.5, 64, 128)
        atlas = np.zeros((total, int(tex_heights.max()), int(widths.max())), dtype=np.uint8)
        for t in range(total):
            atlas[t, : tex_heights[t], : widths[t]] = rng.integers(0, 256, (int(tex_heights[t]), int(widths[t])), dtype=np.uint8)
        changes.update(texture_atlas=atlas, texture_widths=widths.astype(np.int32), texture_heights=tex_heights.astype(np.int32))
    elif textures is not None:
        raise ValueError("textures must be 'mixed' or 'npot'")
    if lights:
        changes["sector_lights"] = rng.integers(96, 256, count).astype(np.int16)
    return dataclasses.replace(smap, **changes)


def split_linedefs(smap: SynthMap, seed: int, share: float = 0.2, slots: int = 3) -> SynthMap:
    """Give a share of the linedefs two or three BSP projection fragments (scenario.py:420-454).

    A node builder splits a linedef at points rounded to 16.16, a hair off the line; the copy
    returned carries such fragments, the linedefs themselves stay as they are.
    """

    rng = np.random.default_rng(seed)
    walls_fixed = np.rint(smap.wall_segments.astype(np.float64) * 65536.0).astype(np.int64)
    wall_count = len(walls_fixed)
    fragments = np.zeros((wall_count, slots, 4), dtype=np.int64)
    mask = np.zeros((wall_count, slots), dtype=bool)
    for w in range(wall_count):
        start, end = walls_fixed[w, :2], walls_fixed[w, 2:]
        pieces = int(rng.integers(2, slots + 1)) if rng.random() < share else 1
        cuts = np.sort(rng.uniform(0.1, 0.9, pieces - 1))
        points = [start] + [np.rint(start + (end - start) * t).astype(np.int64) for t in cuts] + [end]
        for k in range(pieces):
            fragments[w, k, :2] = points[k]
            fragments[w, k, 2:] = points[k + 1]
            mask[w, k] = True
    return dataclasses.replace(smap, wall_projection_fragments_fixed=fragments, wall_projection_fragment_mask=mask)


def _add_pinched_pillars(rng, edges, sector_quads, hosts):
    """Two square void pillars that touch at one corner, in the middle of every host cell.

    Four one-sided linedefs of the same sector meet at the shared corner, so each of them has more than
    one endpoint neighbour there: the reference then drops its direct neighbour tables and takes the
    general neighbour-slot search (``engine.py:1558-1577``, ``engine.py:11672-11712``).
    """

    boxes = []
    for host in hosts:
        cx, cy = (float(v) for v in np.round(np.mean(sector_quads[host], axis=0)))
        a = float(rng.integers(2, 5) * 8)
        b = float(rng.integers(2, 5) * 8)
        for x0, y0, x1, y1 in ((cx - a, cy - a, cx, cy), (cx, cy, cx + b, cy + b)):
            corners = [(x0, y0), (x1, y0), (x1, y1), (x0, y1)]  # counter-clockwise: the void is on the left
            for k in range(4):
                edges.append((corners[k], corners[(k + 1) % 4], int(host), -1, MAX_SPLIT_DEPTH))
            boxes.append((x0, y0, x1, y1))
    return edges, np.asarray(boxes, dtype=np.float64)


def _finish_map(
    rng, edges, sector_cells, points, sector_quads, *, linedefs, midtex, wall_textures, flats, sprite_patches, islands=0,
    pillars=0,
):
    void_boxes = None
    if pillars:
        if islands + pillars > len(sector_cells):
            raise ValueError("more islands and pillars than cells")
        # hosts the islands (which draw the same permutation first) will not use
        state = rng.bit_generator.state
        island_hosts = set(int(h) for h in rng.permutation(len(sector_cells))[:islands]) if islands else set()
        rng.bit_generator.state = state
        free = [h for h in range(len(sector_cells)) if h not in island_hosts]
    if islands:
        edges, sector_cells, sector_quads = _add_islands(rng, edges, sector_cells, sector_quads, islands)
    if pillars:
        hosts = [free[int(k)] for k in rng.permutation(len(free))[:pillars]]
        edges, void_boxes = _add_pinched_pillars(rng, edges, sector_quads, hosts)
    edges = _split_edges(rng, edges, linedefs)
    order = rng.permutation(len(edges))
    edges = [edges[k] for k in order]
    wall_count = len(edges)
    wall_segments = np.asarray([(p[0], p[1], q[0], q[1]) for p, q, *_ in edges], dtype=np.float32)
    wall_sectors = np.asarray([(f, b) for _p, _q, f, b, _d in edges], dtype=np.int32)
    assert np.all(wall_segments.astype(np.float64) * 8 == np.round(wall_segments.astype(np.float64) * 8))
    vertices = np.unique(wall_segments.reshape(-1, 2), axis=0).astype(np.float32)

    sector_count = len(sector_cells)
    floors = rng.integers(0, 13, sector_count) * 8.0
    ceilings = 160.0 + rng.integers(0, 13, sector_count) * 8.0
    sector_heights = np.stack((floors, ceilings), axis=1).astype(np.float32)
    sector_lights = rng.integers(96, 256, sector_count).astype(np.int16)
    sector_floor_texture_ids = (wall_textures + rng.integers(0, flats, sector_count)).astype(np.int32)
    sector_ceiling_texture_ids = (wall_textures + rng.integers(0, flats, sector_count)).astype(np.int32)

    side_ids = np.full((wall_count, 2, 3), -1, dtype=np.int32)
    side_offsets = np.zeros((wall_count, 2, 2), dtype=np.float32)
    for w in range(wall_count):
        one_sided = wall_sectors[w, 1] < 0
        for side in range(1 if one_sided else 2):
            side_offsets[w, side] = rng.integers(0, 64, 2)
            if one_sided:
                side_ids[w, side, 0] = rng.integers(0, wall_textures)
            else:
                side_ids[w, side, 1] = rng.integers(0, wall_textures)
                side_ids[w, side, 2] = rng.integers(0, wall_textures)
                if midtex > 0.0 and rng.random() < midtex:
                    side_ids[w, side, 0] = rng.integers(0, wall_textures)

    sector_edge_mask = np.zeros((sector_count, wall_count), dtype=bool)
    for w in range(wall_count):
        front, back = wall_sectors[w]
        if front == back:
            continue
        sector_edge_mask[front, w] = True
        if back >= 0:
            sector_edge_mask[back, w] = True

    texture_total = wall_textures + flats
    atlas = np.zeros((texture_total, 128, 64), dtype=np.uint8)
    atlas[:wall_textures] = rng.integers(0, 256, (wall_textures, 128, 64), dtype=np.uint8)
    atlas[wall_textures:, :64, :] = rng.integers(0, 256, (flats, 64, 64), dtype=np.uint8)
    texture_widths = np.full(texture_total, 64, dtype=np.int32)
    texture_heights = np.concatenate(
        (np.full(wall_textures, 128, dtype=np.int32), np.full(flats, 64, dtype=np.int32))
    )
    playpal = rng.integers(0, 256, (256, 3), dtype=np.uint8)
    colormap = rng.integers(0, 256, (34, 256), dtype=np.uint8)

    sprite_widths = rng.integers(32, 65, sprite_patches).astype(np.int32)
    sprite_heights = rng.integers(32, 65, sprite_patches).astype(np.int32)
    sprite_atlas = np.zeros((sprite_patches, 64, 64), dtype=np.uint8)
    for p in range(sprite_patches):
        w, h = int(sprite_widths[p]), int(sprite_heights[p])
        patch = rng.integers(0, 256, (h, w), dtype=np.uint8)
        # Carve transparent holes so posts start below row 0 in some columns.
        holes = rng.random((h, w)) < 0.2
        patch[holes] = 0
        sprite_atlas[p, :h, :w] = patch
    sprite_left_offsets = (sprite_widths // 2).astype(np.int32)
    sprite_top_offsets = sprite_heights.astype(np.int32)

    return SynthMap(
        vertices=vertices,
        wall_segments=wall_segments,
        wall_sectors=wall_sectors,
        wall_side_texture_ids=side_ids,
        wall_side_texture_offsets=side_offsets,
        blocking_wall_indices=np.flatnonzero(wall_sectors[:, 1] < 0).astype(np.int32),
        sector_edge_mask=sector_edge_mask,
        sector_heights=sector_heights,
        sector_lights=sector_lights,
        sector_floor_texture_ids=sector_floor_texture_ids,
        sector_ceiling_texture_ids=sector_ceiling_texture_ids,
        texture_atlas=atlas,
        texture_widths=texture_widths,
        texture_heights=texture_heights,
        playpal=playpal,
        colormap=colormap,
        sprite_atlas=sprite_atlas,
        sprite_widths=sprite_widths,
        sprite_heights=sprite_heights,
        sprite_left_offsets=sprite_left_offsets,
        sprite_top_offsets=sprite_top_offsets,
        sector_cells=np.asarray(sector_cells, dtype=np.int32),
        grid_points=np.asarray(points, dtype=np.float32),
        sector_quads=sector_quads,
        void_boxes=void_boxes,
    )


def _generate_brick_map(seed, *, grid, sectors, linedefs, midtex, wall_textures, flats, sprite_patches, islands=0, pillars=0):
    """Staggered rows: odd rows are shifted by half a cell, so every interior vertex joins three sectors.

    At such a T-junction all three pairwise linedefs exist, which is what the reference's
    three-sector "bridge" tables (``engine.py:399-484``) index; the plain grid never produces one.
    """

    rng = np.random.default_rng(seed)
    gx, gy = grid
    jitter = 24
    origin_x = -gx * CELL / 2.0
    origin_y = -gy * CELL / 2.0

    def row_boundaries(j):
        if j % 2 == 0:
            return [origin_x + i * CELL for i in range(gx + 1)]
        return [origin_x] + [origin_x + (i + 0.5) * CELL for i in range(gx)] + [origin_x + gx * CELL]

    # vertices on horizontal line j (between rows j-1 and j), keyed by nominal x
    line_points: list[dict[float, tuple[float, float]]] = []
    for j in range(gy + 1):
        xs = set()
        if j < gy:
            xs.update(row_boundaries(j))
        if j > 0:
            xs.update(row_boundaries(j - 1))
        line = {}
        for x in sorted(xs):
            line[x] = (x + int(rng.integers(-jitter, jitter + 1)), origin_y + j * CELL + int(rng.integers(-jitter, jitter + 1)))
        line_points.append(line)

    cells = [(i, j) for j in range(gy) for i in range(len(row_boundaries(j)) - 1)]
    if sectors > len(cells):
        raise ValueError("more sectors than brick cells")
    void = np.zeros(len(cells), dtype=bool)
    void[rng.permutation(len(cells))[: len(cells) - sectors]] = True
    cell_sector = {}
    sector_cells = []
    for index, cell in enumerate(cells):
        if not void[index]:
            cell_sector[cell] = len(sector_cells)
            sector_cells.append(cell)

    def sector_of_x(j, x):
        """Sector of the row-j cell whose nominal x-range contains x (x is an interval midpoint)."""
        if not 0 <= j < gy:
            return -1
        bounds = row_boundaries(j)
        for i in range(len(bounds) - 1):
            if bounds[i] < x < bounds[i + 1]:
                return cell_sector.get((i, j), -1)
        return -1

    edges = []

    def add_edge(p, q, left_sector, right_sector):
        if left_sector < 0 and right_sector < 0:
            return
        if right_sector < 0:
            p, q, left_sector, right_sector = q, p, right_sector, left_sector
        elif left_sector >= 0 and rng.random() < 0.5:
            p, q, left_sector, right_sector = q, p, right_sector, left_sector
        edges.append((tuple(p), tuple(q), right_sector, left_sector, 0))

    for j in range(gy + 1):
        xs = sorted(line_points[j])
        for a, b in zip(xs[:-1], xs[1:]):
            mid = (a + b) / 2.0
            # direction +x: the row above (j) is on the left, the row below (j-1) on the right
            add_edge(line_points[j][a], line_points[j][b], sector_of_x(j, mid), sector_of_x(j - 1, mid))
    for j in range(gy):
        bounds = row_boundaries(j)
        for i, x in enumerate(bounds):
            left = cell_sector.get((i - 1, j), -1) if i > 0 else -1
            right = cell_sector.get((i, j), -1) if i < len(bounds) - 1 else -1
            # direction +y: the cell at smaller x is on the left
            add_edge(line_points[j][x], line_points[j + 1][x], left, right)

    quads = np.zeros((len(sector_cells), 4, 2), dtype=np.float64)
    for index, (i, j) in enumerate(sector_cells):
        bounds = row_boundaries(j)
        quads[index] = (line_points[j][bounds[i]], line_points[j][bounds[i + 1]], line_points[j + 1][bounds[i]], line_points[j + 1][bounds[i + 1]])
    points = np.zeros((1, 1, 2), dtype=np.float64)
    return _finish_map(
        rng, edges, sector_cells, points, quads, linedefs=linedefs, midtex=midtex, wall_textures=wall_textures,
        flats=flats, sprite_patches=sprite_patches, islands=islands, pillars=pillars,
    )


def generate_config_map(name: str, seed: int | None = None) -> SynthMap:
    cfg = CONFIGS[name]
    if seed is None:
        seed = 1000 + int(name[-1])
    return generate_map(
        seed,
        grid=cfg["grid"],
        sectors=cfg["sectors"],
        linedefs=cfg["linedefs"],
        midtex=cfg["midtex"],
    )


def _point_in_cell(smap: SynthMap, sector: int, u: float, v: float) -> tuple[float, float]:
    p00, p10, p01, p11 = smap.sector_quads[sector]
    point = (1 - u) * (1 - v) * p00 + u * (1 - v) * p10 + (1 - u) * v * p01 + u * v * p11
    # 1/16 map unit keeps the float32 value and its 16.16 image both exact.
    return float(np.round(point[0] * 16) / 16), float(np.round(point[1] * 16) / 16)


def generate_poses(
    smap: SynthMap,
    lanes: int,
    seed: int,
    *,
    pitch: bool = False,
    flash: bool = False,
    frame: int = 0,
    margin: float = 0.15,
    eye: str = "standing",
) -> Poses:
    """Random camera poses strictly inside sectors (bilinear margin keeps them off the walls).

    A small ``margin`` puts cameras close to walls and vertices, where linedefs are seen edge-on and
    the thin-span ownership rules of the wall traversal come into play.
    """

    return generate_picked_poses(
        smap, [(seed, lane) for lane in range(lanes)], pitch=pitch, flash=flash, frame=frame, margin=margin, eye=eye
    )


def generate_picked_poses(
    smap: SynthMap,
    picks,
    *,
    pitch: bool = False,
    flash: bool = False,
    frame: int = 0,
    margin: float = 0.15,
    eye: str = "standing",
) -> Poses:
    """The poses ``generate_poses`` gives lane ``lane`` under ``seed``, for a list of (seed, lane) pairs.

    Cameras stand in sectors at least 56 units high, eyes 41 units above the floor (``eye="standing"``) or anywhere
    from 8 units above the floor to 8 below the ceiling (``eye="any"``: crouching, falling, on a lift).
    """

    lanes = len(picks)
    x = np.zeros(lanes, dtype=np.float32)
    y = np.zeros(lanes, dtype=np.float32)
    angle_bam = np.zeros(lanes, dtype=np.int64)
    pitch_bam = np.zeros(lanes, dtype=np.int64)
    view_z = np.zeros(lanes, dtype=np.float32)
    flash_light = np.zeros(lanes, dtype=np.int64)
    sector = np.zeros(lanes, dtype=np.int32)
    sector_count = len(smap.sector_heights)
    if lanes and not np.any(smap.sector_heights[:, 1] - smap.sector_heights[:, 0] >= 56.0):
        raise ValueError("no sector of the map is high enough for a camera to stand in (56 units)")
    for slot, (seed, lane) in enumerate(picks):
        rng = np.random.default_rng((seed * 65536 + lane) * 4096 + frame)
        s = int(rng.integers(0, sector_count))
        while smap.sector_heights[s, 1] - smap.sector_heights[s, 0] < 56.0:   # no room to stand (closed doors, crawl spaces)
            s = int(rng.integers(0, sector_count))
        for attempt in range(10000):
            u, v = rng.uniform(margin, 1.0 - margin, 2)
            px, py = _point_in_cell(smap, s, float(u), float(v))
            if smap.void_boxes is None or not np.any(
                (px > smap.void_boxes[:, 0] - 4) & (px < smap.void_boxes[:, 2] + 4)
                & (py > smap.void_boxes[:, 1] - 4) & (py < smap.void_boxes[:, 3] + 4)
            ):
                break
        else:
            raise ValueError(f"sector {s} has no spot clear of the map's void boxes for a camera")
        x[slot], y[slot] = px, py
        angle_bam[slot] = int(rng.integers(0, 1 << 32))
        view_z[slot] = smap.sector_heights[s, 0] + 41.0
        if pitch:
            pitch_bam[slot] = int(rng.integers(-10, 11)) * (182 << 16)
        if flash:
            flash_light[slot] = int(rng.integers(0, 3))
        if eye == "any":
            headroom = int(smap.sector_heights[s, 1] - smap.sector_heights[s, 0])
            view_z[slot] = smap.sector_heights[s, 0] + float(rng.integers(8, headroom - 7))
        elif eye != "standing":
            raise ValueError("eye must be 'standing' or 'any'")
        sector[slot] = s
    return Poses(x, y, angle_bam, pitch_bam, view_z, flash_light, sector)


def generate_sprites(smap: SynthMap, lanes: int, count: int, seed: int, frame: int = 0) -> Sprites:
    """Random billboards standing on sector floors; depths are distinct with probability one."""

    shape = (lanes, max(count, 0))
    x = np.zeros(shape, dtype=np.float32)
    y = np.zeros(shape, dtype=np.float32)
    z = np.zeros(shape, dtype=np.float32)
    sprite = np.zeros(shape, dtype=np.int32)
    alive = np.zeros(shape, dtype=bool)
    fullbright = np.zeros(shape, dtype=bool)
    sector_count = len(smap.sector_heights)
    patches = len(smap.sprite_widths)
    for lane in range(lanes):
        rng = np.random.default_rng(((seed + 7919) * 65536 + lane) * 4096 + frame)
        for a in range(count):
            s = int(rng.integers(0, sector_count))
            u, v = rng.uniform(0.1, 0.9, 2)
            px, py = _point_in_cell(smap, s, float(u), float(v))
            x[lane, a], y[lane, a] = px, py
            z[lane, a] = smap.sector_heights[s, 0]
            sprite[lane, a] = int(rng.integers(0, patches))
            alive[lane, a] = rng.random() < 0.9
            fullbright[lane, a] = rng.random() < 0.1
    return Sprites(x, y, z, sprite, alive, fullbright)


def bam_to_radians_f32(angle_bam: np.ndarray) -> np.ndarray:
    """float32 view angle the reference derives from a retained BAM (``engine.py:10651``)."""

    return (angle_bam.astype(np.float32) * np.float32(2.0 * math.pi / float(1 << 32))).astype(np.float32)


def _points_in_cells(smap: SynthMap, sectors: np.ndarray, u: np.ndarray, v: np.ndarray):
    """Vectorised ``_point_in_cell`` (same bilinear map, same 1/16-unit snapping)."""

    quads = smap.sector_quads[sectors]
    p00, p10, p01, p11 = quads[..., 0, :], quads[..., 1, :], quads[..., 2, :], quads[..., 3, :]
    u = u[..., None]
    v = v[..., None]
    point = (1 - u) * (1 - v) * p00 + u * (1 - v) * p10 + (1 - u) * v * p01 + u * v * p11
    point = np.round(point * 16) / 16
    return point[..., 0].astype(np.float32), point[..., 1].astype(np.float32)


def generate_poses_batch(smap: SynthMap, lanes: int, seed: int, *, pitch: bool = False, flash: bool = False) -> Poses:
    """Same distribution as ``generate_poses`` from one generator (for large batches)."""

    rng = np.random.default_rng(seed)
    sector = rng.integers(0, len(smap.sector_heights), lanes)
    x, y = _points_in_cells(smap, sector, rng.uniform(0.15, 0.85, lanes), rng.uniform(0.15, 0.85, lanes))
    angle_bam = rng.integers(0, 1 << 32, lanes).astype(np.int64)
    pitch_bam = (rng.integers(-10, 11, lanes) * (182 << 16)).astype(np.int64) if pitch else np.zeros(lanes, np.int64)
    flash_light = rng.integers(0, 3, lanes).astype(np.int64) if flash else np.zeros(lanes, np.int64)
    view_z = (smap.sector_heights[sector, 0] + 41.0).astype(np.float32)
    return Poses(x, y, angle_bam, pitch_bam, view_z, flash_light, sector.astype(np.int32))


def generate_sprites_batch(smap: SynthMap, lanes: int, count: int, seed: int) -> Sprites:
    """Same distribution as ``generate_sprites`` from one generator (for large batches)."""

    rng = np.random.default_rng(seed + 7919)
    shape = (lanes, count)
    sector = rng.integers(0, len(smap.sector_heights), shape)
    x, y = _points_in_cells(smap, sector, rng.uniform(0.1, 0.9, shape), rng.uniform(0.1, 0.9, shape))
    z = smap.sector_heights[sector, 0].astype(np.float32)
    sprite = rng.integers(0, len(smap.sprite_widths), shape).astype(np.int32)
    alive = rng.random(shape) < 0.9
    fullbright = rng.random(shape) < 0.1
    return Sprites(x, y, z, sprite, alive, fullbright)


def generate_overlays(seed: int, *, weapon_patches: int = 12, cooldowns: int = 8) -> dict:
    """Seeded weapon psprite and status bar patches, named like ``gd_overlay_desc``'s fields.

    Shapes follow the reference's assets: psprite patches with the negative offsets Doom uses
    to place them (``engine.py:14997-15020``), a 320x32 status bar, an arms panel, 14-pixel big
    digits, 4-pixel small digits, faces, owned / missing weapon numbers (patch ids as in
    ``engine.py:15186-15259``).  Also the ``[8, 2, cooldowns]`` weapon frame / flash / flash
    light tables of ``engine.py:14949-14967``.
    """

    rng = np.random.default_rng(seed)
    wh, ww = 112, 160
    weapon_atlas = np.zeros((weapon_patches, wh, ww), dtype=np.uint8)
    weapon_opaque = np.zeros((weapon_patches, wh, ww), dtype=np.uint8)
    weapon_w = rng.integers(40, ww + 1, weapon_patches).astype(np.int32)
    weapon_h = rng.integers(40, wh + 1, weapon_patches).astype(np.int32)
    weapon_left = -rng.integers(60, 200, weapon_patches).astype(np.int32)
    weapon_top = -rng.integers(40, 150, weapon_patches).astype(np.int32)
    for p in range(weapon_patches):
        w, h = int(weapon_w[p]), int(weapon_h[p])
        weapon_atlas[p, :h, :w] = rng.integers(1, 256, (h, w), dtype=np.uint8)
        weapon_opaque[p, :h, :w] = rng.random((h, w)) < 0.8
    hud_patches = 70
    hh, hw = 32, 320
    hud_w = np.zeros(hud_patches, dtype=np.int32)
    hud_h = np.zeros(hud_patches, dtype=np.int32)
    hud_left = np.zeros(hud_patches, dtype=np.int32)
    hud_top = np.zeros(hud_patches, dtype=np.int32)
    for p in range(hud_patches):
        if p == 0:
            size, offsets = (320, 32), (0, 0)
        elif p == 1:
            size, offsets = (40, 32), (0, 0)
        elif 2 <= p <= 12:
            size, offsets = (14, 16), (int(rng.integers(-2, 3)), int(rng.integers(-2, 3)))
        elif 28 <= p <= 43:
            size, offsets = (4, 6), (int(rng.integers(-1, 2)), int(rng.integers(-1, 2)))
        else:  # faces
            size, offsets = (int(rng.integers(22, 27)), int(rng.integers(27, 32))), (int(rng.integers(-3, 4)), int(rng.integers(-3, 2)))
        hud_w[p], hud_h[p] = size
        hud_left[p], hud_top[p] = offsets
    hud_atlas = np.zeros((hud_patches, hh, hw), dtype=np.uint8)
    hud_opaque = np.zeros((hud_patches, hh, hw), dtype=np.uint8)
    for p in range(hud_patches):
        w, h = int(hud_w[p]), int(hud_h[p])
        hud_atlas[p, :h, :w] = rng.integers(1, 256, (h, w), dtype=np.uint8)
        hud_opaque[p, :h, :w] = rng.random((h, w)) < 0.85
    frame_ids = rng.integers(0, weapon_patches, (8, 2, cooldowns)).astype(np.int32)
    flash_ids = np.where(rng.random((8, 2, cooldowns)) < 0.4, rng.integers(0, weapon_patches, (8, 2, cooldowns)), -1).astype(np.int32)
    flash_lights = np.where(flash_ids >= 0, rng.integers(1, 3, (8, 2, cooldowns)), 0).astype(np.int64)
    # bullet chip decals (scenario.py:370-375): five variants of one width, transparent where 0
    dh, dw = 16, 12
    decal_h = rng.integers(8, dh + 1, 5).astype(np.int32)
    decal_atlas = np.zeros((5, dh, dw), dtype=np.uint8)
    for v in range(5):
        patch = rng.integers(1, 256, (int(decal_h[v]), dw), dtype=np.uint8)
        patch[rng.random(patch.shape) < 0.25] = 0
        decal_atlas[v, : decal_h[v]] = patch
    decal_left = rng.integers(3, 9, 5).astype(np.int32)
    decal_top = rng.integers(3, 12, 5).astype(np.int32)
    decal_opacity_lut = rng.integers(0, 65, (32, 256), dtype=np.uint8)
    decal_black_lut = rng.integers(0, 256, (65, 256), dtype=np.uint8)
    return dict(
        weapon_atlas=weapon_atlas, weapon_opaque=weapon_opaque, weapon_w=weapon_w, weapon_h=weapon_h,
        weapon_left=weapon_left, weapon_top=weapon_top, hud_atlas=hud_atlas, hud_opaque=hud_opaque, hud_w=hud_w,
        hud_h=hud_h, hud_left=hud_left, hud_top=hud_top, weapon_frame_ids=frame_ids, weapon_flash_ids=flash_ids,
        weapon_flash_lights=flash_lights, decal_atlas=decal_atlas, decal_h=decal_h, decal_left=decal_left,
        decal_top=decal_top, decal_opacity_lut=decal_opacity_lut, decal_black_lut=decal_black_lut,
    )
