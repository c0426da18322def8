"""Host-side derivation of the map tables the renderer consumes (NumPy only).

Restates, in compact form, what the reference derives once per scenario in
``DeviceScenario.from_host`` (``/root/reference/src/gradoom/engine.py:721-849``)
and in ``TorchDeathmatchEngine.__init__`` (``engine.py:1527-1634``).  The
reference's dense ``[W, W]`` / ``[2, W, W]`` tables do not scale to thousands of
linedefs; here every pairwise relation is reduced to (a) vertex ids assigned by
exact float32 equality of endpoints and (b) CSR adjacency lists, from which the
kernels answer the same queries on the fly.
"""

from __future__ import annotations

import numpy as np

FIXED_UNIT = 65536


def _csr(rows: list[list[int]]) -> tuple[np.ndarray, np.ndarray]:
    offsets = np.zeros(len(rows) + 1, dtype=np.int32)
    for i, row in enumerate(rows):
        offsets[i + 1] = offsets[i] + len(row)
    flat = [v for row in rows for v in row]
    return offsets, np.asarray(flat if flat else [0], dtype=np.int32)


def build_blend_tables(smap) -> dict[str, np.ndarray]:
    """Blend tables of styled sprites, with the reference's defaults when the map has none (engine.py:1017-1032):
    the additive default shows the lit texel, the translucent default the pixel under the sprite."""

    additive = getattr(smap, "projectile_additive_luts", None)
    translucent = getattr(smap, "sprite_translucent_lut", None)
    if additive is None:
        additive = np.broadcast_to(np.arange(256, dtype=np.uint8)[None, None, :], (2, 256, 256))
    if translucent is None:
        translucent = np.broadcast_to(np.arange(256, dtype=np.uint8)[:, None], (256, 256))
    additive = np.ascontiguousarray(additive, dtype=np.uint8)
    translucent = np.ascontiguousarray(translucent, dtype=np.uint8)
    if additive.shape != (2, 256, 256) or translucent.shape != (256, 256):
        raise ValueError("projectile_additive_luts must be [2,256,256] and sprite_translucent_lut [256,256]")
    return dict(additive_luts=additive, translucent_lut=translucent)


def build_split_tables(smap, walls_fixed: np.ndarray) -> dict[str, np.ndarray | int]:
    """Projection fragments of the linedefs a BSP builder split (scenario.py:420-454).

    A linedef whose only fragment is the linedef itself needs no row: the renderer then projects with
    the linedef's own FWallCoords, which is what the reference computes for it (engine.py:12310-12380).
    """

    fragments = getattr(smap, "wall_projection_fragments_fixed", None)
    mask = getattr(smap, "wall_projection_fragment_mask", None)
    wall_count = len(walls_fixed)
    if (fragments is None) != (mask is None):
        raise ValueError("wall projection fragments and their mask must be provided together")
    if fragments is None:
        fragments = walls_fixed.astype(np.int64)[:, None, :]
        mask = np.ones((wall_count, 1), dtype=bool)
    fragments = np.asarray(fragments, dtype=np.int64)
    mask = np.asarray(mask, dtype=bool)
    if fragments.shape[:2] != mask.shape or fragments.shape[2:] != (4,) or len(fragments) != wall_count:
        raise ValueError("invalid wall projection fragment arrays")
    if np.abs(fragments).max(initial=0) >= 2**31:
        raise ValueError("projection fragment coordinates do not fit 16.16 in int32")
    slots = max(1, mask.shape[1])
    plain = mask[:, 0] & ~mask[:, 1:].any(axis=1) & np.all(fragments[:, 0] == walls_fixed, axis=1)
    rows = np.flatnonzero(~plain)
    wall_split_slot = np.full(wall_count, -1, dtype=np.int32)
    wall_split_slot[rows] = np.arange(len(rows), dtype=np.int32)
    if len(rows):
        split_fragments = np.ascontiguousarray(fragments[rows], dtype=np.int32)
        split_mask = np.ascontiguousarray(mask[rows], dtype=np.uint8)
    else:
        split_fragments = np.zeros((1, slots, 4), dtype=np.int32)
        split_mask = np.zeros((1, slots), dtype=np.uint8)
    return dict(
        fragment_slots=int(slots), split_count=int(len(rows)), wall_split_slot=wall_split_slot,
        split_fragments_fixed=split_fragments, split_fragment_mask=split_mask,
    )


def build_map_tables(smap) -> dict[str, np.ndarray | int]:
    """Return contiguous arrays keyed by the field names of ``gd_map_desc``."""

    walls = np.ascontiguousarray(smap.wall_segments, dtype=np.float32)
    wall_count = len(walls)
    sectors = np.ascontiguousarray(smap.wall_sectors, dtype=np.int32)
    sector_count = len(smap.sector_heights)
    if wall_count == 0 or sector_count == 0:
        raise ValueError("a map needs at least one linedef and one sector")
    if np.abs(walls).max() >= 16384:
        raise ValueError("map coordinates must stay below 16384 units (16.16 in int32)")

    # rint(walls * 65536): engine.py:749-751 (float64) and engine.py:10876 (float32) agree
    # whenever the product is exact, which the int32 range check above guarantees only for
    # coordinates with <= 8 fractional bits; verify instead of assuming.
    fixed32 = np.rint(walls * np.float32(FIXED_UNIT))
    fixed64 = np.rint(walls.astype(np.float64) * FIXED_UNIT)
    if not np.array_equal(fixed32.astype(np.float64), fixed64):
        raise ValueError("linedef coordinates are not exactly representable in 16.16")
    walls_fixed = fixed64.astype(np.int32)

    # Vertex ids by exact float equality (-0.0 == 0.0), as engine.py:776-781 compares them.
    vertex_ids: dict[tuple[float, float], int] = {}
    wall_vertex = np.zeros((wall_count, 2), dtype=np.int32)
    for w in range(wall_count):
        for slot in range(2):
            key = (float(walls[w, 2 * slot]) + 0.0, float(walls[w, 2 * slot + 1]) + 0.0)
            wall_vertex[w, slot] = vertex_ids.setdefault(key, len(vertex_ids))
    vertex_count = len(vertex_ids)
    vertex_rows: list[list[int]] = [[] for _ in range(vertex_count)]
    for w in range(wall_count):
        for slot in range(2):
            v = int(wall_vertex[w, slot])
            if not vertex_rows[v] or vertex_rows[v][-1] != w:
                vertex_rows[v].append(w)
    vertex_wall_ofs, vertex_wall_idx = _csr(vertex_rows)

    one_sided = sectors[:, 1] < 0

    def same_pair(a: int, b: int) -> bool:
        return (sectors[a, 0] == sectors[b, 0] and sectors[a, 1] == sectors[b, 1]) or (
            sectors[a, 0] == sectors[b, 1] and sectors[a, 1] == sectors[b, 0]
        )

    def shares(a: int, slot: int, b: int) -> bool:
        v = wall_vertex[a, slot]
        return wall_vertex[b, 0] == v or wall_vertex[b, 1] == v

    # Endpoint neighbours: same sector pair and a shared endpoint (engine.py:769-786, 831-849).
    neighbor_rows: list[list[int]] = []
    for w in range(wall_count):
        near = set()
        for slot in range(2):
            v = int(wall_vertex[w, slot])
            near.update(vertex_rows[v])
        near.discard(w)
        neighbor_rows.append(sorted(n for n in near if same_pair(w, n)))
    slots = max(1, max(len(row) for row in neighbor_rows))
    endpoint_neighbors = np.repeat(np.arange(wall_count, dtype=np.int32)[:, None], slots, axis=1)
    neighbor_starts = np.zeros((wall_count, slots), dtype=np.uint8)
    neighbor_ends = np.zeros((wall_count, slots), dtype=np.uint8)
    for w, row in enumerate(neighbor_rows):
        for k, n in enumerate(row):
            endpoint_neighbors[w, k] = n
            neighbor_starts[w, k] = shares(w, 0, n)
            neighbor_ends[w, k] = shares(w, 1, n)
    direct = bool(np.all(neighbor_starts.sum(axis=1) <= 1) and np.all(neighbor_ends.sum(axis=1) <= 1))

    # engine.py:1558-1575: argmax over the start / end flags picks the first set slot (0 when none)
    direct_table = np.zeros((wall_count, 4), dtype=np.int32)
    every = np.arange(wall_count)
    start_slot = np.argmax(neighbor_starts, axis=1)
    end_slot = np.argmax(neighbor_ends, axis=1)
    direct_table[:, 0] = endpoint_neighbors[every, start_slot]
    direct_table[:, 1] = endpoint_neighbors[every, end_slot]
    direct_table[:, 2] = (
        start_slot | (end_slot << 8) | (neighbor_starts.any(axis=1).astype(np.int64) << 16) | (neighbor_ends.any(axis=1).astype(np.int64) << 17)
    )

    # One-hop solid bridges (engine.py:787-830): bridge[w] = { k : exists j one-sided,
    # sharing w's start (resp. end), with sectors[j,0] in sectors[w], and k one-sided,
    # k != j, sharing any endpoint with j, sectors[k,0] == sectors[j,0] }.
    def solid_bridges(slot: int) -> list[list[int]]:
        rows: list[list[int]] = []
        for w in range(wall_count):
            found = set()
            for j in vertex_rows[int(wall_vertex[w, slot])]:
                if not one_sided[j]:
                    continue
                if not (sectors[w, 0] == sectors[j, 0] or sectors[w, 1] == sectors[j, 0]):
                    continue
                for jslot in range(2):
                    for k in vertex_rows[int(wall_vertex[j, jslot])]:
                        if k != j and one_sided[k] and sectors[k, 0] == sectors[j, 0]:
                            found.add(k)
            rows.append(sorted(found))
        return rows

    solid_bridge_start_ofs, solid_bridge_start_idx = _csr(solid_bridges(0))
    solid_bridge_end_ofs, solid_bridge_end_idx = _csr(solid_bridges(1))

    sector_wall_rows: list[list[int]] = [[] for _ in range(sector_count)]
    for w in range(wall_count):
        front, back = int(sectors[w, 0]), int(sectors[w, 1])
        if front >= 0:
            sector_wall_rows[front].append(w)
        if back >= 0 and back != front:
            sector_wall_rows[back].append(w)
    sector_wall_ofs, sector_wall_idx = _csr(sector_wall_rows)
    edge_mask = np.asarray(smap.sector_edge_mask, dtype=bool)
    sector_edge_ofs, sector_edge_idx = _csr([np.flatnonzero(edge_mask[s]).tolist() for s in range(sector_count)])

    dx = walls[:, 2] - walls[:, 0]
    dy = walls[:, 3] - walls[:, 1]
    wall_len = np.floor(np.sqrt(np.square(dx) + np.square(dy)) + 0.5).astype(np.float32)

    tex_atlas = np.ascontiguousarray(smap.texture_atlas, dtype=np.uint8)
    tex_w = np.ascontiguousarray(smap.texture_widths, dtype=np.int32)
    tex_h = np.ascontiguousarray(smap.texture_heights, dtype=np.int32)
    # Any size from 1 to 32768: wall columns wrap modulo the width, rows and flats modulo 2^floor(log2(size))
    # (engine.py:12792-12843, 10886-10889), so sizes need not be powers of two.
    for name, values in (("width", tex_w), ("height", tex_h)):
        if np.any(values <= 0) or np.any(values > 32768):
            raise ValueError(f"texture {name}s must lie in 1..32768")
    if np.any(tex_w > tex_atlas.shape[2]) or np.any(tex_h > tex_atlas.shape[1]):
        raise ValueError("a texture is larger than the atlas")

    spr_atlas = np.ascontiguousarray(smap.sprite_atlas, dtype=np.uint8)
    spr_opaque = np.ascontiguousarray(smap.sprite_opaque, dtype=np.uint8)
    # First source row of the opaque post containing each texel (engine.py:14230-14256).
    prior = np.concatenate((np.zeros_like(spr_opaque[:, :1]), spr_opaque[:, :-1]), axis=1)
    starts = (spr_opaque != 0) & (prior == 0)
    rows = np.arange(spr_opaque.shape[1], dtype=np.int64)[None, :, None]
    spr_post_top = np.maximum.accumulate(np.where(starts, rows, 0), axis=1).astype(np.uint8)

    heights = np.ascontiguousarray(smap.sector_heights, dtype=np.float32)
    # Plane levels in the order that makes plane height (and so ray distance) ascend:
    # floors from the highest down, ceilings from the lowest up.
    floor_levels = np.unique(heights[:, 0])[::-1].astype(np.float32).copy()
    ceil_levels = np.unique(heights[:, 1]).astype(np.float32).copy()
    fine_cell = fine_cell_size(walls)
    grid = build_sector_grid(walls, sector_edge_ofs, sector_edge_idx, sector_count, cell=fine_cell * FINE_PER_COARSE)
    grid.update(build_fine_grid(walls, sector_edge_ofs, sector_edge_idx, sector_count, grid["grid_min_x"], grid["grid_min_y"],
                                fine_cell, heights, floor_levels, ceil_levels))

    split = build_split_tables(smap, walls_fixed)

    return dict(
        **split,
        floor_level_count=int(len(floor_levels)),
        ceil_level_count=int(len(ceil_levels)),
        floor_levels=floor_levels,
        ceil_levels=ceil_levels,
        **grid,
        wall_count=wall_count,
        sector_count=sector_count,
        vertex_count=vertex_count,
        texture_count=int(tex_atlas.shape[0]),
        tex_max_h=int(tex_atlas.shape[1]),
        tex_max_w=int(tex_atlas.shape[2]),
        sprite_count=int(spr_atlas.shape[0]),
        spr_max_h=int(spr_atlas.shape[1]),
        spr_max_w=int(spr_atlas.shape[2]),
        blocking_count=int(len(smap.blocking_wall_indices)),
        neighbor_slots=int(slots),
        direct_neighbors=int(direct),
        walls=walls,
        walls_fixed=walls_fixed,
        wall_sectors=sectors,
        wall_vertex=wall_vertex,
        side_tex=np.ascontiguousarray(smap.wall_side_texture_ids, dtype=np.int32),
        side_off=np.ascontiguousarray(smap.wall_side_texture_offsets, dtype=np.float32),
        wall_len=wall_len,
        endpoint_neighbors=endpoint_neighbors,
        endpoint_neighbor_starts=neighbor_starts,
        endpoint_neighbor_ends=neighbor_ends,
        direct_neighbor_table=direct_table,
        solid_bridge_start_ofs=solid_bridge_start_ofs,
        solid_bridge_start_idx=solid_bridge_start_idx,
        solid_bridge_end_ofs=solid_bridge_end_ofs,
        solid_bridge_end_idx=solid_bridge_end_idx,
        vertex_wall_ofs=vertex_wall_ofs,
        vertex_wall_idx=vertex_wall_idx,
        sector_wall_ofs=sector_wall_ofs,
        sector_wall_idx=sector_wall_idx,
        sector_edge_ofs=sector_edge_ofs,
        sector_edge_idx=sector_edge_idx,
        blocking_walls=np.ascontiguousarray(smap.blocking_wall_indices, dtype=np.int32),
        sector_heights=np.ascontiguousarray(smap.sector_heights, dtype=np.float32),
        sector_lights=np.ascontiguousarray(smap.sector_lights).astype(np.float32),
        sector_floor_tex=np.ascontiguousarray(smap.sector_floor_texture_ids, dtype=np.int32),
        sector_ceil_tex=np.ascontiguousarray(smap.sector_ceiling_texture_ids, dtype=np.int32),
        tex_atlas=tex_atlas,
        tex_w=tex_w,
        tex_h=tex_h,
        playpal=np.ascontiguousarray(smap.playpal, dtype=np.uint8),
        colormap=np.ascontiguousarray(smap.colormap, dtype=np.uint8),
        spr_atlas=spr_atlas,
        spr_opaque=spr_opaque,
        spr_post_top=spr_post_top,
        spr_w=np.ascontiguousarray(smap.sprite_widths, dtype=np.int32),
        spr_h=np.ascontiguousarray(smap.sprite_heights, dtype=np.int32),
        spr_left=np.ascontiguousarray(smap.sprite_left_offsets, dtype=np.int32),
        spr_top=np.ascontiguousarray(smap.sprite_top_offsets, dtype=np.int32),
        **build_blend_tables(smap),
    )


GRID_CELL = 64.0
GRID_PAD = 0.5
GRID_ALWAYS_INSIDE = 1 << 30  # flag on a grid item: every point of the cell is inside that sector


def _segments_near_boxes(segments: np.ndarray, x0, y0, x1, y1) -> np.ndarray:
    """For every axis-aligned box (``x0..y1`` broadcast against each other with a trailing axis of length one): does
    some segment [x1,y1,x2,y2] intersect it (Liang-Barsky clip)?  Returns the boxes' shape without the trailing axis."""

    px, py = segments[:, 0], segments[:, 1]
    dx, dy = segments[:, 2] - px, segments[:, 3] - py
    t0, t1, alive = 0.0, 1.0, True
    for p, q in ((-dx, px - x0), (dx, x1 - px), (-dy, py - y0), (dy, y1 - py)):
        parallel = p == 0
        alive = alive & ~(parallel & (q < 0))
        with np.errstate(divide="ignore", invalid="ignore"):
            r = np.where(parallel, 0.0, q / np.where(parallel, 1.0, p))
        t0 = np.where((p < 0) & ~parallel, np.maximum(t0, r), t0)
        t1 = np.where((p > 0) & ~parallel, np.minimum(t1, r), t1)
    return np.any(alive & (t0 <= t1), axis=-1)


def _points_in_polygon(segments: np.ndarray, x, y) -> np.ndarray:
    """Even-odd test of the points (``x``, ``y`` broadcast, trailing axis of length one) against the segments."""

    x1, y1, x2, y2 = segments[:, 0], segments[:, 1], segments[:, 2], segments[:, 3]
    crosses = (y1 > y) != (y2 > y)
    with np.errstate(divide="ignore", invalid="ignore"):
        crossing_x = x1 + (y - y1) * (x2 - x1) / np.where(y2 == y1, 1.0, y2 - y1)
    return (np.count_nonzero(crosses & (x < crossing_x), axis=-1) & 1).astype(bool)


FINE_CELL = 8.0
FINE_PER_COARSE = 8         # the coarse grid cell is this many fine cells wide, same origin
FINE_MAX_CELLS = 1 << 21
FINE_EMPTY = 0x40000000     # fine cell wholly outside every sector
FINE_MIXED = 0x80000000     # crossing test needed; bits 0..14 / 15..29 = floor / ceiling levels that can win there
FINE_UNKNOWN = 0xC0000000   # crossing test needed, nothing known about the levels
FINE_MASK_LEVELS = 15


def closed_boundaries(walls, sector_edge_ofs, sector_edge_idx, sector_count: int) -> np.ndarray:
    """bool [S]: is the sector's boundary a set of closed loops (every vertex touched by an even number of its edges)?"""

    counts = np.diff(sector_edge_ofs[: sector_count + 1])
    sector = np.repeat(np.arange(sector_count), counts)
    edges = np.asarray(sector_edge_idx[: sector_edge_ofs[sector_count]], dtype=np.int64)
    segments = np.asarray(walls)[edges]
    owner = np.concatenate([sector, sector])
    x = np.concatenate([segments[:, 0], segments[:, 2]]) + 0.0   # + 0.0: -0.0 and 0.0 are one vertex
    y = np.concatenate([segments[:, 1], segments[:, 3]]) + 0.0
    order = np.lexsort((y, x, owner))
    owner, x, y = owner[order], x[order], y[order]
    starts = np.ones(len(owner), dtype=bool)
    starts[1:] = (owner[1:] != owner[:-1]) | (x[1:] != x[:-1]) | (y[1:] != y[:-1])
    run_start = np.nonzero(starts)[0]
    run_length = np.diff(np.concatenate([run_start, [len(owner)]]))
    odd = np.zeros(sector_count, dtype=bool)
    np.logical_or.at(odd, owner[run_start], run_length % 2 == 1)
    return ~odd


def fine_cell_size(walls) -> float:
    """Fine raster cell: FINE_CELL map units, doubled until the raster stays below FINE_MAX_CELLS."""

    walls64 = np.asarray(walls, dtype=np.float64)
    width = float(walls64[:, (0, 2)].max() - walls64[:, (0, 2)].min()) + 4 * GRID_PAD + 1
    height = float(walls64[:, (1, 3)].max() - walls64[:, (1, 3)].min()) + 4 * GRID_PAD + 1
    cell = FINE_CELL
    while (np.ceil(width / cell) + 1) * (np.ceil(height / cell) + 1) > FINE_MAX_CELLS:
        cell *= 2.0
    return cell


def build_fine_grid(walls, sector_edge_ofs, sector_edge_idx, sector_count, min_x: float, min_y: float, cell: float,
                    sector_heights, floor_levels, ceil_levels) -> dict:
    """Fine raster of the even-odd point location (``engine.py:9598-9617``, ``10994-11015``).

    A cell that no linedef comes within ``GRID_PAD`` of is wholly inside or wholly outside
    each sector, and the float32 crossing test agrees with exact geometry there (its error is
    orders of magnitude below the pad).  Such a cell stores the one sector that contains its
    centre (with the indices of its floor and ceiling in the level lists), or ``FINE_EMPTY``.  Every other cell is ``FINE_MIXED`` and the caller falls back to
    the crossing test; it carries the plane levels of the sectors that can contain one of its
    points (those with an edge near the cell or containing its centre), so a probe for any other
    level is a miss without testing.  The raster shares its origin with the coarse grid.
    """

    walls64 = np.asarray(walls, dtype=np.float64)
    max_x = float(walls64[:, (0, 2)].max()) + 2 * GRID_PAD
    max_y = float(walls64[:, (1, 3)].max()) + 2 * GRID_PAD
    nx = int(np.ceil((max_x - min_x) / cell)) + 1
    ny = int(np.ceil((max_y - min_y) / cell)) + 1
    masks_known = len(floor_levels) <= FINE_MASK_LEVELS and len(ceil_levels) <= FINE_MASK_LEVELS
    mixed = np.zeros((ny, nx), dtype=bool)
    level_bits = np.zeros((ny, nx), dtype=np.uint32)
    owners = np.zeros((ny, nx), dtype=np.int32)
    owner = np.full((ny, nx), FINE_EMPTY, dtype=np.uint32)
    sector_bits = np.zeros(sector_count, dtype=np.uint32)
    sector_level_index = np.full(sector_count, 0xFF << 16, dtype=np.uint32)  # decided cells: floor / ceiling level index in bits 16..19 / 20..23, 15 = unknown
    if masks_known:
        # position of each sector's height in the level lists (at most FINE_MASK_LEVELS entries, in the caller's order)
        floor_index = np.argmax(np.asarray(floor_levels)[None, :] == sector_heights[:, 0:1], axis=1).astype(np.uint32)
        ceil_index = np.argmax(np.asarray(ceil_levels)[None, :] == sector_heights[:, 1:2], axis=1).astype(np.uint32)
        sector_bits = (np.uint32(1) << floor_index) | (np.uint32(1) << (np.uint32(FINE_MASK_LEVELS) + ceil_index))
        sector_level_index = (floor_index << np.uint32(16)) | (ceil_index << np.uint32(20))
    closed_sector = closed_boundaries(walls64, sector_edge_ofs, sector_edge_idx, sector_count)
    edge_counts = np.diff(sector_edge_ofs)
    pair_sector = np.repeat(np.arange(sector_count), edge_counts)       # one entry per (sector, edge of its boundary)
    pair_edge = np.asarray(sector_edge_idx[: sector_edge_ofs[sector_count]], dtype=np.int64)
    in_closed = closed_sector[pair_sector]

    # cells that an edge of a closed sector comes near: every (edge, cell of its padded bounding box) at once
    edges = np.unique(pair_edge[in_closed])
    x1, y1, x2, y2 = (walls64[edges, k] for k in range(4))
    ex0 = np.maximum(np.floor((np.minimum(x1, x2) - GRID_PAD - min_x) / cell).astype(np.int64), 0)
    ex1 = np.minimum(np.floor((np.maximum(x1, x2) + GRID_PAD - min_x) / cell).astype(np.int64), nx - 1)
    ey0 = np.maximum(np.floor((np.minimum(y1, y2) - GRID_PAD - min_y) / cell).astype(np.int64), 0)
    ey1 = np.minimum(np.floor((np.maximum(y1, y2) + GRID_PAD - min_y) / cell).astype(np.int64), ny - 1)
    box_w, box_h = np.maximum(ex1 - ex0 + 1, 0), np.maximum(ey1 - ey0 + 1, 0)
    box_cells = box_w * box_h
    box_start = np.concatenate([[0], np.cumsum(box_cells)])
    of_edge = np.repeat(np.arange(len(edges)), box_cells)               # which edge each listed cell belongs to
    local = np.arange(box_start[-1]) - box_start[of_edge]
    cell_y = ey0[of_edge] + local // np.maximum(box_w[of_edge], 1)
    cell_x = ex0[of_edge] + local % np.maximum(box_w[of_edge], 1)
    # Liang-Barsky clip of the segment against the padded cell box; an edge along an axis, or whose box is one cell
    # wide or high, is near every cell of its box
    trivial = (ex0 == ex1) | (ey0 == ey1) | (x1 == x2) | (y1 == y2)
    bx0 = min_x + cell_x * cell - GRID_PAD
    by0 = min_y + cell_y * cell - GRID_PAD
    bx1 = bx0 + cell + 2 * GRID_PAD
    by1 = by0 + cell + 2 * GRID_PAD
    dx, dy = (x2 - x1)[of_edge], (y2 - y1)[of_edge]
    with np.errstate(divide="ignore", invalid="ignore"):
        tx_a, tx_b = (bx0 - x1[of_edge]) / dx, (bx1 - x1[of_edge]) / dx
        ty_a, ty_b = (by0 - y1[of_edge]) / dy, (by1 - y1[of_edge]) / dy
        t_in = np.maximum(np.maximum(np.minimum(tx_a, tx_b), np.minimum(ty_a, ty_b)), 0.0)
        t_out = np.minimum(np.minimum(np.maximum(tx_a, tx_b), np.maximum(ty_a, ty_b)), 1.0)
        near = trivial[of_edge] | (t_in <= t_out)
    near_flat = (cell_y * nx + cell_x)[near]
    near_edge = of_edge[near]
    mixed.reshape(-1)[near_flat] = True
    if masks_known:
        # the levels of both sectors an edge bounds (closed ones) reach every cell the edge comes near
        edge_slot = np.full(len(walls64), -1, dtype=np.int64)
        edge_slot[edges] = np.arange(len(edges))
        edge_bits = np.zeros(len(edges), dtype=np.uint32)
        np.bitwise_or.at(edge_bits, edge_slot[pair_edge[in_closed]], sector_bits[pair_sector[in_closed]])
        np.bitwise_or.at(level_bits.reshape(-1), near_flat, edge_bits[near_edge])

    for s in range(sector_count):
        edges = sector_edge_idx[sector_edge_ofs[s] : sector_edge_ofs[s + 1]]
        if len(edges) == 0:
            continue
        bits, level_index = sector_bits[s], sector_level_index[s]
        seg = walls64[edges]
        closed = bool(closed_sector[s])
        ix0 = 0 if not closed else max(int(np.floor((seg[:, (0, 2)].min() - GRID_PAD - min_x) / cell)), 0)
        ix1 = min(int(np.floor((seg[:, (0, 2)].max() + GRID_PAD - min_x) / cell)), nx - 1)
        iy0 = max(int(np.floor((seg[:, (1, 3)].min() - GRID_PAD - min_y) / cell)), 0)
        iy1 = min(int(np.floor((seg[:, (1, 3)].max() + GRID_PAD - min_y) / cell)), ny - 1)
        if ix1 < ix0 or iy1 < iy0:
            continue
        if not closed:  # an open boundary can give odd parity anywhere to its left
            mixed[iy0 : iy1 + 1, ix0 : ix1 + 1] = True
            level_bits[iy0 : iy1 + 1, ix0 : ix1 + 1] |= bits
            continue
        # cells whose centre the sector contains
        cx = (min_x + (np.arange(ix0, ix1 + 1) + 0.5) * cell)[None, :, None]
        cy = (min_y + (np.arange(iy0, iy1 + 1) + 0.5) * cell)[:, None, None]
        inside = _points_in_polygon(seg, cx, cy)
        view_owners = owners[iy0 : iy1 + 1, ix0 : ix1 + 1]
        view_owner = owner[iy0 : iy1 + 1, ix0 : ix1 + 1]
        view_owner[inside & (view_owners == 0)] = np.uint32(s) | level_index
        view_owners += inside
        level_bits[iy0 : iy1 + 1, ix0 : ix1 + 1] |= np.where(inside, bits, np.uint32(0))
    mixed |= owners > 1
    owner[mixed] = (np.uint32(FINE_MIXED) | level_bits[mixed]) if masks_known else np.uint32(FINE_UNKNOWN)
    return dict(fine_nx=nx, fine_ny=ny, fine_cell=float(cell), fine_sector=np.ascontiguousarray(owner.reshape(-1)))


def build_sector_grid(walls, sector_edge_ofs, sector_edge_idx, sector_count, cell: float = GRID_CELL) -> dict:
    """Uniform grid of candidate (sector, edge sub-list) pairs for the even-odd polygon test.

    The reference tests a point against every edge of every sector
    (``engine.py:9598-9617`` and ``engine.py:10994-11015``).  An edge can only be
    counted for a point ``(px, py)`` when ``py`` lies between its endpoints' y and
    ``px < crossing_x <= max(x1, x2)`` (up to float32 rounding, covered by the
    pad), and a sector whose boundary is a set of closed loops can only have odd
    parity when ``px`` is not left of all its edges.  A cell therefore lists, per
    sector whose padded bounding box meets it, exactly the edges that can be
    counted for points inside the cell; the parity over that sub-list equals the
    parity over the full edge list.  Sectors with an open boundary are treated
    as unbounded on the left.
    """

    all_x = walls[:, (0, 2)]
    all_y = walls[:, (1, 3)]
    min_x = float(np.floor(all_x.min() - 2 * GRID_PAD))
    min_y = float(np.floor(all_y.min() - 2 * GRID_PAD))
    nx = int(np.ceil((float(all_x.max()) + 2 * GRID_PAD - min_x) / cell)) + 1
    ny = int(np.ceil((float(all_y.max()) + 2 * GRID_PAD - min_y) / cell)) + 1
    closed_sector = closed_boundaries(walls, sector_edge_ofs, sector_edge_idx, sector_count)
    item_cells, item_sectors, item_counts, item_edge_lists = [], [], [], []
    for s in range(sector_count):
        edges = sector_edge_idx[sector_edge_ofs[s] : sector_edge_ofs[s + 1]]
        if len(edges) == 0:
            continue
        ex = walls[edges][:, (0, 2)]
        ey = walls[edges][:, (1, 3)]
        closed = bool(closed_sector[s])
        sx0 = -np.inf if not closed else float(ex.min()) - GRID_PAD
        sx1 = float(ex.max()) + GRID_PAD
        sy0 = float(ey.min()) - GRID_PAD
        sy1 = float(ey.max()) + GRID_PAD
        ix0 = 0 if not closed else max(int(np.floor((sx0 - min_x) / cell)), 0)
        ix1 = min(int(np.floor((sx1 - min_x) / cell)), nx - 1)
        iy0 = max(int(np.floor((sy0 - min_y) / cell)), 0)
        iy1 = min(int(np.floor((sy1 - min_y) / cell)), ny - 1)
        if ix1 < ix0 or iy1 < iy0:
            continue
        edge_max_x = ex.max(axis=1)
        edge_min_y = ey.min(axis=1)
        edge_max_y = ey.max(axis=1)
        segments = walls[edges].astype(np.float64)
        # every cell of the sector's box at once: [rows, columns, edges]
        columns = np.arange(ix0, ix1 + 1)
        rows = np.arange(iy0, iy1 + 1)
        cx0 = np.where(columns > 0, min_x + columns * cell - GRID_PAD, -np.inf)[None, :, None]
        cx1 = (min_x + (columns + 1) * cell + GRID_PAD)[None, :, None]
        cy0 = (min_y + rows * cell - GRID_PAD)[:, None, None]
        cy1 = (min_y + (rows + 1) * cell + GRID_PAD)[:, None, None]
        keep = ((edge_max_y[None, None, :] >= cy0) & (edge_min_y[None, None, :] <= cy1)) & (edge_max_x[None, None, :] >= cx0)
        # A cell that no edge of the sector comes near (padded by GRID_PAD, far more than the
        # float32 error of the crossing test) lies wholly inside or wholly outside the sector:
        # decide once at its centre and spare the kernels every edge test there.
        decided = np.zeros((len(rows), len(columns)), dtype=bool)
        inside = np.zeros_like(decided)
        if closed:
            first = 1 if ix0 == 0 else 0   # the leftmost column of the grid stands for everything to its left
            if len(columns) > first:
                decided[:, first:] = ~_segments_near_boxes(segments, cx0[:, first:], cy0, cx1[:, first:], cy1)
                centre_x = (min_x + (columns + 0.5) * cell)[None, :, None]
                centre_y = (min_y + (rows + 0.5) * cell)[:, None, None]
                inside = decided & _points_in_polygon(segments, centre_x, centre_y)
        # one item per cell that lists the sector: decided cells inside it (no edges), undecided cells (their sub-list)
        listed = ~decided | inside
        keep &= ~decided[:, :, None]
        cell_index = (rows[:, None] * nx + columns[None, :])[listed]
        item_cells.append(cell_index)
        item_sectors.append(np.where(inside[listed], s | GRID_ALWAYS_INSIDE, s))
        item_counts.append(np.count_nonzero(keep, axis=2)[listed])
        item_edge_lists.append(np.asarray(edges)[np.nonzero(keep)[2]])   # row-major over (row, column, edge): cell by cell
    # gather the items cell by cell; within a cell they stay in the order they were made, ascending by sector
    if item_cells:
        cells = np.concatenate(item_cells)
        order = np.argsort(cells, kind="stable")
        counts = np.concatenate(item_counts)
        starts = np.concatenate([[0], np.cumsum(counts)])[:-1]
        counts_sorted = counts[order]
        sorted_starts = np.concatenate([[0], np.cumsum(counts_sorted)])
        gather = np.repeat(starts[order], counts_sorted) + (np.arange(sorted_starts[-1]) - np.repeat(sorted_starts[:-1], counts_sorted))
        item_edges = np.concatenate(item_edge_lists)[gather]
        item_sector = np.concatenate(item_sectors)[order]
        item_edge_ofs = sorted_starts
        cell_ofs = np.concatenate([[0], np.cumsum(np.bincount(cells, minlength=nx * ny))]).astype(np.int32)
    else:
        item_edges, item_sector, item_edge_ofs = np.zeros(0, np.int64), np.zeros(0, np.int64), np.zeros(1, np.int64)
        cell_ofs = np.zeros(nx * ny + 1, dtype=np.int32)
    return dict(
        grid_nx=nx,
        grid_ny=ny,
        grid_min_x=min_x,
        grid_min_y=min_y,
        grid_cell=float(cell),
        grid_cell_ofs=cell_ofs,
        grid_item_sector=np.asarray(item_sector if len(item_sector) else [0], dtype=np.int32),  # | GRID_ALWAYS_INSIDE
        grid_item_edge_ofs=np.asarray(item_edge_ofs, dtype=np.int32),
        grid_item_edges=np.asarray(item_edges if len(item_edges) else [0], dtype=np.int32),
    )
