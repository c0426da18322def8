"""Derived map tables (mapbuild + the on-the-fly relations) against the reference's own tables."""

from __future__ import annotations

import numpy as np
import pytest

from conftest import load_fixture

CASES = ["tiny_stages", "small_midtex_sprites"]


@pytest.mark.parametrize("name", CASES)
def test_compact_tables_equal_reference(name):
    _meta, data, _smap, tables = load_fixture(name)
    walls = tables["wall_count"]
    assert np.array_equal(tables["wall_len"], data["ref_wall_lengths"])
    assert np.array_equal(tables["walls_fixed"].astype(np.int64), data["ref_walls_fixed"])
    assert np.array_equal(tables["blocking_walls"], data["ref_blocking_wall_indices"])
    assert np.array_equal(tables["sector_lights"], data["ref_sector_lights"])
    assert bool(tables["direct_neighbors"]) == bool(data["ref_direct_neighbors"])
    # endpoint neighbours: same compact [W,K] layout, ascending, self-padded (engine.py:833-849)
    assert np.array_equal(tables["endpoint_neighbors"], data["ref_endpoint_neighbors"])
    assert np.array_equal(tables["endpoint_neighbor_starts"].astype(bool), data["ref_endpoint_neighbor_starts"])
    assert np.array_equal(tables["endpoint_neighbor_ends"].astype(bool), data["ref_endpoint_neighbor_ends"])
    # solid bridges: CSR rows equal the masked prefix of the reference's padded rows (engine.py:811-830)
    for side in ("start", "end"):
        ofs, idx = tables[f"solid_bridge_{side}_ofs"], tables[f"solid_bridge_{side}_idx"]
        ref_idx, ref_mask = data[f"ref_solid_bridge_{side}_indices"], data[f"ref_solid_bridge_{side}_mask"]
        for w in range(walls):
            ours = idx[ofs[w] : ofs[w + 1]].tolist()
            assert ours == ref_idx[w][ref_mask[w]].tolist()
            assert not ref_mask[w][len(ours) :].any()


@pytest.mark.parametrize("name", CASES)
def test_on_the_fly_relations_equal_reference_dense_tables(oracle, name):
    _meta, data, _smap, tables = load_fixture(name)
    ours = oracle.relation_tables(tables)
    assert np.array_equal(ours["same_pair"].astype(bool), data["ref_same_pair"])
    assert np.array_equal(ours["opposing"].astype(bool), data["ref_opposing"])
    for kind in ("portal", "sector"):
        mask = ours[f"{kind}_bridge_mask"].astype(bool)
        assert np.array_equal(mask, data[f"ref_{kind}_bridge_mask"])
        assert np.array_equal(ours[f"{kind}_bridge_index"], data[f"ref_{kind}_bridge_index"])


def test_sector_grid_lists_every_edge_that_can_count():
    # brute force: for random points, parity over the cell's edge sub-list == parity over the full edge list
    _meta, _data, smap, tables = load_fixture("small_midtex_sprites")
    rng = np.random.default_rng(1)
    walls = tables["walls"]
    lo = walls[:, (0, 2)].min() - 50, walls[:, (1, 3)].min() - 50
    hi = walls[:, (0, 2)].max() + 50, walls[:, (1, 3)].max() + 50
    nx, ny = tables["grid_nx"], tables["grid_ny"]

    def parity(edges, px, py):
        count = 0
        for w in edges:
            x1, y1, x2, y2 = (np.float32(v) for v in walls[w])
            dy = np.float32(y2 - y1)
            safe = np.float32(1.0) if abs(dy) < 1e-6 else dy
            crossing = np.float32(x1 + np.float32(np.float32(np.float32(py - y1) * np.float32(x2 - x1)) / safe))
            if ((y1 > py) != (y2 > py)) and px < crossing:
                count += 1
        return count & 1

    for _ in range(1500):
        px = np.float32(rng.uniform(lo[0], hi[0]))
        py = np.float32(rng.uniform(lo[1], hi[1]))
        fx = np.floor(np.float32(np.float32(px - np.float32(tables["grid_min_x"])) / np.float32(tables["grid_cell"])))
        fy = np.floor(np.float32(np.float32(py - np.float32(tables["grid_min_y"])) / np.float32(tables["grid_cell"])))
        listed = {}
        if 0 <= fy < ny and fx < nx:
            cell = int(fy) * nx + max(int(fx), 0)
            for item in range(tables["grid_cell_ofs"][cell], tables["grid_cell_ofs"][cell + 1]):
                e0, e1 = tables["grid_item_edge_ofs"][item], tables["grid_item_edge_ofs"][item + 1]
                entry = int(tables["grid_item_sector"][item])
                listed[entry & ~(1 << 30)] = None if entry & (1 << 30) else tables["grid_item_edges"][e0:e1]
        for s in range(tables["sector_count"]):
            full = tables["sector_edge_idx"][tables["sector_edge_ofs"][s] : tables["sector_edge_ofs"][s + 1]]
            expected = parity(full, px, py)
            got = (1 if listed[s] is None else parity(listed[s], px, py)) if s in listed else 0
            assert got == expected


@pytest.mark.parametrize("fixture", ["small_midtex_sprites", "brick_islands"])
def test_fine_raster_agrees_with_the_crossing_test(fixture):
    # every decided cell of the fine raster must name exactly the set of sectors with odd float32 parity;
    # points are drawn uniformly and also snapped close to linedefs, where a wrong "decided" cell would show
    _meta, _data, smap, tables = load_fixture(fixture)
    rng = np.random.default_rng(2)
    walls = tables["walls"].astype(np.float32)
    S = tables["sector_count"]
    count = 6000
    px = rng.uniform(walls[:, (0, 2)].min() - 30, walls[:, (0, 2)].max() + 30, count)
    py = rng.uniform(walls[:, (1, 3)].min() - 30, walls[:, (1, 3)].max() + 30, count)
    pick = rng.integers(0, len(walls), count // 2)
    t = rng.uniform(0, 1, count // 2)
    px[: count // 2] = walls[pick, 0] + t * (walls[pick, 2] - walls[pick, 0]) + rng.uniform(-1.5, 1.5, count // 2)
    py[: count // 2] = walls[pick, 1] + t * (walls[pick, 3] - walls[pick, 1]) + rng.uniform(-1.5, 1.5, count // 2)
    px, py = px.astype(np.float32), py.astype(np.float32)
    inv = np.float32(1.0) / np.float32(tables["fine_cell"])
    fx = np.floor((px - np.float32(tables["grid_min_x"])) * inv)
    fy = np.floor((py - np.float32(tables["grid_min_y"])) * inv)
    inside_raster = (fx >= 0) & (fx < tables["fine_nx"]) & (fy >= 0) & (fy < tables["fine_ny"])
    entry = np.full(count, 0xC0000000, dtype=np.int64)
    entry[inside_raster] = tables["fine_sector"][fy[inside_raster].astype(int) * tables["fine_nx"] + fx[inside_raster].astype(int)]
    kind = entry >> 30
    parity = np.zeros((count, S), dtype=bool)
    for s in range(S):
        e = walls[tables["sector_edge_idx"][tables["sector_edge_ofs"][s] : tables["sector_edge_ofs"][s + 1]]]
        x1, y1, x2, y2 = (e[:, k][None, :] for k in range(4))
        dy = y2 - y1
        safe = np.where(np.abs(dy) < 1e-6, np.float32(1.0), dy)
        crossing = x1 + (py[:, None] - y1) * (x2 - x1) / safe
        assert crossing.dtype == np.float32
        parity[:, s] = np.count_nonzero(((y1 > py[:, None]) != (y2 > py[:, None])) & (px[:, None] < crossing), axis=1) & 1
    decided = kind <= 1
    assert decided.mean() > 0.3  # the raster must actually decide a good share of the points
    empty = kind == 1
    assert not parity[empty].any()
    owned = kind == 0
    assert np.array_equal(parity[owned].sum(axis=1), np.ones(owned.sum(), dtype=int))
    assert np.array_equal(parity[owned].argmax(axis=1), entry[owned] & 0xFFFF)
    sector_of = entry[owned] & 0xFFFF
    assert np.array_equal(tables["floor_levels"][(entry[owned] >> 16) & 15], tables["sector_heights"][sector_of, 0])
    assert np.array_equal(tables["ceil_levels"][(entry[owned] >> 20) & 15], tables["sector_heights"][sector_of, 1])
    # undecided cells with level masks: every sector that contains the point has its levels flagged
    heights = tables["sector_heights"]
    floor_index = {float(v): k for k, v in enumerate(tables["floor_levels"])}
    ceil_index = {float(v): k for k, v in enumerate(tables["ceil_levels"])}
    masked = np.nonzero(kind == 2)[0]
    assert len(masked) > 100
    for i in masked:
        for s in np.nonzero(parity[i])[0]:
            assert (entry[i] >> floor_index[float(heights[s, 0])]) & 1
            assert (entry[i] >> (15 + ceil_index[float(heights[s, 1])])) & 1
    assert tables["grid_cell"] == 8 * tables["fine_cell"]


def test_split_tables_hold_only_linedefs_whose_fragments_differ_from_the_linedef():
    """scenario.py:420-454: every linedef has a fragment row; only split ones need a row on the device."""

    import dataclasses

    import pytest

    from gradoom_amd import mapbuild, synthmap

    smap = synthmap.generate_map(7, grid=(4, 3), sectors=10, linedefs=48)
    plain = mapbuild.build_map_tables(smap)
    assert plain["split_count"] == 0 and plain["fragment_slots"] == 1
    assert np.all(plain["wall_split_slot"] == -1)

    split = synthmap.split_linedefs(smap, 5, share=0.3)
    tables = mapbuild.build_map_tables(split)
    mask = split.wall_projection_fragment_mask
    expected_rows = np.flatnonzero(mask.sum(axis=1) > 1)
    assert tables["split_count"] == len(expected_rows) > 0
    assert tables["fragment_slots"] == mask.shape[1]
    assert np.array_equal(np.flatnonzero(tables["wall_split_slot"] >= 0), expected_rows)
    for row, w in enumerate(expected_rows):
        assert tables["wall_split_slot"][w] == row
        assert np.array_equal(tables["split_fragments_fixed"][row], split.wall_projection_fragments_fixed[w])
        assert np.array_equal(tables["split_fragment_mask"][row].astype(bool), mask[w])
        pieces = split.wall_projection_fragments_fixed[w][mask[w]]
        # consecutive fragments chain from the linedef's start to its end
        assert np.array_equal(pieces[0, :2], tables["walls_fixed"][w, :2])
        assert np.array_equal(pieces[-1, 2:], tables["walls_fixed"][w, 2:])
        assert np.array_equal(pieces[1:, :2], pieces[:-1, 2:])

    # a single fragment that is not the linedef itself still needs its row; so does a linedef with none
    moved = dataclasses.replace(
        smap,
        wall_projection_fragments_fixed=tables["walls_fixed"].astype(np.int64)[:, None, :] + np.asarray([0, 0, 0, 1])[None, None, :] * (np.arange(len(tables["walls_fixed"])) == 3)[:, None, None],
        wall_projection_fragment_mask=(np.arange(len(tables["walls_fixed"])) != 5)[:, None],
    )
    rows = mapbuild.build_map_tables(moved)
    assert rows["split_count"] == 2
    assert list(np.flatnonzero(rows["wall_split_slot"] >= 0)) == [3, 5]

    with pytest.raises(ValueError):
        mapbuild.build_map_tables(dataclasses.replace(smap, wall_projection_fragments_fixed=np.zeros((48, 1, 4), np.int64)))


def test_closed_doors_and_ceilings_below_floors_build():
    """The reference puts no order on a sector's two heights (``scenario.py:302-401``): closed doors (ceiling == floor)
    and ceilings below floors build, and each height finds its own plane level."""
    from gradoom_amd import mapbuild, synthmap

    smap = synthmap.generate_map(5, grid=(3, 3), sectors=8, linedefs=80, layout="grid", islands=2, pillars=1)
    smap.sector_heights[2, 1] = smap.sector_heights[2, 0]
    mapbuild.build_map_tables(smap)
    smap.sector_heights[2, 1] = smap.sector_heights[2, 0] - 16
    tables = mapbuild.build_map_tables(smap)
    assert smap.sector_heights[2, 1] in tables["ceil_levels"] and smap.sector_heights[2, 0] in tables["floor_levels"]


def test_pose_generator_refuses_a_map_with_no_room_to_stand():
    # every sector lower than a standing camera: the generator says so instead of drawing sectors for ever
    from gradoom_amd import synthmap

    smap = synthmap.generate_map(3, grid=(3, 3), sectors=8, linedefs=80)
    smap.sector_heights[:, 1] = smap.sector_heights[:, 0] + 40.0
    with pytest.raises(ValueError, match="high enough"):
        synthmap.generate_poses(smap, 2, 1)
