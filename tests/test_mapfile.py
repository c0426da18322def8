"""The on-disk map schema: what is written can be read back into the same map tables, and bad files are refused."""

from __future__ import annotations

import numpy as np
import pytest

from conftest import load_fixture


def test_round_trip_gives_the_same_map_tables(tmp_path):
    from gradoom_amd import mapbuild, mapfile

    for case in ("actors", "split_linedefs", "styled_sprites"):
        _meta, _data, smap, tables = load_fixture(case)
        path = str(tmp_path / f"{case}.npz")
        mapfile.save_map(path, smap)
        loaded = mapfile.load_map(path)
        rebuilt = mapbuild.build_map_tables(loaded)
        assert set(rebuilt) == set(tables)
        for key, value in tables.items():
            assert np.array_equal(np.asarray(rebuilt[key]), np.asarray(value)), (case, key)
        with np.load(path, allow_pickle=False) as stored:
            assert int(stored["map_schema_version"]) == mapfile.SCHEMA_VERSION
            for name, (dtype, _ndim, _trailing) in mapfile.REQUIRED.items():
                assert stored[name].dtype == np.dtype(dtype), name


def test_bad_files_are_refused(tmp_path):
    from gradoom_amd import mapfile

    _meta, _data, smap, _tables = load_fixture("tiny_stages")
    arrays = mapfile.scenario_arrays(smap)
    good = dict(map_schema_version=np.int32(mapfile.SCHEMA_VERSION), **arrays)

    def written(**changes):
        path = str(tmp_path / "case.npz")
        content = {k: v for k, v in {**good, **changes}.items() if v is not None}
        np.savez(path, **content)
        return path

    assert mapfile.load_map(written()).wall_segments.shape == smap.wall_segments.shape
    with pytest.raises(ValueError, match="not a map file"):
        mapfile.load_map(written(map_schema_version=None))
    with pytest.raises(ValueError, match="schema version 7"):
        mapfile.load_map(written(map_schema_version=np.int32(7)))
    with pytest.raises(ValueError, match="lacks sector_heights"):
        mapfile.load_map(written(sector_heights=None))
    with pytest.raises(ValueError, match="wall_sectors must be stored as int32"):
        mapfile.load_map(written(wall_sectors=arrays["wall_sectors"].astype(np.int64)))
    with pytest.raises(ValueError, match=r"wall_segments must have shape \[\?x4\]"):
        mapfile.load_map(written(wall_segments=arrays["wall_segments"][:, :3]))
    with pytest.raises(ValueError, match="sector_lights must hold one value per sector"):
        mapfile.load_map(written(sector_lights=arrays["sector_lights"][:-1]))
    with pytest.raises(ValueError, match="come together"):
        mapfile.load_map(written(wall_projection_fragment_mask=np.ones((len(arrays["wall_segments"]), 2), dtype=bool)))
    # an object array would need pickle to load: refused by numpy itself
    path = str(tmp_path / "pickled.npz")
    np.savez(path, **{**good, "playpal": np.array([{"a": 1}], dtype=object)})
    with pytest.raises(ValueError):
        mapfile.load_map(path)
    # values that do not fit the schema's integer types are not silently wrapped
    huge = smap.wall_sectors.astype(np.int64).copy()
    huge[0, 0] = 1 << 40
    view = type("Scenario", (), {})()
    for name in dir(smap):
        if not name.startswith("_"):
            try:
                setattr(view, name, getattr(smap, name))
            except AttributeError:
                pass
    view.wall_sectors = huge
    with pytest.raises(ValueError, match="wall_sectors does not fit int32"):
        mapfile.scenario_arrays(view)
