from __future__ import annotations

import ast
import functools
import glob
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import __graft_entry__ as entry  # noqa: E402

entry.load_package()

FIXTURE_DIR = os.path.join(ROOT, "tests", "golden", "fixtures")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def fixture_names():
    return sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(FIXTURE_DIR, "*.npz")))


@functools.lru_cache(maxsize=None)
def load_fixture(name: str):
    """Return (meta, data, smap, tables) for a golden case; the map is regenerated from its seed."""

    from gradoom_amd import mapbuild, synthmap

    sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
    from make_golden_meta import fragment_digest, map_digest

    data = dict(np.load(os.path.join(FIXTURE_DIR, f"{name}.npz")))
    meta = ast.literal_eval(str(data.pop("meta")))
    if meta.get("recipe"):   # a case of tests/random_cases.py
        import random_cases

        smap = random_cases.build_parts(meta["recipe"], meta["lanes"])[0]
        assert map_digest(smap) == meta["map_sha256"], "random case generator drifted from the golden fixtures"
        return meta, data, smap, mapbuild.build_map_tables(smap)
    smap = synthmap.generate_map(
        meta["map_seed"], grid=tuple(meta["grid"]), sectors=meta["sectors"], linedefs=meta["linedefs"],
        midtex=meta.get("midtex", 0.0), layout=meta.get("layout", "grid"), islands=meta.get("islands", 0),
        pillars=meta.get("pillars", 0),
    )
    assert map_digest(smap) == meta["map_sha256"], "synthetic map generator drifted from the golden fixtures"
    if meta.get("variant"):
        smap = synthmap.with_variant(smap, **meta["variant"])
        assert map_digest(smap) == meta["variant_sha256"], "map variant generator drifted from the golden fixtures"
    if meta.get("blend_seed"):
        smap = synthmap.with_blend_tables(smap, meta["blend_seed"])
    if meta.get("split_seed"):
        smap = synthmap.split_linedefs(smap, meta["split_seed"])
        assert fragment_digest(smap) == meta["fragment_sha256"], "linedef splitter drifted from the golden fixtures"
    tables = mapbuild.build_map_tables(smap)
    return meta, data, smap, tables


LANE_KEYS = (
    "x", "y", "angle", "view_z", "x_fixed", "y_fixed", "angle_bam", "pitch_bam", "flash_light", "ray_cos", "ray_sin",
    "sprite_x", "sprite_y", "sprite_z", "sprite_depth", "sprite_id", "sprite_alive", "sprite_fullbright",
    "weapon_state", "hud_state", "sprite_style", "screen_blend", "decal_state", "decal_geom",
)


def fixture_overlays(meta: dict):
    """The seeded weapon / status bar patches of a case that has them, else None."""

    from gradoom_amd import synthmap

    return synthmap.generate_overlays(meta["overlays"]) if meta.get("overlays") else None


def lane_inputs(data: dict) -> dict:
    return {key: data[key] for key in LANE_KEYS if key in data}


@pytest.fixture(scope="session")
def oracle():
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as oracle_module

    oracle_module.library()
    return oracle_module
