"""The golden fixtures must actually exercise the ownership rules of the wall traversal."""

from __future__ import annotations

from conftest import fixture_names, lane_inputs, load_fixture

# Rules the reference-rendered fixtures are known to fire at least once (engine.py:11768-13371).
EXERCISED = (
    "projected_solid", "endpoint_owner", "near_projected", "topological_owner", "opposing_boundary", "excluded_right_edge",
    "continues_owner_boundary", "forward_bridge", "completes_endpoint_bridge", "endpoint_only_portal", "enters_other",
    "enters_shared", "geometric_path", "portal_bridge", "completes_portal_bridge", "ps_keeps_path", "no_keeps_path",
    "bottom_tail", "masked_column", "masked_extends", "dead_column_revived", "equal_depth_solid", "solid_bridge",
    "sector_bridge", "tied_strip",
)
# Rules no fixture reaches; parity of such branches would rest on reading alone.
NOT_EXERCISED = ()


def test_fixture_set_fires_the_listed_rules(oracle):
    oracle.coverage(reset=True)
    for name in fixture_names():
        meta, data, _smap, tables = load_fixture(name)
        lanes = min(meta["lanes"], 4 if "subset" in name else meta["lanes"])
        oracle.render(tables, lane_inputs(data), data["cosine_correction"], lane_range=(0, lanes))
    counts = oracle.coverage(reset=True)
    missing = [rule for rule in EXERCISED if counts[rule] == 0]
    assert not missing, f"rules no longer exercised by the fixtures: {missing}"
    newly = [rule for rule in NOT_EXERCISED if counts[rule] > 0]
    assert not newly, f"rules now exercised, move them to EXERCISED: {newly}"


def test_one_fixture_takes_the_general_endpoint_neighbour_search():
    """Every other case has at most one neighbour per endpoint and uses the direct tables (engine.py:1558-1577)."""

    _meta, _data, _smap, tables = load_fixture("pinched_pillars")
    assert tables["direct_neighbors"] == 0 and tables["neighbor_slots"] >= 3
    _meta, _data, _smap, tables = load_fixture("config1")
    assert tables["direct_neighbors"] == 1
