"""actor_inputs.pack_actors on the gameplay tensors the ``actors`` golden case stores.

The case's frames were rendered by the reference from those tensors, and the oracle and the HIP path reproduce
them from the packed list (test_oracle_golden, test_gpu_parity); here the packing is re-run without the
reference and its list compaction is checked."""

from __future__ import annotations

import types

import numpy as np
import pytest
import torch

from conftest import lane_inputs, load_fixture


def stored_engine(data: dict):
    from gradoom_amd import actor_inputs

    engine = types.SimpleNamespace(**{field: torch.as_tensor(data[f"actor_engine_{field}"]) for field in actor_inputs.ENGINE_FIELDS})
    engine.map = types.SimpleNamespace(**{field: torch.as_tensor(data[f"actor_map_{field}"]) for field in actor_inputs.MAP_FIELDS})
    return engine


def test_packing_the_stored_gameplay_tensors_gives_the_list_the_reference_frames_were_checked_with():
    from gradoom_amd import actor_inputs

    _meta, data, _smap, _tables = load_fixture("actors")
    packed = actor_inputs.pack_actors(stored_engine(data))
    for key, value in packed.items():
        assert np.array_equal(value.numpy(), data[key]), key
    # monsters 64, start dolls 3, corpses 64, rockets/plasma 32, fireballs 64, their explosions 32 + 64,
    # teleport fog 64, bullet puffs 20, map items 24, drops 64
    assert packed["sprite_x"].shape[1] == 64 + 3 + 64 + 32 + 64 + 32 + 64 + 64 + 20 + 24 + 64
    alive = packed["sprite_alive"].bool()
    for style in (-2, -1, 0, 1):
        assert (alive & (packed["sprite_style"] == style)).any()
    assert (alive & packed["sprite_fullbright"].bool()).any()
    assert int(alive.sum(dim=1).min()) > 200


def test_cutting_the_list_keeps_live_actors_in_order(oracle):
    """A list longer than the renderer's slot limit is compacted on the device; live actors keep their order,
    so the picture (ties between equally distant sprites included) stays the reference's."""

    from gradoom_amd import actor_inputs, hostmath

    _meta, data, _smap, tables = load_fixture("actors")
    full = actor_inputs.pack_actors(stored_engine(data), limit=0)
    limit = 320
    assert int(full["sprite_alive"].sum(dim=1).max()) <= limit < full["sprite_alive"].shape[1]
    cut = actor_inputs.compact_actors(full, limit)
    assert cut["sprite_x"].shape[1] == limit
    for lane in range(full["sprite_alive"].shape[0]):
        alive, kept = full["sprite_alive"][lane].bool(), cut["sprite_alive"][lane].bool()
        assert torch.equal(full["sprite_x"][lane][alive], cut["sprite_x"][lane][kept])
        assert torch.equal(full["sprite_id"][lane][alive], cut["sprite_id"][lane][kept])
    arrays = lane_inputs(data)
    arrays.update({key: value.numpy() for key, value in cut.items()})
    arrays["sprite_depth"] = hostmath.sprite_depth(
        torch.as_tensor(data["x"]), torch.as_tensor(data["y"]), torch.as_tensor(data["angle"]), cut["sprite_x"], cut["sprite_y"]
    ).numpy()
    result = oracle.render(tables, arrays, data["cosine_correction"], lane_range=(0, 4))
    assert np.array_equal(result["indexed"][:4], data["indexed"][:4])


@pytest.mark.gpu
def test_fused_packing_kernel_gives_the_same_list_as_the_torch_ops():
    """gd_pack_actors against pack_actors (pinned by the reference's frames) on the stored tensors, tiled to
    many lanes with the cameras moved about so that every rotation and animation frame comes up."""

    from gradoom_amd import actor_inputs

    _meta, data, _smap, _tables = load_fixture("actors")
    engine = stored_engine(data)
    lanes = 512
    generator = torch.Generator().manual_seed(3)
    per_map = ("_enemy_walk_frame_tics", "_enemy_idle_frame_tics", "_enemy_attack_recovery", "_player_start_z", "_item_z")
    for field in actor_inputs.ENGINE_FIELDS:
        value = getattr(engine, field)
        if field not in per_map:
            value = value.repeat(lanes // value.shape[0], *([1] * (value.ndim - 1)))
        setattr(engine, field, value.to("cuda:0"))
    for field in actor_inputs.MAP_FIELDS:
        setattr(engine.map, field, getattr(engine.map, field).to("cuda:0"))
    engine.x = engine.x + (torch.rand(lanes, generator=generator) * 64 - 32).to("cuda:0")
    engine.y = engine.y + (torch.rand(lanes, generator=generator) * 64 - 32).to("cuda:0")
    engine.episode_time = torch.randint(0, 2000, (lanes,), generator=generator, dtype=torch.int32).to("cuda:0")
    engine.enemy_animation_tics = torch.randint(0, 400, engine.enemy_animation_tics.shape, generator=generator, dtype=torch.int32).to("cuda:0")
    for limit in (0, 512, 300):
        expected = actor_inputs.pack_actors(engine, limit=limit)
        fused = actor_inputs.pack_actors_fused(engine, limit=limit)
        torch.cuda.synchronize()
        assert set(fused) == set(expected)
        for key in expected:
            assert fused[key].dtype == expected[key].dtype and fused[key].shape == expected[key].shape, key
            assert torch.equal(fused[key], expected[key]), key
    # the first eight lanes before the cameras moved are the golden case itself
    assert int(expected["sprite_alive"].sum()) > 100 * lanes
