"""The vector-env front end on the real renderer (needs an MI355X)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import load_fixture

pytestmark = pytest.mark.gpu


def test_step_and_reset_device_matches_oracle_frame_by_frame(oracle):
    from gradoom_amd import hostmath
    from gradoom_amd.env import GraDoomVecEnv

    _meta, _data, smap, tables = load_fixture("small_midtex_sprites")
    lanes = 5
    env = GraDoomVecEnv(smap, lanes, device="cuda:0", render_mode="rgb_array", episode_timeout=2, sprites=16)
    cosine = env._renderer._cosine   # the renderer's own table (the GPU's float32 cosines, like its ray tables)

    def expected_obs():
        state = env._dynamics.lane_state()
        arrays = {}
        for name in ("x", "y", "angle", "view_z", "x_fixed", "y_fixed", "angle_bam", "pitch_bam", "flash_light",
                     "sprite_x", "sprite_y", "sprite_z", "sprite_id", "sprite_alive", "sprite_fullbright"):
            arrays[name] = getattr(state, name).cpu().numpy()
        # the env computes the float32 tables with Torch on the GPU; hand the oracle the same values
        ray_cos, ray_sin = hostmath.ray_tables(state.angle, env._renderer.ray_offsets)
        arrays["ray_cos"], arrays["ray_sin"] = ray_cos.cpu().numpy(), ray_sin.cpu().numpy()
        arrays["sprite_depth"] = hostmath.sprite_depth(state.x, state.y, state.angle, state.sprite_x, state.sprite_y).cpu().numpy()
        return oracle.render(tables, arrays, cosine)

    mask = torch.ones(lanes, dtype=torch.bool, device="cuda:0")
    seeds = torch.arange(lanes, device="cuda:0")
    obs, _signals = env.reset_device(mask, seeds)
    first = expected_obs()
    for k in range(4):
        assert np.array_equal(obs[:, k].cpu().numpy(), first["obs"])
    actions = torch.zeros(lanes, dtype=torch.int64, device="cuda:0")
    transition = env.step_and_reset_device(actions, seeds)
    second = expected_obs()
    assert np.array_equal(transition.observations[:, 3].cpu().numpy(), second["obs"])
    assert np.array_equal(transition.observations[:, 2].cpu().numpy(), first["obs"])
    assert not bool(transition.truncated.any())
    transition = env.step_and_reset_device(actions, seeds + 7)
    assert bool(transition.truncated.all())
    third = expected_obs()   # dynamics already reset: all four stack entries show the reset frame
    for k in range(4):
        assert np.array_equal(transition.observations[:, k].cpu().numpy(), third["obs"])
    assert not np.array_equal(transition.final_observations.cpu().numpy(), transition.observations.cpu().numpy())
    image = env.render()
    assert image.shape == (240, 320, 3)
    assert np.array_equal(image, np.asarray(tables["playpal"])[third["indexed"][0]])
    assert env._renderer.status() == 0
    env.close()


def test_host_api_safe_view_buffers_are_written_by_the_renderer():
    # reset()/step() hand out two buffers in turn (env.py:459-472, 678-688); they hold the stack, in either layout
    from gradoom_amd.env import GraDoomVecEnv

    _meta, _data, smap, _tables = load_fixture("small_midtex_sprites")
    lanes = 6
    actions = torch.zeros(lanes, dtype=torch.int64, device="cuda:0")
    for layout in ("chw", "hwc"):
        env = GraDoomVecEnv(smap, lanes, device="cuda:0", episode_timeout=50, sprites=8, obs_layout=layout, obs_copy="safe_view")
        view = (lambda t: t) if layout == "chw" else (lambda t: t.permute(0, 2, 3, 1))
        first, _ = env.reset(seed=4)
        assert first.data_ptr() != env.frames.data_ptr() and torch.equal(first, view(env.frames))
        held = first.clone()
        second = env.step(actions)[0]
        assert second.data_ptr() != first.data_ptr()
        assert torch.equal(first, held) and torch.equal(second, view(env.frames))
        assert not torch.equal(first, second)
        third = env.step(actions)[0]
        assert third.data_ptr() == first.data_ptr() and torch.equal(third, view(env.frames))
        env.close()


def test_more_than_256_linedefs_in_one_column_raise_in_the_environment(monkeypatch):
    # A corridor of 300 narrow sectors seen end on: every divider lands in the same few screen columns, more than the 256
    # candidates a column can hold in the spill pool (64 in its own slots).  The environment must say so rather than hand
    # out the frame.
    from gradoom_amd import synthmap
    from gradoom_amd.env import GraDoomVecEnv, PosePoolDynamics

    monkeypatch.setattr(synthmap, "CELL", 48)   # 300 cells of the usual 256 units would leave the 16.16 coordinate range
    smap = synthmap.generate_map(5, grid=(300, 1), sectors=300, linedefs=901)
    lanes = 2
    dynamics = PosePoolDynamics(smap, lanes, "cuda:0", pool=4)
    quad = smap.sector_quads[0]
    centre = quad.mean(axis=0)
    dynamics._pool["x"].fill_(float(centre[0]))
    dynamics._pool["y"].fill_(float(centre[1]))
    dynamics._pool["angle_bam"].zero_()       # looking along +x, down the corridor
    dynamics._pool["pitch_bam"].zero_()
    dynamics._pool["view_z"].fill_(float(smap.sector_heights[0, 0]) + 41.0)
    env = GraDoomVecEnv(smap, lanes, device="cuda:0", dynamics=dynamics, render_mode="rgb_array")
    mask = torch.ones(lanes, dtype=torch.bool, device="cuda:0")
    env.reset_device(mask, torch.arange(lanes, device="cuda:0"))
    assert env._renderer.status() & 1
    with pytest.raises(RuntimeError, match="truncated a screen column's candidate list"):
        env.step_and_reset_device(torch.zeros(lanes, dtype=torch.int64, device="cuda:0"), torch.arange(lanes, device="cuda:0"))
    with pytest.raises(RuntimeError, match="truncated"):
        env.render()
    with pytest.raises(RuntimeError, match="truncated"):
        env.close()
    assert env.closed
