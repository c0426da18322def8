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
    cosine = hostmath.cosine_correction("cpu").numpy()

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
