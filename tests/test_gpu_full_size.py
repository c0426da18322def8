"""The headline shape (config4: 4096 lanes, 4000 linedefs, 128 sprites per lane) through properties that need no
reference run: lanes are independent, batches are order free, the observation is a function of the frame, and a
handful of lanes equal the CPU oracle."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

LANES = 4096
PROBES = (0, 1337, 2048, 4095)


@pytest.fixture(scope="module")
def full_size():
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    print("full size: building the config4 map and 4096 poses", flush=True)
    smap = synthmap.generate_config_map("config4")
    tables = mapbuild.build_map_tables(smap)
    cosine = hostmath.cosine_correction("cpu").numpy()
    poses = synthmap.generate_poses_batch(smap, LANES, 321, flash=True)
    sprites = synthmap.generate_sprites_batch(smap, LANES, synthmap.CONFIGS["config4"]["sprites"], 321)
    arrays = make_lane_arrays(smap, poses, sprites)
    renderer = HipRenderer(smap, LANES, "cuda:0", cosine_correction=cosine, tables=tables)
    lanes = LaneState.from_numpy(arrays, "cuda:0")
    indexed = torch.zeros((LANES, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((LANES, 84, 84), dtype=torch.uint8, device="cuda:0")
    renderer.render(lanes, indexed=indexed, obs=obs)
    torch.cuda.synchronize()
    assert renderer.status() == 0
    yield dict(smap=smap, tables=tables, cosine=cosine, arrays=arrays, renderer=renderer, lanes=lanes, indexed=indexed, obs=obs)
    renderer.close()


def _subset(arrays: dict, picks) -> dict:
    return {key: np.ascontiguousarray(np.asarray(value)[list(picks)]) for key, value in arrays.items()}


def test_probe_lanes_equal_the_oracle(full_size, oracle):
    arrays = _subset(full_size["arrays"], PROBES)
    expected = oracle.render(full_size["tables"], arrays, full_size["cosine"])
    ours = full_size["indexed"][list(PROBES)].cpu().numpy()
    assert np.array_equal(ours, expected["indexed"])
    assert np.array_equal(full_size["obs"][list(PROBES)].cpu().numpy(), expected["obs"])


def test_a_lane_renders_the_same_alone_and_in_any_order(full_size):
    from gradoom_amd.renderer import LaneState

    renderer = full_size["renderer"]
    rng = np.random.default_rng(11)
    picks = rng.permutation(LANES)[:96]
    lanes = LaneState.from_numpy(_subset(full_size["arrays"], picks), "cuda:0")
    indexed = torch.zeros((len(picks), 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((len(picks), 84, 84), dtype=torch.uint8, device="cuda:0")
    renderer.render(lanes, indexed=indexed, obs=obs)
    torch.cuda.synchronize()
    index = torch.as_tensor(picks, device="cuda:0")
    assert torch.equal(indexed, full_size["indexed"][index])
    assert torch.equal(obs, full_size["obs"][index])


def test_a_second_frame_of_the_same_state_is_identical(full_size):
    again = torch.zeros_like(full_size["indexed"])
    obs = torch.zeros_like(full_size["obs"])
    full_size["renderer"].render(full_size["lanes"], indexed=again, obs=obs)
    torch.cuda.synchronize()
    assert torch.equal(again, full_size["indexed"])
    assert torch.equal(obs, full_size["obs"])


def test_observation_is_a_function_of_the_frame(full_size):
    # the standalone pooling entry point over the frames already rendered gives the fused observation
    renderer = full_size["renderer"]
    obs = torch.zeros_like(full_size["obs"])
    renderer.observe(full_size["indexed"][:, :208].contiguous(), obs=obs)   # view rows only: the status bar pools as black
    torch.cuda.synchronize()
    assert torch.equal(obs, full_size["obs"])
    # status bar rows hold index 0 and the view rows are not blank
    assert int(full_size["indexed"][:, 208:].max()) == 0
    assert int((full_size["indexed"][:, :208].amax(dim=(1, 2)) > 0).sum()) == LANES
