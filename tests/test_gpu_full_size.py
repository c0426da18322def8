"""The headline shape (config4: 4096 lanes, 4000 linedefs, 128 sprites per lane) through properties that need no
reference run: lanes are independent, batches are order free, the observation is a function of the frame, and a
handful of lanes equal the CPU oracle.  Every shape runs with both height distributions: the benchmark's (floors
uniform over 0..255, ceilings 64..256 above: a plane level per sector) and the map generator's quantised one."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

LANES = 4096
PROBES = (0, 1337, 2048, 4095)


HEIGHTS = ("uniform", "quantised")


def _config_map(config: str, heights: str):
    from gradoom_amd import synthmap

    smap = synthmap.generate_config_map(config)
    if heights == "uniform":    # the variant seed bench.py uses
        smap = synthmap.with_variant(smap, 5, heights="uniform")
    return smap


@pytest.fixture(scope="module", params=HEIGHTS)
def full_size(request):
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    print(f"full size: building the config4 map ({request.param} heights) and 4096 poses", flush=True)
    smap = _config_map("config4", request.param)
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


def test_both_assemblies_give_the_same_bytes(full_size):
    # frames put together band by band in LDS equal the ones assembled kernel by kernel through device memory
    renderer = full_size["renderer"]
    again = torch.zeros_like(full_size["indexed"])
    obs = torch.zeros_like(full_size["obs"])
    renderer.set_assembly("fused")
    try:
        renderer.render(full_size["lanes"], indexed=again, obs=obs)
        torch.cuda.synchronize()
    finally:
        renderer.set_assembly("auto")
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


# The other shapes of the benchmark list at their full lane counts: 256 lanes on the 800-linedef map with 32 sprites,
# 1024 lanes on the 2000-linedef map with 64 sprites and per-lane light offsets, and on the 4000-linedef map 16384 lanes
# with the observation stack as the only output (four chunks of 4096) and 512 lanes with an RGB24 frame.
SHAPES = {
    "config2_256": dict(config="config2", lanes=256, outputs=("indexed", "frames"), probes=(0, 101, 255)),
    "config3_1024": dict(config="config3", lanes=1024, outputs=("indexed", "frames"), probes=(0, 517, 1023)),
    "config5_obs_only_16384": dict(config="config4", lanes=16384, outputs=("frames",), probes=(0, 4095, 4096, 9999, 16383)),
    "config5_rgb_512": dict(config="config4", lanes=512, outputs=("indexed", "rgb"), probes=(0, 300, 511)),
}


@pytest.mark.parametrize("heights", HEIGHTS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_other_benchmark_shapes_at_full_lane_count(oracle, shape, heights):
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    spec = SHAPES[shape]
    count = spec["lanes"]
    print(f"shape {shape}, {heights} heights: building the map and {count} poses", flush=True)
    smap = _config_map(spec["config"], heights)
    tables = mapbuild.build_map_tables(smap)
    cosine = hostmath.cosine_correction("cpu").numpy()
    poses = synthmap.generate_poses_batch(smap, count, 77, flash=True)
    sprites = synthmap.generate_sprites_batch(smap, count, synthmap.CONFIGS[spec["config"]]["sprites"], 77)
    arrays = make_lane_arrays(smap, poses, sprites)
    renderer = HipRenderer(smap, count, "cuda:0", cosine_correction=cosine, tables=tables)
    lanes = LaneState.from_numpy(arrays, "cuda:0")
    rng = np.random.default_rng(23)
    start = rng.integers(0, 256, (count, 4, 84, 84), dtype=np.uint8)

    def render(state, n, first):
        out = {}
        if "indexed" in spec["outputs"]:
            out["indexed"] = torch.zeros((n, 240, 320), dtype=torch.uint8, device="cuda:0")
        if "frames" in spec["outputs"]:
            out["frames"] = torch.as_tensor(first).to("cuda:0")
        if "rgb" in spec["outputs"]:
            out["rgb"] = torch.zeros((n, 240, 320, 3), dtype=torch.uint8, device="cuda:0")
        renderer.render(state, **out)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        return out

    print(f"shape {shape}: rendering", flush=True)
    full = render(lanes, count, start)
    # probe lanes equal the CPU oracle bit for bit: frame, RGB24 expansion and rolled stack
    probes = list(spec["probes"])
    expected = oracle.render(tables, _subset(arrays, probes), cosine, frames=start[probes], want_rgb=True)
    for name, ours in full.items():
        assert np.array_equal(ours[probes].cpu().numpy(), expected[name]), name
    # lanes are independent of their batch: a shuffled sample rendered alone gives the same bytes
    picks = rng.permutation(count)[:64]
    alone = render(LaneState.from_numpy(_subset(arrays, picks), "cuda:0"), len(picks), start[picks])
    index = torch.as_tensor(picks, device="cuda:0")
    for name, ours in alone.items():
        assert torch.equal(ours, full[name][index]), name
    if "frames" in full:   # the stack rolled: three older frames kept, no lane left blank
        assert torch.equal(full["frames"][:, :3].cpu(), torch.as_tensor(start[:, 1:]))
        assert int((full["frames"][:, 3].amax(dim=(1, 2)) > 0).sum()) == count
    if "indexed" not in spec["outputs"]:
        # no frame handed out: the same stacks when every frame stays in LDS and never reaches device memory
        renderer.set_assembly("fused")
        in_lds = render(lanes, count, start)
        renderer.set_assembly("auto")
        for name, ours in in_lds.items():
            assert torch.equal(ours, full[name]), name
    renderer.close()
