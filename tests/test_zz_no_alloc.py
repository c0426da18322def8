"""gd_render_static, the entry point that allocates nothing, against gd_render (needs an MI355X)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import lane_inputs, load_fixture

pytestmark = pytest.mark.gpu


def _render(renderer, call, lanes, count, start, mask):
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
    frames = torch.as_tensor(start).to("cuda:0")
    rgb = torch.zeros((count, 240, 320, 3), dtype=torch.uint8, device="cuda:0")
    call(lanes, indexed=indexed, obs=obs, frames=frames, reset_mask=torch.as_tensor(mask).to("cuda:0"), rgb=rgb)
    torch.cuda.synchronize()
    assert renderer.status() == 0
    return [t.cpu().numpy() for t in (indexed, obs, frames, rgb)]


def test_static_entry_point_equals_gd_render_on_two_calls_in_a_row():
    # the second call is smaller than the first and finds the array as the first left it
    from gradoom_amd.renderer import HipRenderer, LaneState

    meta, data, smap, tables = load_fixture("small_midtex_sprites")
    base = lane_inputs(data)
    count = meta["lanes"]
    plain = HipRenderer(smap, 64, "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)
    bare = HipRenderer(smap, 0, "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)   # the map only
    rng = np.random.default_rng(17)
    for total in (61, 7):
        print(f"static entry point: {total} lanes", flush=True)
        picks = rng.permutation(total) % count
        arrays = {k: np.ascontiguousarray(v[picks]) for k, v in base.items()}
        lanes = LaneState.from_numpy(arrays, "cuda:0")
        start = rng.integers(0, 256, (total, 4, 84, 84), dtype=np.uint8)
        mask = (rng.random(total) < 0.4).astype(np.uint8)
        expected = _render(plain, plain.render, lanes, total, start, mask)
        ours = _render(bare, bare.render_static, lanes, total, start, mask)
        for name, a, b in zip(("indexed", "obs", "frames", "rgb"), ours, expected):
            assert np.array_equal(a, b), name
        assert np.array_equal(ours[0], data["indexed"][picks])   # and both equal the reference's golden frames
    with pytest.raises(ValueError):
        bare.render(lanes, indexed=torch.zeros((total, 240, 320), dtype=torch.uint8, device="cuda:0"))   # no working memory of its own
    plain.close()
    bare.close()


def test_static_entry_point_lists_long_columns_in_its_own_spill_pool():
    # an 80-sector corridor seen end on: a few columns of every lane see more than 64 linedefs and move to the spill pool,
    # of which the static array holds one block (320 columns) per chunk
    from gradoom_amd import hostmath
    from gradoom_amd.renderer import HipRenderer, LaneState
    from test_gpu_random_maps import corridor_case

    total = 12
    smap, tables, arrays = corridor_case(total)
    cosine = hostmath.cosine_correction("cpu").numpy()
    lanes = LaneState.from_numpy(arrays, "cuda:0")
    plain = HipRenderer(smap, total, "cuda:0", cosine_correction=cosine, tables=tables)
    bare = HipRenderer(smap, 0, "cuda:0", cosine_correction=cosine, tables=tables)
    rng = np.random.default_rng(5)
    start = rng.integers(0, 256, (total, 4, 84, 84), dtype=np.uint8)
    mask = np.zeros(total, dtype=np.uint8)
    expected = _render(plain, plain.render, lanes, total, start, mask)
    ours = _render(bare, bare.render_static, lanes, total, start, mask)
    for name, a, b in zip(("indexed", "obs", "frames", "rgb"), ours, expected):
        assert np.array_equal(a, b), name
    plain.close()
    bare.close()


def test_static_entry_point_rejects_more_lanes_than_its_limit():
    import ctypes as C

    from gradoom_amd import _abi, _lib, hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    smap = synthmap.generate_map(31, grid=(6, 5), sectors=26, linedefs=160)
    tables = mapbuild.build_map_tables(smap)
    cosine = hostmath.cosine_correction("cpu").numpy()
    renderer = HipRenderer(smap, 0, "cuda:0", cosine_correction=cosine, tables=tables)
    lanes = LaneState.from_numpy(make_lane_arrays(smap, synthmap.generate_poses(smap, 2, 5)), "cuda:0")
    indexed = torch.zeros((2, 240, 320), dtype=torch.uint8, device="cuda:0")
    renderer.render_static(lanes, indexed=indexed)   # two lanes fit
    torch.cuda.synchronize()
    assert int(indexed[:, :208].amax()) > 0
    # the limit is checked before anything is launched, so claiming more lanes than the tensors hold is safe here
    desc, keep = renderer._lanes_desc(lanes)
    desc.lane_count = _abi.STATIC_MAX_LANES + 1
    out, keep_out = renderer._out_desc(2, indexed, None, None, None, None)
    with pytest.raises(ValueError, match="at most"):
        _lib.check(renderer._lib.gd_render_static(renderer._handle, C.byref(desc), C.byref(out), None))
    del keep, keep_out
    renderer.close()


def test_static_entry_point_at_the_headline_map_size_in_several_chunks():
    # the 4000-linedef map with uniform heights: a chunk of the 64 MiB array holds about twenty lanes, so 100 lanes take
    # five; the hand-off options of gd_render (hwc final frames, status bar rows pooled) go through unchanged
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    total = 100
    print("static entry point: config4 map, uniform heights, 100 lanes", flush=True)
    smap = synthmap.with_variant(synthmap.generate_config_map("config4"), 5, heights="uniform")
    tables = mapbuild.build_map_tables(smap)
    cosine = hostmath.cosine_correction("cpu").numpy()
    poses = synthmap.generate_poses_batch(smap, total, 55, flash=True)
    sprites = synthmap.generate_sprites_batch(smap, total, synthmap.CONFIGS["config4"]["sprites"], 55)
    lanes = LaneState.from_numpy(make_lane_arrays(smap, poses, sprites), "cuda:0")
    plain = HipRenderer(smap, total, "cuda:0", cosine_correction=cosine, tables=tables)
    bare = HipRenderer(smap, 0, "cuda:0", cosine_correction=cosine, tables=tables)
    rng = np.random.default_rng(41)
    start = rng.integers(0, 256, (total, 4, 84, 84), dtype=np.uint8)
    results = []
    for call in (plain.render, bare.render_static):
        indexed = torch.zeros((total, 240, 320), dtype=torch.uint8, device="cuda:0")
        frames = torch.as_tensor(start).to("cuda:0")
        final = torch.zeros((total, 84, 84, 4), dtype=torch.uint8, device="cuda:0")
        call(lanes, indexed=indexed, frames=frames, final_frames=final, final_layout="hwc", obs_source_rows=240)
        torch.cuda.synchronize()
        results.append((indexed, frames, final))
    assert plain.status() == 0 and bare.status() == 0
    for ours, expected in zip(results[1], results[0]):
        assert torch.equal(ours, expected)
    assert torch.equal(results[1][2], results[1][1].permute(0, 2, 3, 1))
    assert int((results[1][0][:, :208].amax(dim=(1, 2)) > 0).sum()) == total
    plain.close()
    bare.close()


def test_static_entry_point_replays_from_a_captured_graph():
    # the callers the entry point is for: a captured graph allocates nothing when it is replayed.  Every replay, after the
    # poses changed and with eager work in between, equals the eager frame of gd_render.
    from gradoom_amd.renderer import HipRenderer, LaneState

    meta, data, smap, tables = load_fixture("small_midtex_sprites")
    count = meta["lanes"]
    base = lane_inputs(data)
    plain = HipRenderer(smap, count, "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)
    bare = HipRenderer(smap, 0, "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)
    lanes = LaneState.from_numpy(base, "cuda:0")
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    frames = torch.zeros((count, 4, 84, 84), dtype=torch.uint8, device="cuda:0")
    bare.render_static(lanes, indexed=indexed, frames=frames)    # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        bare.render_static(lanes, indexed=indexed, frames=frames)
    rng = np.random.default_rng(3)
    for replay in range(4):
        order = rng.permutation(count)
        for name in ("x", "y", "angle", "view_z", "x_fixed", "y_fixed", "angle_bam", "pitch_bam", "flash_light", "ray_cos", "ray_sin",
                     "sprite_x", "sprite_y", "sprite_z", "sprite_depth", "sprite_id", "sprite_alive", "sprite_fullbright"):
            getattr(lanes, name).copy_(torch.as_tensor(np.ascontiguousarray(base[name][order])).to("cuda:0").to(getattr(lanes, name).dtype))
        before = frames.clone()
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.zeros_like(indexed)
        eager_frames = before.clone()
        plain.render(lanes, indexed=eager, frames=eager_frames)
        torch.cuda.synchronize()
        assert torch.equal(indexed, eager), f"replay {replay}"
        assert torch.equal(frames, eager_frames), f"replay {replay}"
        assert np.array_equal(indexed.cpu().numpy(), data["indexed"][order])
    plain.close()
    bare.close()
