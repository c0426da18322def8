"""HIP path against the reference's golden vectors and against the CPU oracle (needs an MI355X)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import fixture_names, fixture_overlays, lane_inputs, load_fixture

pytestmark = pytest.mark.gpu


def _renderer(name):
    from gradoom_amd.renderer import HipRenderer, LaneState

    meta, data, smap, tables = load_fixture(name)
    renderer = HipRenderer(smap, meta["lanes"], "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)
    overlays = fixture_overlays(meta)
    if overlays is not None:
        renderer.set_overlays(overlays)
    lanes = LaneState.from_numpy(lane_inputs(data), "cuda:0")
    return meta, data, tables, renderer, lanes


@pytest.mark.parametrize("name", fixture_names())
def test_indexed_frame_bit_exact_vs_reference_golden(name):
    print(f"case {name}", flush=True)
    meta, data, _tables, renderer, lanes = _renderer(name)
    count = meta["lanes"]
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
    # both ways of putting a frame together (kernel by kernel through device memory; band by band in LDS), the second one
    # into working memory filled with ones: nothing is cleared between frames
    for assembly, fill in (("separate", None), ("fused", 0xFF)):
        if meta.get("decals") and assembly == "fused":
            continue   # frames with wall decals are always assembled kernel by kernel
        renderer.set_assembly(assembly)
        if fill is not None:
            renderer.scribble(fill)
            indexed.zero_()
            obs.zero_()
        renderer.render(lanes, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        ours = indexed.cpu().numpy()
        mismatched = int((ours != data["indexed"]).sum())
        assert mismatched == 0, f"{mismatched} palette indices differ from the reference ({assembly} assembly, working memory fill {fill})"
        delta = np.abs(obs.cpu().numpy().astype(np.int32) - data["obs"].astype(np.int32))
        assert delta.max() <= 1 and delta.mean() < 0.01  # tolerance: tests/test_rendering.py:138-139
    renderer.close()


@pytest.mark.parametrize("name", ["config1", "small_midtex_sprites", "screen_flashes"])
def test_observation_and_stack_bit_exact_vs_oracle(oracle, name):
    meta, data, tables, renderer, lanes = _renderer(name)
    count = meta["lanes"]
    rng = np.random.default_rng(3)
    start = rng.integers(0, 256, (count, 4, 84, 84), dtype=np.uint8)
    mask = (rng.random(count) < 0.4).astype(np.uint8)
    expected = oracle.render(tables, lane_inputs(data), data["cosine_correction"], frames=start, reset_mask=mask, want_rgb=True)
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
    frames = torch.as_tensor(start).to("cuda:0")
    rgb = torch.zeros((count, 240, 320, 3), dtype=torch.uint8, device="cuda:0")
    for assembly in ("separate", "fused"):
        renderer.set_assembly(assembly)
        frames = torch.as_tensor(start).to("cuda:0")
        for tensor in (indexed, obs, rgb):
            tensor.zero_()
        renderer.render(lanes, indexed=indexed, obs=obs, frames=frames, reset_mask=torch.as_tensor(mask).to("cuda:0"), rgb=rgb)
        torch.cuda.synchronize()
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), assembly
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), assembly
        assert np.array_equal(frames.cpu().numpy(), expected["frames"]), assembly
        assert np.array_equal(rgb.cpu().numpy(), expected["rgb"]), assembly
        assert np.array_equal(rgb[0].cpu().numpy(), data["rgb_lane0"])
        if "rgb_all" in data:   # the case with per-lane screen blends carries every lane's reference RGB24 frame
            assert np.array_equal(rgb.cpu().numpy(), data["rgb_all"][:count])
    renderer.close()


def test_observe_entry_point_matches_oracle(oracle):
    _meta, _data, _tables, renderer, _lanes = _renderer("tiny_stages")
    rng = np.random.default_rng(11)
    for rows in (208, 240):
        indexed = rng.integers(0, 256, (5, rows, 320), dtype=np.uint8)
        start = rng.integers(0, 256, (5, 4, 84, 84), dtype=np.uint8)
        mask = np.asarray([1, 0, 0, 1, 0], dtype=np.uint8)
        expected_obs, expected_frames = oracle.observe(indexed, renderer.tables["playpal"], frames=start, reset_mask=mask)
        obs = torch.zeros((5, 84, 84), dtype=torch.uint8, device="cuda:0")
        frames = torch.as_tensor(start).to("cuda:0")
        renderer.observe(torch.as_tensor(indexed).to("cuda:0"), obs=obs, frames=frames, reset_mask=torch.as_tensor(mask).to("cuda:0"))
        torch.cuda.synchronize()
        assert np.array_equal(obs.cpu().numpy(), expected_obs)
        assert np.array_equal(frames.cpu().numpy(), expected_frames)
    renderer.close()


def test_chunked_batches_render_every_lane_like_the_golden():
    # a renderer made for a few lanes given more than that renders chunk by chunk, the last one short
    from gradoom_amd.renderer import HipRenderer, LaneState

    meta, data, smap, tables = load_fixture("small_midtex_sprites")
    base = lane_inputs(data)
    count = meta["lanes"]
    for max_lanes, total in ((4, 11), (16, 40)):
        picks = np.arange(total) % count
        arrays = {k: np.ascontiguousarray(v[picks]) for k, v in base.items()}
        renderer = HipRenderer(smap, max_lanes, "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)
        lanes = LaneState.from_numpy(arrays, "cuda:0")
        indexed = torch.zeros((total, 240, 320), dtype=torch.uint8, device="cuda:0")
        for _ in range(2):  # the second frame reuses every working set
            indexed.zero_()
            renderer.render(lanes, indexed=indexed)
            torch.cuda.synchronize()
            assert renderer.status() == 0
            assert np.array_equal(indexed.cpu().numpy(), data["indexed"][picks])
        renderer.close()


def test_empty_single_lane_and_billboard_free_batches(oracle):
    # the ragged ends of the input domain: a batch of no lanes (the call does nothing and writes nothing), one lane on its
    # own, lanes whose billboards are all dead, and the same lanes handed over without any billboard tensor
    import dataclasses

    meta, data, tables, renderer, lanes = _renderer("small_midtex_sprites")
    count = meta["lanes"]
    arrays = lane_inputs(data)
    none = lanes.select(slice(0, 0))
    guard = torch.full((1, 240, 320), 7, dtype=torch.uint8, device="cuda:0")
    for call in (renderer.render, renderer.render_static):
        call(none, indexed=guard[:0], obs=torch.empty((0, 84, 84), dtype=torch.uint8, device="cuda:0"),
             frames=torch.empty((0, 4, 84, 84), dtype=torch.uint8, device="cuda:0"))
    renderer.observe(guard[:0, :208], obs=torch.empty((0, 84, 84), dtype=torch.uint8, device="cuda:0"))
    torch.cuda.synchronize()
    assert renderer.status() == 0 and bool((guard == 7).all())
    for lane in (0, count - 1):
        indexed = torch.zeros((1, 240, 320), dtype=torch.uint8, device="cuda:0")
        renderer.render(lanes.select(slice(lane, lane + 1)), indexed=indexed)
        assert np.array_equal(indexed.cpu().numpy(), data["indexed"][lane:lane + 1])
    dead = dict(arrays, sprite_alive=np.zeros_like(arrays["sprite_alive"]))
    expected = oracle.render(tables, dead, data["cosine_correction"])
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
    bare = {f.name: None for f in dataclasses.fields(lanes) if f.name.startswith("sprite_")}
    for variant in (dataclasses.replace(lanes, sprite_alive=torch.zeros_like(lanes.sprite_alive)), dataclasses.replace(lanes, **bare)):
        for assembly in ("separate", "fused"):
            renderer.set_assembly(assembly)
            indexed.zero_()
            obs.zero_()
            renderer.render(variant, indexed=indexed, obs=obs)
            assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), assembly
            assert np.array_equal(obs.cpu().numpy(), expected["obs"]), assembly
    renderer.close()


def test_final_frames_and_stack_modes_match_the_oracle(oracle):
    # the three ways a call leaves the stack (step; step with some lanes reset; reset of the masked lanes only), each
    # against the oracle's stack, with the fused final-observation clone (env.py:915-917) equal to it
    meta, data, tables, renderer, lanes = _renderer("config1")
    count = meta["lanes"]
    rng = np.random.default_rng(5)
    start = rng.integers(0, 256, (count, 4, 84, 84), dtype=np.uint8)
    mask_np = (rng.random(count) < 0.5).astype(np.uint8)
    assert 0 < mask_np.sum() < count
    mask = torch.as_tensor(mask_np).to("cuda:0")
    for mode, kwargs, oracle_kwargs in (
        ("step", dict(), dict(stack_mode=0)),
        ("step+reset", dict(reset_mask=mask), dict(stack_mode=0, reset_mask=mask_np)),
        ("reset", dict(reset_mask=mask, stack_only_masked=True), dict(stack_mode=1, reset_mask=mask_np)),
    ):
        print(f"stack mode {mode}", flush=True)
        expected = oracle.render(tables, lane_inputs(data), data["cosine_correction"], frames=start, **oracle_kwargs)
        # kernel by kernel through the caller's frame, through the working memory's own when the caller takes none, and
        # band by band in LDS: all must roll alike
        scratch_frame = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
        separate = torch.as_tensor(start).to("cuda:0")
        renderer.render(lanes, frames=separate, indexed=scratch_frame, **kwargs)
        own_frame = torch.as_tensor(start).to("cuda:0")
        renderer.render(lanes, frames=own_frame, **kwargs)
        renderer.set_assembly("fused")
        frames = torch.as_tensor(start).to("cuda:0")
        final = torch.full((count, 4, 84, 84), 7, dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(lanes, frames=frames, final_frames=final, obs=obs, **kwargs)
        renderer.set_assembly("auto")
        torch.cuda.synchronize()
        assert torch.equal(frames, separate) and torch.equal(own_frame, separate), mode
        ours = frames.cpu().numpy()
        assert np.array_equal(ours, expected["frames"]), mode
        assert np.array_equal(final.cpu().numpy(), expected["frames"]), mode
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), mode
        assert final.data_ptr() != frames.data_ptr()
        # the same copy with the four stacked values of a pixel side by side (obs_layout="hwc", env.py:678-680), from
        # both assemblies
        for with_frame in (False, True):
            again = torch.as_tensor(start).to("cuda:0")
            interleaved = torch.full((count, 84, 84, 4), 9, dtype=torch.uint8, device="cuda:0")
            renderer.render(lanes, frames=again, final_frames=interleaved, final_layout="hwc",
                            indexed=scratch_frame if with_frame else None, **kwargs)
            torch.cuda.synchronize()
            assert torch.equal(again, frames), (mode, with_frame)
            assert torch.equal(interleaved, frames.permute(0, 2, 3, 1)), (mode, with_frame)
        if mode == "step":
            assert np.array_equal(ours[:, :3], start[:, 1:]) and np.array_equal(ours[:, 3], expected["obs"])
        if mode == "reset":   # lanes outside the mask keep the stack they had
            keep = mask_np == 0
            assert np.array_equal(ours[keep], start[keep])
            assert np.array_equal(ours[~keep], np.repeat(expected["obs"][~keep, None], 4, axis=1))
    renderer.close()


def test_sector_lights_replaced_between_frames_match_the_reference():
    # config1 under its own lights, then under the lights of config1_relit (same map, same cameras): the second frame
    # must be the reference's frame of the relit map, and going back must give the first again
    meta, data, tables, renderer, lanes = _renderer("config1")
    _meta2, relit, _smap2, relit_tables = load_fixture("config1_relit")
    assert np.array_equal(relit["x"], data["x"]) and not np.array_equal(relit_tables["sector_lights"], tables["sector_lights"])
    count = meta["lanes"]
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
    for lights, golden in ((None, data), (relit_tables["sector_lights"], relit), (tables["sector_lights"], data)):
        if lights is not None:
            renderer.set_sector_lights(torch.as_tensor(np.asarray(lights, dtype=np.float32)).to("cuda:0"))
        renderer.render(lanes, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert np.array_equal(indexed.cpu().numpy(), golden["indexed"])
        delta = np.abs(obs.cpu().numpy().astype(np.int32) - golden["obs"].astype(np.int32))
        assert delta.max() <= 1 and delta.mean() < 0.01
    assert (relit["indexed"] != data["indexed"]).mean() > 0.3   # the two light vectors really give different pictures
    renderer.close()


def test_status_bar_rows_pooled_into_the_observation(oracle):
    # obs_source_rows=240 (an environment made with obs_crop=None, engine.py:15440): within 1 of the reference's float
    # pooling, equal to the oracle's integer pooling, and equal to gd_observe over all 240 rows of the frame
    meta, data, tables, renderer, lanes = _renderer("overlays")
    count = meta["lanes"]
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((count, 84, 84), dtype=torch.uint8, device="cuda:0")
    renderer.render(lanes, indexed=indexed, obs=obs, obs_source_rows=240)
    again = torch.zeros_like(obs)
    renderer.observe(indexed, obs=again)
    torch.cuda.synchronize()
    delta = np.abs(obs.cpu().numpy().astype(np.int32) - data["obs_with_hud"].astype(np.int32))
    assert delta.max() <= 1 and delta.mean() < 0.01
    assert torch.equal(obs, again)
    own_frame, fused = torch.zeros_like(obs), torch.zeros_like(obs)
    renderer.render(lanes, obs=own_frame, obs_source_rows=240)   # no frame asked for: the working memory's own
    renderer.set_assembly("fused")
    renderer.render(lanes, obs=fused, obs_source_rows=240)       # weapon, status bar and pooling all in LDS
    renderer.set_assembly("auto")
    torch.cuda.synchronize()
    assert torch.equal(obs, fused) and torch.equal(obs, own_frame)
    oracle.set_overlays(fixture_overlays(meta))
    try:
        expected = oracle.render(tables, lane_inputs(data), data["cosine_correction"], obs_source_rows=240)
    finally:
        oracle.set_overlays(None)
    assert np.array_equal(obs.cpu().numpy(), expected["obs"])
    renderer.close()


def test_render_replays_from_a_captured_graph():
    # the reference replays its background pass as a CUDA graph (engine.py:15308-15336, tests/test_rendering.py:142-171):
    # gd_render neither allocates nor synchronises, so a caller can capture it; replays after the lane tensors were
    # rewritten in place must give the frames of the new poses, each checked against the reference's golden frames
    import dataclasses

    meta, data, tables, renderer, lanes = _renderer("small_midtex_sprites")
    count = meta["lanes"]
    base = lane_inputs(data)
    indexed = torch.zeros((count, 240, 320), dtype=torch.uint8, device="cuda:0")
    frames = torch.zeros((count, 4, 84, 84), dtype=torch.uint8, device="cuda:0")
    eager = torch.zeros_like(indexed)
    eager_frames = torch.zeros_like(frames)
    renderer.render(lanes, indexed=eager, frames=eager_frames)   # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        renderer.render(lanes, indexed=indexed, frames=frames)
    fields = [f.name for f in dataclasses.fields(lanes) if isinstance(getattr(lanes, f.name), torch.Tensor)]
    for replay, shift in enumerate((0, 3, 5, 0)):
        picks = (np.arange(count) + shift) % count
        for name in fields:   # new poses, written into the very tensors the graph reads
            getattr(lanes, name).copy_(torch.as_tensor(np.ascontiguousarray(base[name][picks])).to("cuda:0"))
        eager_frames.copy_(frames)
        graph.replay()
        renderer.render(lanes, indexed=eager, frames=eager_frames)   # the program's own eager work between replays
        torch.cuda.synchronize()
        assert np.array_equal(indexed.cpu().numpy(), data["indexed"][picks]), f"replay {replay}"
        assert torch.equal(indexed, eager) and torch.equal(frames, eager_frames), f"replay {replay}"
    assert renderer.status() == 0
    renderer.close()


@pytest.mark.parametrize("case", ["many_sectors", "twenty_levels", "eighty_levels"])
def test_maps_beyond_the_fast_paths_match_the_oracle(oracle, case):
    # more sectors than the LDS tables hold, more plane levels than the raster's level masks
    # (15) and than the per-lane plane tables (64): the general paths, checked against the oracle
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    print(f"case {case}", flush=True)
    if case == "many_sectors":
        smap = synthmap.generate_map(77, grid=(25, 24), sectors=600, linedefs=1300, midtex=0.1)
    else:
        smap = synthmap.generate_map(78, grid=(12, 12), sectors=144, linedefs=320, midtex=0.1)
        levels = 20 if case == "twenty_levels" else 400
        rng = np.random.default_rng(9)
        count = len(smap.sector_heights)
        smap.sector_heights[:, 0] = (rng.integers(0, levels, count) * (96.0 / levels)).astype(np.float32)
        smap.sector_heights[:, 1] = (160.0 + rng.integers(0, levels, count) * (96.0 / levels)).astype(np.float32)
    tables = mapbuild.build_map_tables(smap)
    if case == "many_sectors":
        assert tables["sector_count"] > 512
    else:
        assert tables["floor_level_count"] > (15 if case == "twenty_levels" else 64)
    lanes = 3
    poses = synthmap.generate_poses(smap, lanes, 31, flash=True)
    sprites = synthmap.generate_sprites(smap, lanes, 8, 31)
    arrays = make_lane_arrays(smap, poses, sprites)
    cosine = hostmath.cosine_correction("cpu").numpy()
    expected = oracle.render(tables, arrays, cosine, frames=np.zeros((lanes, 4, 84, 84), np.uint8))
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
    frames = torch.zeros((lanes, 4, 84, 84), dtype=torch.uint8, device="cuda:0")
    renderer.render(LaneState.from_numpy(arrays, "cuda:0"), indexed=indexed, frames=frames)
    torch.cuda.synchronize()
    assert renderer.status() == 0
    assert np.array_equal(indexed.cpu().numpy(), expected["indexed"])
    assert np.array_equal(frames.cpu().numpy(), expected["frames"])
    renderer.close()
