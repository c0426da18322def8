"""HIP against the CPU oracle on seeded random small maps: every layout the generator knows, split linedefs,
styled sprites, cameras a hair from walls, extreme pitch.  (A 137,600 lane-frame run of the same generator
over 8,600 seeds found no differing pixel; this keeps a slice of it as a regression test.)"""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from random_cases import SHAPES, awkward_billboard_parts, closed_door_case, corridor_case, outside_parts  # noqa: E402,F401  (other test modules import corridor_case from here)

LANES = 8


def random_case(seed: int):
    from gradoom_amd import mapbuild, synthmap
    from gradoom_amd.selfcheck import make_lane_arrays

    rng = np.random.default_rng(seed)
    layout, grid, sectors, linedefs, islands, pillars = SHAPES[seed % len(SHAPES)]
    smap = synthmap.generate_map(
        seed, grid=grid, sectors=sectors, linedefs=linedefs, layout=layout, islands=islands, pillars=pillars,
        midtex=float(rng.choice([0.0, 0.1, 0.3])),
    )
    if rng.random() < 0.4:
        smap = synthmap.split_linedefs(smap, seed + 1)
    if rng.random() < 0.5:
        smap = synthmap.with_blend_tables(smap, seed + 2)
    margin = float(rng.choice([0.005, 0.02, 0.15]))
    poses = synthmap.generate_poses(smap, LANES, seed + 3, pitch=bool(rng.random() < 0.6), flash=bool(rng.random() < 0.5), margin=margin)
    if rng.random() < 0.3:
        poses.pitch_bam[:] = rng.integers(-30, 31, LANES) * (182 << 16)
    sprites = synthmap.generate_sprites(smap, LANES, 24, seed + 4)
    arrays = make_lane_arrays(smap, poses, sprites)
    arrays["sprite_style"] = rng.choice(np.array([-1, -1, -1, -2, 0, 1], dtype=np.int8), size=sprites.x.shape)
    return smap, mapbuild.build_map_tables(smap), arrays


@pytest.mark.parametrize("first_seed", [7000, 7008, 7016])
def test_random_maps_and_grazing_poses_match_the_oracle(oracle, first_seed):
    from gradoom_amd import hostmath
    from gradoom_amd.renderer import HipRenderer, LaneState

    cosine = hostmath.cosine_correction("cpu").numpy()
    for seed in range(first_seed, first_seed + 8):
        print(f"random case {seed}", flush=True)
        smap, tables, arrays = random_case(seed)
        expected = oracle.render(tables, arrays, cosine)
        renderer = HipRenderer(smap, LANES, "cuda:0", cosine_correction=cosine, tables=tables)
        indexed = torch.zeros((LANES, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((LANES, 84, 84), dtype=torch.uint8, device="cuda:0")
        state = LaneState.from_numpy(arrays, "cuda:0")
        renderer.render(state, indexed=indexed, obs=obs)
        own_frame_obs, fused_obs = torch.zeros_like(obs), torch.zeros_like(obs)
        renderer.render(state, obs=own_frame_obs)   # observations only: through the working memory's own frame
        renderer.set_assembly("fused")
        renderer.render(state, obs=fused_obs)       # or assembled in LDS
        renderer.set_assembly("auto")
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), f"seed {seed}"
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), f"seed {seed}"
        assert torch.equal(fused_obs, obs) and torch.equal(own_frame_obs, obs), f"seed {seed}"
        renderer.close()


@pytest.mark.parametrize("first_seed", [9000, 9006])
def test_random_maps_with_other_heights_and_textures_whatever_the_working_memory_held(oracle, first_seed):
    # doors and crawl spaces, uniform heights, odd texture sizes and eyes at any height, each rendered three times: into
    # fresh working memory, then after it was filled with 0xFF and with 0xA5 (no frame may depend on what an earlier
    # frame, or nobody, left there: the kernels clear nothing between frames)
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    cosine = hostmath.cosine_correction("cpu").numpy()
    variants = (dict(heights="doors"), dict(heights="uniform"), dict(heights="doors", textures="npot"), dict(textures="mixed"),
                dict(heights="uniform", textures="npot"), dict(heights="doors"))
    for seed in range(first_seed, first_seed + 6):
        print(f"variant case {seed}", flush=True)
        rng = np.random.default_rng(seed)
        layout, grid, sectors, linedefs, islands, pillars = SHAPES[seed % len(SHAPES)]
        smap = synthmap.generate_map(seed, grid=grid, sectors=sectors, linedefs=linedefs, layout=layout, islands=islands,
                                     pillars=pillars, midtex=float(rng.choice([0.0, 0.2])))
        smap = synthmap.with_variant(smap, seed + 1, **variants[seed % len(variants)])
        poses = synthmap.generate_poses(smap, LANES, seed + 3, pitch=bool(rng.random() < 0.5), flash=True,
                                        margin=float(rng.choice([0.02, 0.15])), eye="any")
        arrays = make_lane_arrays(smap, poses, synthmap.generate_sprites(smap, LANES, 16, seed + 4))
        tables = mapbuild.build_map_tables(smap)
        expected = oracle.render(tables, arrays, cosine)
        renderer = HipRenderer(smap, LANES, "cuda:0", cosine_correction=cosine, tables=tables)
        lanes = LaneState.from_numpy(arrays, "cuda:0")
        for fill, assembly in ((None, "separate"), (0xFF, "fused"), (0xA5, "separate"), (0x5A, "fused")):
            renderer.set_assembly(assembly)
            if fill is not None:
                renderer.scribble(fill)
            indexed = torch.zeros((LANES, 240, 320), dtype=torch.uint8, device="cuda:0")
            obs = torch.zeros((LANES, 84, 84), dtype=torch.uint8, device="cuda:0")
            renderer.render(lanes, indexed=indexed, obs=obs)
            torch.cuda.synchronize()
            assert renderer.status() == 0
            assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), f"seed {seed} fill {fill} {assembly}"
            assert np.array_equal(obs.cpu().numpy(), expected["obs"]), f"seed {seed} fill {fill} {assembly}"
        renderer.close()


@pytest.mark.parametrize("seed", [50078, 50079, 50082])
def test_rows_that_only_a_portal_path_clip_closes_show_the_flat_picture(oracle, seed):
    """Seed 50078, lanes 7 and 14: a column loses its sector, picks a linedef beyond a projected solid and takes that
    path's clips, which close the window over rows 51..97 without painting or claiming one of them (engine.py:12969-13069).
    The reference shows the flat pass's picture there; the traversal has to hand those rows to the flat pass itself, since
    nothing clears its working memory between frames."""
    from gradoom_amd import hostmath
    from gradoom_amd.renderer import HipRenderer, LaneState

    lanes = 16
    cosine = hostmath.cosine_correction("cpu").numpy()
    smap, tables, arrays = closed_door_case(seed, lanes)
    expected = oracle.render(tables, arrays, cosine)
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    state = LaneState.from_numpy(arrays, "cuda:0")
    for fill, assembly in ((None, "separate"), (0xA5, "fused"), (0xFF, "separate")):
        renderer.set_assembly(assembly)
        if fill is not None:
            renderer.scribble(fill)
        indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(state, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), f"seed {seed} fill {fill} {assembly}"
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), f"seed {seed} fill {fill} {assembly}"
    renderer.close()


@pytest.mark.parametrize("seed, variants, eye_any", [(70017, False, False), (70034, False, False), (70047, False, False), (80127, True, True),
                                                    (80300, True, True), (80301, True, True), (80302, True, True), (80303, True, True)])
def test_sectors_with_ceilings_below_their_floors_match_the_oracle(oracle, seed, variants, eye_any):
    """Up to four sectors per map with the ceiling 16 units below the floor.  Seen from a neighbour, such a sector's upper
    and lower tier share rows: the lower tier paints them, and they take the four-column group's shade as soon as EITHER
    tier's common bottom row is passed (engine.py:12688-12761; seeds 70017, 70034, 70047).  Seen from inside, the ceiling's
    and the floor's plane rows overlap: the floor's claim has the say, the ceiling's stands where the floor makes none, and
    either silhouette records the sprite clip (engine.py:12637-12687, 12943-12964; seed 80127)."""
    from gradoom_amd import hostmath
    from gradoom_amd.renderer import HipRenderer, LaneState

    lanes = 16
    cosine = hostmath.cosine_correction("cpu").numpy()
    smap, tables, arrays = closed_door_case(seed, lanes, inverted=True, variants=variants, eye_any=eye_any)
    assert (smap.sector_heights[:, 1] < smap.sector_heights[:, 0]).any() or seed >= 80300
    expected = oracle.render(tables, arrays, cosine)
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    state = LaneState.from_numpy(arrays, "cuda:0")
    for fill, assembly in ((None, "separate"), (0x5A, "fused")):
        renderer.set_assembly(assembly)
        if fill is not None:
            renderer.scribble(fill)
        indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(state, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), f"seed {seed} fill {fill} {assembly}"
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), f"seed {seed} fill {fill} {assembly}"
    renderer.close()


def test_a_ceiling_clip_carried_below_the_floor_clip_still_records_its_silhouette(oracle):
    """A zero-height sector closes a column's window at row 94; behind it a sector with its ceiling below its floor moves
    the ceiling clip on to row 130, past the floor clip.  Nothing is painted in the rows between, yet the pass's top
    silhouette reaches over them, and being nearer by a rounding error (three linedefs meet in that column) than the
    bottom silhouette of the pass before, it decides whether a billboard behind shows there (engine.py:12943-12964)."""
    from gradoom_amd import hostmath
    from gradoom_amd.renderer import HipRenderer, LaneState

    lanes = 16
    cosine = hostmath.cosine_correction("cpu").numpy()
    smap, tables, arrays = closed_door_case(503259, lanes, mixed=True, variants=True, eye_any=True)
    heights = np.asarray(smap.sector_heights)
    assert (heights[:, 1] < heights[:, 0]).any() and (heights[:, 1] == heights[:, 0]).any()
    expected = oracle.render(tables, arrays, cosine)
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    state = LaneState.from_numpy(arrays, "cuda:0")
    for assembly in ("separate", "fused"):
        renderer.set_assembly(assembly)
        indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(state, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), assembly
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), assembly
    renderer.close()


@pytest.mark.parametrize("seed", [1200007, 1200011, 1200018])
def test_billboards_in_awkward_places_match_the_oracle(oracle, seed):
    """Billboards at exactly the same depth (the oracle and the HIP path paint those in slot order; the reference's order
    among them is torch.topk's and not defined), at the eye, a step from it, on vertices and linedefs, far outside the map,
    lifted or sunk, some of them blending with what is under them."""
    from gradoom_amd import hostmath, mapbuild
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    lanes = 16
    cosine = hostmath.cosine_correction("cpu").numpy()
    smap, poses, sprites = awkward_billboard_parts(seed, lanes)
    tables = mapbuild.build_map_tables(smap)
    arrays = make_lane_arrays(smap, poses, sprites)
    arrays["sprite_style"] = np.random.default_rng(seed).choice(np.array([-1, -1, -2, 0, 1], dtype=np.int8), size=sprites.x.shape)
    arrays["sprite_style"][::2] = -1    # every other lane's billboards all plain: painted beside the flat pass
    expected = oracle.render(tables, arrays, cosine)
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    state = LaneState.from_numpy(arrays, "cuda:0")
    for assembly in ("separate", "fused"):
        renderer.set_assembly(assembly)
        indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(state, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), assembly
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), assembly
    renderer.close()


@pytest.mark.parametrize("sectors", [80, 124])
def test_columns_that_see_more_than_64_linedefs_match_the_oracle(oracle, sectors):
    """Such columns get a slot in the spill pool, where every linedef their ray can reach is listed (the reference keeps a
    dense [columns, linedefs] table, engine.py:11446-11451, and has no limit).  124 sectors: the longest corridor of
    256-unit cells the 16.16 coordinates hold; its columns draw more than a hundred passes."""
    from gradoom_amd import hostmath
    from gradoom_amd.renderer import HipRenderer, LaneState

    lanes = 6
    cosine = hostmath.cosine_correction("cpu").numpy()
    smap, tables, arrays = corridor_case(lanes, sectors)
    expected = oracle.render(tables, arrays, cosine)
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    state = LaneState.from_numpy(arrays, "cuda:0")
    for fill, assembly in ((None, "separate"), (0xA5, "fused"), (None, "separate")):
        renderer.set_assembly(assembly)
        if fill is not None:
            renderer.scribble(fill)
        indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(state, indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"]), f"fill {fill} {assembly}"
        assert np.array_equal(obs.cpu().numpy(), expected["obs"]), f"fill {fill} {assembly}"
    renderer.close()


def test_cameras_outside_the_map_match_the_oracle(oracle):
    """Cameras in the void beside the map: no wall pass claims most of the screen, so nearly every pixel shows the
    flat pass's picture (far more than the per-lane gap pixel list holds) and most of them stay unresolved."""
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    cosine = hostmath.cosine_correction("cpu").numpy()
    smap, poses, sprites = outside_parts(LANES)
    tables = mapbuild.build_map_tables(smap)
    rng = np.random.default_rng(6)
    arrays = make_lane_arrays(smap, poses, sprites)
    renderer = HipRenderer(smap, LANES, "cuda:0", cosine_correction=cosine, tables=tables)
    # Billboards over pixels that show the flat pass's picture, three ways: no styles at all (every lane's billboards are
    # painted ahead of the flat pass's pixels and mark the ones they take), styles on the odd lanes only (the two kinds of
    # lane share a frame; lane 1 of them carries a style on a dead billboard only and counts as plain), styles everywhere.
    styles = rng.choice(np.array([-1, -2, 0, 1], dtype=np.int8), size=sprites.x.shape)
    odd_only = styles.copy()
    odd_only[0::2] = -1
    odd_only[1] = np.where(arrays["sprite_alive"][1] != 0, -1, -2)
    for case in (None, odd_only, styles):
        if case is not None:
            arrays["sprite_style"] = case
        expected = oracle.render(tables, arrays, cosine)
        indexed = torch.zeros((LANES, 240, 320), dtype=torch.uint8, device="cuda:0")
        obs = torch.zeros((LANES, 84, 84), dtype=torch.uint8, device="cuda:0")
        renderer.render(LaneState.from_numpy(arrays, "cuda:0"), indexed=indexed, obs=obs)
        torch.cuda.synchronize()
        assert renderer.status() == 0
        assert np.array_equal(indexed.cpu().numpy(), expected["indexed"])
        assert np.array_equal(obs.cpu().numpy(), expected["obs"])
    renderer.close()
