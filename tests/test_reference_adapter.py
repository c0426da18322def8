"""reference_adapter: the reference engine's render methods served by the library.

The engines here are ``SimpleNamespace`` objects holding the gameplay tensors that the ``actors`` and ``overlays``
golden cases store; those cases' frames were rendered by the reference from the same tensors, so the adapter has
to reproduce them (on the GPU) from nothing but the engine and a ``CompiledScenario``-shaped object.
"""

from __future__ import annotations

import types

import numpy as np
import pytest
import torch

from conftest import fixture_overlays, load_fixture

POSE_FIELDS = dict(x="x", y="y", angle="angle", view_z="view_z", _x_fixed="x_fixed", _y_fixed="y_fixed", _angle_bam="angle_bam",
                   _pitch_bam="pitch_bam")


def compiled_scenario(smap, overlays=None, **extra):
    """A ``CompiledScenario`` look-alike (scenario.py:302-401): palette-index textures and raw patches in the fields the
    engine prefers, decoys in the fields it falls back to."""

    scenario = types.SimpleNamespace(
        vertices=smap.vertices, wall_segments=smap.wall_segments, wall_sectors=smap.wall_sectors,
        wall_side_texture_ids=smap.wall_side_texture_ids, wall_side_texture_offsets=smap.wall_side_texture_offsets,
        blocking_wall_indices=smap.blocking_wall_indices, sector_edge_mask=smap.sector_edge_mask, sector_heights=smap.sector_heights,
        sector_lights=smap.sector_lights, sector_floor_texture_ids=smap.sector_floor_texture_ids,
        sector_ceiling_texture_ids=smap.sector_ceiling_texture_ids, playpal=smap.playpal, colormap=smap.colormap,
        texture_atlas=np.zeros_like(smap.texture_atlas), texture_index_atlas=smap.texture_atlas,
        texture_widths=smap.texture_widths, texture_heights=smap.texture_heights,
        sprite_atlas=np.zeros((1, 1, 1), np.uint8), sprite_opaque=np.zeros((1, 1, 1), bool), sprite_widths=np.ones(1, np.int32),
        sprite_heights=np.ones(1, np.int32), sprite_left_offsets=np.zeros(1, np.int32), sprite_top_offsets=np.zeros(1, np.int32),
        raw_sprite_atlas=smap.sprite_atlas, raw_sprite_opaque=smap.sprite_opaque, raw_sprite_widths=smap.sprite_widths,
        raw_sprite_heights=smap.sprite_heights, raw_sprite_left_offsets=smap.sprite_left_offsets,
        raw_sprite_top_offsets=smap.sprite_top_offsets,
        wall_projection_fragments_fixed=smap.wall_projection_fragments_fixed,
        wall_projection_fragment_mask=smap.wall_projection_fragment_mask,
        projectile_additive_luts=smap.projectile_additive_luts, sprite_translucent_lut=smap.sprite_translucent_lut,
    )
    if overlays is not None:
        scenario.native_weapon_patch_atlas, scenario.native_weapon_patch_opaque = overlays["weapon_atlas"], overlays["weapon_opaque"].astype(bool)
        scenario.hud_patch_atlas, scenario.hud_patch_opaque = overlays["hud_atlas"], overlays["hud_opaque"].astype(bool)
        for short, long in (("w", "widths"), ("h", "heights"), ("left", "left_offsets"), ("top", "top_offsets")):
            setattr(scenario, f"native_weapon_patch_{long}", overlays[f"weapon_{short}"])
            setattr(scenario, f"hud_patch_{long}", overlays[f"hud_{short}"])
    for key, value in extra.items():
        setattr(scenario, key, value)
    return scenario


def stored_engine(data: dict, device="cpu", overlays=None):
    """The engine attributes a golden case stores, as tensors on ``device``."""

    from gradoom_amd import actor_inputs

    to = lambda array: torch.as_tensor(np.ascontiguousarray(array)).to(device)  # noqa: E731
    engine = types.SimpleNamespace(num_envs=int(data["x"].shape[0]), device=torch.device(device), mask_hud=True, render_screen_flashes=False)
    for attribute, key in POSE_FIELDS.items():
        setattr(engine, attribute, to(data[key]))
    flash = to(data["flash_light"])
    engine._native_weapon_frame_selection = lambda: (None, None, flash)
    engine.map = types.SimpleNamespace()
    if "actor_engine_enemy_x" in data:
        for field in actor_inputs.ENGINE_FIELDS:
            setattr(engine, field, to(data[f"actor_engine_{field}"]))
        for field in actor_inputs.MAP_FIELDS:
            setattr(engine.map, field, to(data[f"actor_map_{field}"]))
    if overlays is not None:
        from gradoom_amd import reference_adapter

        for name in dict.fromkeys(reference_adapter.WEAPON_ARGUMENTS + reference_adapter.HUD_ARGUMENTS):
            value = to(data[f"engine_{name}"])
            if name == "active_weapon":
                engine._active_weapon = lambda value=value: value
            else:
                setattr(engine, reference_adapter._ENGINE_NAMES.get(name, name), value)
        engine.map.native_weapon_frame_ids = to(overlays["weapon_frame_ids"])
        engine.map.native_weapon_flash_ids = to(overlays["weapon_flash_ids"])
    engine.frames = torch.zeros((engine.num_envs, 4, 84, 84), dtype=torch.uint8, device=device)
    return engine


class RecordingRenderer:
    def __init__(self):
        self.calls, self.overlays = [], None

    def set_overlays(self, overlays):
        self.overlays = overlays

    def render(self, lanes, **outputs):
        self.calls.append((lanes, outputs))

    def close(self):
        pass


def test_scenario_view_prefers_the_fields_the_engine_draws_from():
    # engine.py:869-912: texture_index_atlas and raw_sprite_* win over texture_atlas and sprite_*; no COLORMAP = identity
    from gradoom_amd import mapbuild, reference_adapter

    _meta, _data, smap, tables = load_fixture("actors")
    view = reference_adapter.ScenarioView(compiled_scenario(smap))
    rebuilt = mapbuild.build_map_tables(view)
    assert set(rebuilt) == set(tables)
    for key, value in tables.items():
        assert np.array_equal(np.asarray(rebuilt[key]), np.asarray(value)), key
    plain = compiled_scenario(smap)
    plain.texture_index_atlas, plain.texture_atlas, plain.colormap = None, smap.texture_atlas, None
    for field in reference_adapter.ScenarioView._SPRITE:
        setattr(plain, f"sprite_{field}", getattr(plain, f"raw_sprite_{field}"))
        setattr(plain, f"raw_sprite_{field}", None)
    fallback = reference_adapter.ScenarioView(plain)
    assert np.array_equal(fallback.texture_atlas, smap.texture_atlas) and np.array_equal(fallback.sprite_atlas, smap.sprite_atlas)
    assert np.array_equal(fallback.colormap, np.broadcast_to(np.arange(256, dtype=np.uint8), (34, 256)))
    as_tensors = compiled_scenario(smap)
    as_tensors.wall_segments = torch.as_tensor(smap.wall_segments)
    assert np.array_equal(reference_adapter.ScenarioView(as_tensors).wall_segments, smap.wall_segments)
    broken = compiled_scenario(smap)
    broken.wall_sectors = None
    with pytest.raises(ValueError, match="scenario has no wall_sectors"):
        reference_adapter.ScenarioView(broken)


def test_lane_descriptor_from_the_stored_engine_is_the_one_the_reference_frames_were_checked_with():
    from gradoom_amd import reference_adapter

    _meta, data, smap, _tables = load_fixture("actors")
    engine = stored_engine(data)
    recorder = RecordingRenderer()
    adapter = reference_adapter.HipReferenceRenderer(engine, compiled_scenario(smap), renderer=recorder, fused_actors=False)
    lanes = adapter.lane_state()
    for key in ("x", "y", "angle", "view_z", "x_fixed", "y_fixed", "angle_bam", "pitch_bam", "flash_light", "sprite_x", "sprite_y",
                "sprite_z", "sprite_id", "sprite_alive", "sprite_fullbright", "sprite_style"):
        assert np.array_equal(getattr(lanes, key).numpy(), data[key]), key
    # float32 tables computed with Torch here and by the reference there: the same ops on the same CPU
    for key in ("ray_cos", "ray_sin", "sprite_depth"):
        assert np.array_equal(getattr(lanes, key).numpy(), data[key]), key
    assert lanes.x.data_ptr() == engine.x.data_ptr(), "pose tensors are passed where they are"
    assert lanes.weapon_state is None and lanes.hud_state is None and lanes.screen_blend is None

    # which outputs each engine method asks the renderer for
    assert adapter.render_reference_frame().shape == (8, 84, 84)
    assert set(recorder.calls[-1][1]) == {"obs", "obs_source_rows"} and recorder.calls[-1][1]["obs_source_rows"] == 208
    assert adapter.render_native_indexed_frame(include_hud=False).shape == (8, 208, 320)
    assert adapter.render_native_frame().shape == (8, 240, 320, 3)
    assert adapter.finish_observation() is engine.frames and recorder.calls[-1][1]["frames"] is engine.frames
    mask = torch.tensor([True, False] * 4)
    adapter.reset_stack(mask)
    assert recorder.calls[-1][1]["stack_only_masked"] and recorder.calls[-1][1]["reset_mask"] is mask
    engine.mask_hud = False   # an environment made with obs_crop=None pools the status bar too (engine.py:15440)
    adapter.render_reference_frame()
    assert recorder.calls[-1][1]["obs_source_rows"] == 240
    adapter.install()
    assert engine.render_frame == adapter.render_reference_frame and engine.render_native_frame == adapter.render_native_frame


def test_overlay_words_from_the_stored_engine():
    from gradoom_amd import reference_adapter

    meta, data, smap, _tables = load_fixture("overlays")
    overlays = fixture_overlays(meta)
    engine = stored_engine(data, overlays=overlays)
    recorder = RecordingRenderer()
    adapter = reference_adapter.HipReferenceRenderer(engine, compiled_scenario(smap, overlays), renderer=recorder)
    assert recorder.overlays is not None and set(recorder.overlays) >= {"weapon_atlas", "weapon_w", "hud_atlas", "hud_top"}
    assert np.array_equal(recorder.overlays["hud_left"], overlays["hud_left"])
    lanes = adapter.lane_state(include_hud=True)
    assert np.array_equal(lanes.weapon_state.numpy(), data["weapon_state"])
    assert np.array_equal(lanes.hud_state.numpy(), data["hud_state"])
    assert adapter.lane_state(include_hud=False).hud_state is None
    engine.render_screen_flashes = True
    engine.bonus_count, engine.damage_count = torch.tensor([0, 8] * 6), torch.tensor([0, 50] * 6)
    engine._damage_to_alpha = torch.arange(114, dtype=torch.float32)
    blend = adapter.lane_state().screen_blend
    assert blend.shape == (12, 2) and float(blend[0].abs().sum()) == 0.0 and float(blend[1, 0]) == pytest.approx(64.0 / 255.0)


def test_policy_area_grayscale_argument_errors_are_the_reference_operators():
    # _triton_kernels.py:183-188
    from gradoom_amd.reference_adapter import policy_area_grayscale

    palette = torch.zeros((256, 3), dtype=torch.uint8)
    with pytest.raises(ValueError, match=r"indexed must have shape \(N, 208, 320\) or \(N, 240, 320\)"):
        policy_area_grayscale(torch.zeros((2, 200, 320), dtype=torch.uint8), palette)
    with pytest.raises(ValueError, match="indexed must have shape"):
        policy_area_grayscale(torch.zeros((240, 320), dtype=torch.uint8), palette)
    with pytest.raises(TypeError, match="indexed and palette must be uint8 tensors"):
        policy_area_grayscale(torch.zeros((2, 240, 320), dtype=torch.int32), palette)
    with pytest.raises(TypeError, match="indexed and palette must be uint8 tensors"):
        policy_area_grayscale(torch.zeros((2, 240, 320), dtype=torch.uint8), palette.to(torch.float32))
    with pytest.raises(ValueError, match=r"palette must have shape \(256, 3\)"):
        policy_area_grayscale(torch.zeros((2, 240, 320), dtype=torch.uint8), palette[:255])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        policy_area_grayscale(torch.zeros((2, 240, 320), dtype=torch.uint8), palette)


def host_trigonometry(monkeypatch):
    """The golden frames were made with the CPU's float32 cos / sin / atan2; the GPU's may differ in the last bit, which
    can move a pixel.  Evaluate the adapter's trigonometric inputs on the CPU so the comparison stays bit for bit."""

    from gradoom_amd import hostmath

    ray_tables, sprite_depth = hostmath.ray_tables, hostmath.sprite_depth

    def on_host(function):
        def wrapped(*tensors):
            device = tensors[0].device
            result = function(*(t.cpu() for t in tensors))
            return tuple(r.to(device) for r in result) if isinstance(result, tuple) else result.to(device)
        return wrapped

    monkeypatch.setattr(hostmath, "ray_tables", on_host(ray_tables))
    monkeypatch.setattr(hostmath, "sprite_depth", on_host(sprite_depth))


@pytest.mark.gpu
def test_adapter_reproduces_the_reference_frames_of_the_stored_engine(monkeypatch):
    from gradoom_amd import reference_adapter

    host_trigonometry(monkeypatch)
    _meta, data, smap, _tables = load_fixture("actors")
    engine = stored_engine(data, device="cuda:0")
    adapter = reference_adapter.HipReferenceRenderer(engine, compiled_scenario(smap))
    adapter.install()
    indexed = engine._render_native_indexed_frame(include_hud=True)
    assert indexed.shape == (8, 240, 320) and np.array_equal(indexed.cpu().numpy(), data["indexed"])
    assert np.array_equal(engine._render_native_indexed_frame(include_hud=False).cpu().numpy(), data["indexed"][:, :208])
    obs = engine.render_frame()
    difference = np.abs(obs.cpu().numpy().astype(np.int16) - data["obs"].astype(np.int16))
    assert int(difference.max()) <= 1, "observation within one gray level of the reference's float pipeline"
    assert np.array_equal(engine.render_native_frame(include_hud=True)[0].cpu().numpy(), data["rgb_lane0"])
    # the stack: a reset fills four copies, a step rolls by one
    mask = torch.ones(8, dtype=torch.bool, device="cuda:0")
    adapter.reset_stack(mask)
    for k in range(4):
        assert torch.equal(engine.frames[:, k], obs)
    engine.frames[:, 0] = 1
    adapter.finish_observation()
    assert torch.equal(engine.frames[:, 3], obs) and torch.equal(engine.frames[:, 2], obs) and not torch.equal(engine.frames[:, 0], torch.ones_like(obs))
    # the stand-alone operator on the reference's own indexed frame, both row counts
    palette = torch.as_tensor(smap.playpal).to("cuda:0")
    assert torch.equal(reference_adapter.policy_area_grayscale(indexed[:, :208].contiguous(), palette), obs)
    # 240 rows: the (empty) status bar is pooled as palette entry 0, not masked black, as with mask_hud off (engine.py:15440)
    engine.mask_hud = False
    with_bar = engine.render_frame()
    engine.mask_hud = True
    assert torch.equal(reference_adapter.policy_area_grayscale(indexed, palette), with_bar)
    assert torch.equal(with_bar[:, :72], obs[:, :72]) and not torch.equal(with_bar, obs)
    assert reference_adapter.policy_area_grayscale(indexed[:0], palette).shape == (0, 84, 84)
    assert adapter.renderer.status() == 0
    adapter.close()


@pytest.mark.gpu
def test_adapter_draws_the_weapon_and_the_status_bar_from_engine_tensors(monkeypatch):
    from gradoom_amd import reference_adapter

    host_trigonometry(monkeypatch)
    meta, data, smap, _tables = load_fixture("overlays")
    overlays = fixture_overlays(meta)
    engine = stored_engine(data, device="cuda:0", overlays=overlays)
    # this case's billboards were placed directly (no gameplay tensors stored): hand them to the renderer as they are
    adapter = reference_adapter.HipReferenceRenderer(engine, compiled_scenario(smap, overlays))
    lanes = adapter.lane_state(include_hud=True)
    for key in ("sprite_x", "sprite_y", "sprite_z", "sprite_id", "sprite_alive", "sprite_fullbright", "sprite_style", "sprite_depth"):
        dtype = getattr(torch, str(data[key].dtype)) if data[key].dtype != np.bool_ else torch.uint8
        setattr(lanes, key, torch.as_tensor(data[key]).to("cuda:0").to(dtype).contiguous())
    indexed = torch.empty((12, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.empty((12, 84, 84), dtype=torch.uint8, device="cuda:0")
    adapter.renderer.render(lanes, indexed=indexed, obs=obs, obs_source_rows=240)
    assert np.array_equal(indexed.cpu().numpy(), data["indexed"])
    difference = np.abs(obs.cpu().numpy().astype(np.int16) - data["obs_with_hud"].astype(np.int16))
    assert int(difference.max()) <= 1
    adapter.close()


@pytest.mark.gpu
def test_weapon_words_come_from_one_kernel_and_equal_the_reference_selection():
    from gradoom_amd import overlay_inputs, reference_adapter

    meta, data, _smap, _tables = load_fixture("overlays")
    overlays = fixture_overlays(meta)
    to = lambda array: torch.as_tensor(np.ascontiguousarray(array)).to("cuda:0")  # noqa: E731
    engine = {name: to(data[f"engine_{name}"]) for name in reference_adapter.WEAPON_ARGUMENTS}
    words, light = overlay_inputs.weapon_state(
        **engine, weapon_frame_ids=to(overlays["weapon_frame_ids"]), weapon_flash_ids=to(overlays["weapon_flash_ids"]),
        weapon_flash_lights=to(overlays["weapon_flash_lights"]), fine_sine=to(overlay_inputs.fine_sine_fixed()), want_flash_light=True,
    )
    assert words.device.type == "cuda" and words.dtype == torch.int64
    assert np.array_equal(words.cpu().numpy(), data["weapon_state"])            # what the reference frames were checked with
    assert np.array_equal(words[:, 0].cpu().numpy(), data["ref_weapon_frame_id"])
    assert np.array_equal(words[:, 1].cpu().numpy(), data["ref_weapon_flash_id"])
    assert np.array_equal(light.cpu().numpy(), data["flash_light"])             # engine.py:14949-14967, third result


@pytest.mark.gpu
def test_an_adapter_step_never_waits_for_the_device():
    # the per-lane inputs (ray tables, weapon and status bar words, wall decals) are built by kernels and Torch ops that
    # leave the host alone: with synchronisation reported as an error, a whole step still goes through
    from gradoom_amd import reference_adapter

    meta, data, smap, _tables = load_fixture("overlays")
    overlays = fixture_overlays(meta)
    engine = stored_engine(data, device="cuda:0", overlays=overlays)
    engine.map.native_weapon_flash_lights = torch.as_tensor(overlays["weapon_flash_lights"]).to("cuda:0")
    lanes, slots = engine.num_envs, 6
    rng = np.random.default_rng(9)
    engine.hitscan_decal_serial = torch.as_tensor(np.where(rng.random((lanes, slots)) < 0.5, -1, rng.permutation(lanes * slots).reshape(lanes, slots))).to("cuda:0")
    engine.hitscan_decal_wall = torch.as_tensor(rng.integers(0, len(smap.wall_segments), (lanes, slots))).to("cuda:0")
    engine.hitscan_decal_along = torch.as_tensor(rng.random((lanes, slots)).astype(np.float32)).to("cuda:0")
    engine.hitscan_decal_z = torch.as_tensor((rng.random((lanes, slots)) * 80).astype(np.float32)).to("cuda:0")
    engine.hitscan_decal_style = torch.as_tensor(rng.integers(0, 40, (lanes, slots))).to("cuda:0")
    engine.map.portal_walls = torch.as_tensor(smap.wall_segments).to("cuda:0")
    decal_patches = dict(
        bullet_decal_atlas=overlays["decal_atlas"], bullet_decal_heights=overlays["decal_h"], bullet_decal_left_offsets=overlays["decal_left"],
        bullet_decal_top_offsets=overlays["decal_top"], bullet_decal_opacity_lut=overlays["decal_opacity_lut"],
        bullet_decal_black_lut=overlays["decal_black_lut"],
    )
    adapter = reference_adapter.HipReferenceRenderer(engine, compiled_scenario(smap, overlays, **decal_patches))
    assert adapter._has_decals
    adapter.finish_observation()            # first call: whatever is built lazily
    torch.cuda.synchronize()
    before = engine.frames.clone()
    torch.cuda.set_sync_debug_mode("error")
    try:
        adapter.finish_observation()
        state = adapter.lane_state(include_hud=True)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    torch.cuda.synchronize()
    assert state.decal_state.shape == (lanes, slots, 3) and state.flash_light.dtype == torch.int64
    assert torch.equal(engine.frames[:, 3], before[:, 3]) and torch.equal(engine.frames[:, 2], before[:, 3])
    assert adapter.renderer.status() == 0
    adapter.close()
