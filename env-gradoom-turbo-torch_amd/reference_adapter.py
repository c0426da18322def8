"""The library behind the reference's own renderer interface.

``GraDoomVecEnv`` selects its observation renderer by rebinding one engine attribute
(``/root/reference/src/gradoom/env.py:444-447``)::

    self._engine.render_frame = self._engine.render_reference_frame

``HipReferenceRenderer(engine, scenario)`` offers methods with the signatures and results of the
engine methods on that path, computed by ``gd_render`` from the engine's own tensors:

* ``render_reference_frame(active=None) -> uint8 [N, 84, 84]``           (``engine.py:15436-15451``)
* ``render_native_indexed_frame(include_hud=True) -> uint8 [N, 240|208, 320]``  (``engine.py:15338-15379``)
* ``render_native_frame(include_hud=True) -> uint8 [N, 240|208, 320, 3]``       (``engine.py:15453-15457``)
* ``finish_observation()``: ``_finish_observation(render_frame())`` in one call (``engine.py:9545-9548``)
* ``reset_stack(mask)``: the four-copy fill of ``reset`` (``engine.py:2443-2450``)

``install()`` rebinds the engine attributes.  ``policy_area_grayscale(indexed, palette)`` is the
stand-alone pooling operator of ``_triton_kernels.py:180-203`` with its argument checks.

The engine is anything that carries the reference engine's attribute names (a ``SimpleNamespace`` of
tensors will do); the scenario anything that carries ``CompiledScenario``'s (``scenario.py:302-401``).
"""

from __future__ import annotations

import numpy as np
import torch

from . import actor_inputs, hostmath, overlay_inputs
from .mapfile import ScenarioView, _host
from .renderer import HipRenderer, LaneState

SCREEN_WIDTH, VIEW_HEIGHT, SCREEN_HEIGHT = 320, 208, 240


def scenario_overlays(scenario) -> dict | None:
    """The weapon, status bar and bullet chip patches of a scenario under ``gd_overlay_desc``'s names, or None.

    ``native_weapon_patch_*`` (``scenario.py:382-387``), ``hud_patch_*`` (``scenario.py:391-397``) and
    ``bullet_decal_*`` (``scenario.py:371-376``).
    """

    if getattr(scenario, "native_weapon_patch_atlas", None) is None or getattr(scenario, "hud_patch_atlas", None) is None:
        return None
    overlays = {}
    for prefix, source in (("weapon", "native_weapon_patch"), ("hud", "hud_patch")):
        overlays[f"{prefix}_atlas"] = _host(getattr(scenario, f"{source}_atlas"), np.uint8)
        overlays[f"{prefix}_opaque"] = _host(getattr(scenario, f"{source}_opaque"), np.uint8)
        for short, long in (("w", "widths"), ("h", "heights"), ("left", "left_offsets"), ("top", "top_offsets")):
            overlays[f"{prefix}_{short}"] = _host(getattr(scenario, f"{source}_{long}"), np.int32)
    if getattr(scenario, "bullet_decal_atlas", None) is not None:
        overlays["decal_atlas"] = _host(scenario.bullet_decal_atlas, np.uint8)
        for short, long in (("h", "heights"), ("left", "left_offsets"), ("top", "top_offsets")):
            overlays[f"decal_{short}"] = _host(getattr(scenario, f"bullet_decal_{long}"), np.int32)
        overlays["decal_opacity_lut"] = _host(scenario.bullet_decal_opacity_lut, np.uint8)
        overlays["decal_black_lut"] = _host(scenario.bullet_decal_black_lut, np.uint8)
    return overlays


WEAPON_ARGUMENTS = (
    "active_weapon", "weapon_state_cooldown", "weapon_fire_count", "weapon_ready_tics", "weapon_lower_cooldown",
    "weapon_raise_cooldown", "pending_weapon", "episode_time", "player_bob_fixed", "player_dead",
)
HUD_ARGUMENTS = (
    "active_weapon", "weapon_ammo_slot", "hud_ready_ammo", "health", "armor", "weapons", "hud_ammo_counts",
    "mugshot_face_index", "mugshot_grin_tics", "mugshot_pain_tics", "mugshot_ouch", "mugshot_pain_direction",
    "attack_held_tics",
)
# overlay_inputs argument -> engine attribute, where the names differ (engine.py:14949-14967, 15240-15262)
_ENGINE_NAMES = {"player_bob_fixed": "_player_bob_fixed", "weapon_ammo_slot": "_weapon_ammo_slot"}


def overlay_engine_tensors(engine) -> dict[str, torch.Tensor]:
    """The gameplay tensors the weapon and status bar layers read, by ``overlay_inputs`` argument name."""

    tensors = {}
    for name in dict.fromkeys(WEAPON_ARGUMENTS + HUD_ARGUMENTS):
        if name == "active_weapon":
            tensors[name] = engine._active_weapon()
        else:
            tensors[name] = getattr(engine, _ENGINE_NAMES.get(name, name))
    return tensors


class HipReferenceRenderer:
    """``gd_render`` driven from a reference engine's tensors, behind the engine's render methods."""

    def __init__(self, engine, scenario, *, renderer=None, fused_actors: bool | None = None, actor_limit: int = 512):
        self.engine = engine
        self.num_envs = int(engine.num_envs)
        self.device = torch.device(engine.device)
        offsets = getattr(engine, "_native_ray_offsets", None)
        self._ray_offsets = hostmath.native_ray_offsets(self.device) if offsets is None else offsets
        if renderer is None:
            cosine = torch.cos(self._ray_offsets.to(torch.float32)).cpu().numpy()   # engine.py:1527-1531
            renderer = HipRenderer(ScenarioView(scenario), self.num_envs, self.device, cosine_correction=cosine)
        self.renderer = renderer
        self._overlays = scenario_overlays(scenario)
        if self._overlays is not None:
            renderer.set_overlays(self._overlays)
            m = engine.map
            self._weapon_frame_ids = torch.as_tensor(m.native_weapon_frame_ids).to(self.device)
            self._weapon_flash_ids = torch.as_tensor(m.native_weapon_flash_ids).to(self.device)
            self._fine_sine = torch.as_tensor(overlay_inputs.fine_sine_fixed()).to(self.device)
        self._fused_actors = (self.device.type == "cuda") if fused_actors is None else bool(fused_actors)
        self._actor_limit = int(actor_limit)
        self._has_actors = hasattr(engine, "enemy_x")
        self._has_decals = self._overlays is not None and "decal_atlas" in self._overlays and hasattr(engine, "hitscan_decal_serial")

    # ------------------------------------------------------------------ engine tensors -> lane descriptor
    def lane_state(self, *, include_hud: bool = False) -> LaneState:
        """Everything ``gd_lanes_desc`` takes, from the engine as it stands (no copies of the pose tensors)."""

        e = self.engine
        contiguous = lambda t: t if t.is_contiguous() else t.contiguous()  # noqa: E731
        fields = dict(
            x=contiguous(e.x), y=contiguous(e.y), angle=contiguous(e.angle), view_z=contiguous(e.view_z),
            x_fixed=contiguous(e._x_fixed), y_fixed=contiguous(e._y_fixed), angle_bam=contiguous(e._angle_bam),
            pitch_bam=contiguous(e._pitch_bam),
        )
        flash = None   # extralight of the muzzle flash, engine.py:14949-14967
        ray_cos, ray_sin = hostmath.ray_tables(e.angle, self._ray_offsets)
        fields.update(ray_cos=ray_cos, ray_sin=ray_sin)
        if self._has_actors:
            pack = actor_inputs.pack_actors_fused if self._fused_actors else actor_inputs.pack_actors
            packed = pack(e, limit=self._actor_limit)
            fields.update(packed)
            fields["sprite_depth"] = hostmath.sprite_depth(e.x, e.y, e.angle, packed["sprite_x"], packed["sprite_y"])
        if self._overlays is not None:
            tensors = overlay_engine_tensors(e)
            # the weapon words and, where the map carries the table, the flash's extra light: one kernel, no host round trip
            lights = getattr(e.map, "native_weapon_flash_lights", None)
            packed = overlay_inputs.weapon_state(
                **{k: tensors[k] for k in WEAPON_ARGUMENTS}, weapon_frame_ids=self._weapon_frame_ids,
                weapon_flash_ids=self._weapon_flash_ids, fine_sine=self._fine_sine,
                weapon_flash_lights=lights, want_flash_light=lights is not None,
            )
            fields["weapon_state"], flash = packed if lights is not None else (packed, None)
            if include_hud:
                fields["hud_state"] = overlay_inputs.hud_state(**{k: tensors[k] for k in HUD_ARGUMENTS})
        if self._has_decals:
            state, geometry = overlay_inputs.decal_inputs(
                e.hitscan_decal_serial, e.hitscan_decal_wall, e.hitscan_decal_along, e.hitscan_decal_z, e.hitscan_decal_style,
                e.map.portal_walls, self._fine_sine,
            )
            fields.update(decal_state=state, decal_geom=geometry)
        if flash is None:
            flash = e._native_weapon_frame_selection()[2]
        fields["flash_light"] = flash.to(torch.int64).contiguous()
        if getattr(e, "render_screen_flashes", False):
            fields["screen_blend"] = overlay_inputs.screen_blend(e.bonus_count, e.damage_count, e._damage_to_alpha)
        return LaneState(**fields)

    def _source_rows(self) -> int:
        return VIEW_HEIGHT if getattr(self.engine, "mask_hud", True) else SCREEN_HEIGHT   # engine.py:15440

    # ------------------------------------------------------------------ the engine's render methods
    def render_reference_frame(self, active: torch.Tensor | None = None) -> torch.Tensor:
        del active   # every lane is rendered, as in the reference (engine.py:15439)
        rows = self._source_rows()
        obs = torch.empty((self.num_envs, 84, 84), dtype=torch.uint8, device=self.device)
        self.renderer.render(self.lane_state(include_hud=rows == SCREEN_HEIGHT), obs=obs, obs_source_rows=rows)
        return obs

    def render_native_indexed_frame(self, *, include_hud: bool = True) -> torch.Tensor:
        indexed = torch.empty((self.num_envs, SCREEN_HEIGHT, SCREEN_WIDTH), dtype=torch.uint8, device=self.device)
        self.renderer.render(self.lane_state(include_hud=include_hud), indexed=indexed)
        return indexed if include_hud else indexed[:, :VIEW_HEIGHT]

    def render_native_frame(self, *, include_hud: bool = True) -> torch.Tensor:
        rgb = torch.empty((self.num_envs, SCREEN_HEIGHT, SCREEN_WIDTH, 3), dtype=torch.uint8, device=self.device)
        self.renderer.render(self.lane_state(include_hud=include_hud), rgb=rgb)
        return rgb if include_hud else rgb[:, :VIEW_HEIGHT]

    def finish_observation(self) -> torch.Tensor:
        """Roll ``engine.frames`` by one and append this frame's observation, in the render call itself."""

        rows = self._source_rows()
        self.renderer.render(self.lane_state(include_hud=rows == SCREEN_HEIGHT), frames=self.engine.frames, obs_source_rows=rows)
        return self.engine.frames

    def reset_stack(self, mask: torch.Tensor) -> torch.Tensor:
        """Fill the stacks of the masked lanes with four copies of this frame's observation."""

        rows = self._source_rows()
        self.renderer.render(self.lane_state(include_hud=rows == SCREEN_HEIGHT), frames=self.engine.frames, reset_mask=mask,
                             stack_only_masked=True, obs_source_rows=rows)
        return self.engine.frames

    def install(self) -> None:
        """Rebind the engine's render attributes, as ``env.py:444-447`` does for the built-in renderers."""

        self.engine.render_frame = self.render_reference_frame
        self.engine.render_reference_frame = self.render_reference_frame
        self.engine.render_native_frame = self.render_native_frame
        self.engine._render_native_indexed_frame = self.render_native_indexed_frame

    def close(self) -> None:
        self.renderer.close()


# The stand-alone pooling operator (``_triton_kernels.py:180-203``): a registered Torch operator with a fake
# implementation, see ``ops.py``.
from .ops import policy_area_grayscale  # noqa: E402,F401
