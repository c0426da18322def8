"""Torch-facing front end of the HIP renderer.

Mirrors the seam the reference's environment plugs a renderer into
(``/root/reference/src/gradoom/env.py:444-447``): ``render_frame() -> uint8 [N,84,84]``,
``render_native_frame(include_hud) -> uint8 [N,240,320,3]``, and the engine-owned
``frames`` stack updated by ``_finish_observation`` (``engine.py:9545-9548``) or filled
on reset (``engine.py:2443-2450``).  Tensors stay Torch (ROCm) tensors; this module only
passes their device pointers and the current stream through the C ABI.
"""

from __future__ import annotations

import ctypes as C
import dataclasses

import numpy as np
import torch

from . import _abi, _lib, hostmath, mapbuild

STAGES = ("wall_setup", "wall_select", "wall_raster", "plane_shade", "flat_select", "flat_repair", "sprite_columns", "observe")


@dataclasses.dataclass
class LaneState:
    """Per-lane camera tensors, named like the reference engine's own attributes."""

    x: torch.Tensor  # f32 [N]
    y: torch.Tensor
    angle: torch.Tensor
    view_z: torch.Tensor
    x_fixed: torch.Tensor  # i64 [N] (engine._x_fixed)
    y_fixed: torch.Tensor
    angle_bam: torch.Tensor  # i64 [N] (engine._angle_bam)
    pitch_bam: torch.Tensor
    flash_light: torch.Tensor  # i64 [N]
    sprite_x: torch.Tensor | None = None  # f32 [N,A]
    sprite_y: torch.Tensor | None = None
    sprite_z: torch.Tensor | None = None
    sprite_id: torch.Tensor | None = None  # i32 [N,A]
    sprite_alive: torch.Tensor | None = None  # bool/u8 [N,A]
    sprite_fullbright: torch.Tensor | None = None
    # Optional overrides of the Torch-computed float32 inputs (golden fixtures carry the
    # reference's own CPU values so that parity is independent of the Torch build).
    ray_cos: torch.Tensor | None = None
    ray_sin: torch.Tensor | None = None
    sprite_depth: torch.Tensor | None = None
    # Overlay layers (see overlay_inputs.py); drawn when the renderer holds overlay patches.
    weapon_state: torch.Tensor | None = None  # i64 [N,5]
    hud_state: torch.Tensor | None = None  # i32 [N,9]
    sprite_style: torch.Tensor | None = None  # i8 [N,A]: -1 opaque, -2 translucent, >= 0 additive table
    screen_blend: torch.Tensor | None = None  # f32 [N,2] bonus / damage alphas (overlay_inputs.screen_blend)
    decal_state: torch.Tensor | None = None  # i32 [N,D,3] packed wall decals (overlay_inputs.decal_inputs)
    decal_geom: torch.Tensor | None = None  # f32 [N,D,4]

    def select(self, index) -> "LaneState":
        """The lanes ``index`` picks (a slice or an index tensor), every field cut alike and made contiguous."""

        fields = {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}
        return LaneState(**{name: None if value is None else value[index].contiguous() for name, value in fields.items()})

    @classmethod
    def from_numpy(cls, arrays: dict, device) -> "LaneState":
        def get(name, dtype):
            value = arrays.get(name)
            if value is None:
                return None
            return torch.as_tensor(np.ascontiguousarray(value)).to(device=device, dtype=dtype).contiguous()

        return cls(
            x=get("x", torch.float32), y=get("y", torch.float32), angle=get("angle", torch.float32),
            view_z=get("view_z", torch.float32), x_fixed=get("x_fixed", torch.int64), y_fixed=get("y_fixed", torch.int64),
            angle_bam=get("angle_bam", torch.int64), pitch_bam=get("pitch_bam", torch.int64),
            flash_light=get("flash_light", torch.int64), sprite_x=get("sprite_x", torch.float32),
            sprite_y=get("sprite_y", torch.float32), sprite_z=get("sprite_z", torch.float32),
            sprite_id=get("sprite_id", torch.int32), sprite_alive=get("sprite_alive", torch.uint8),
            sprite_fullbright=get("sprite_fullbright", torch.uint8), ray_cos=get("ray_cos", torch.float32),
            ray_sin=get("ray_sin", torch.float32), sprite_depth=get("sprite_depth", torch.float32),
            weapon_state=get("weapon_state", torch.int64), hud_state=get("hud_state", torch.int32),
            sprite_style=get("sprite_style", torch.int8), screen_blend=get("screen_blend", torch.float32),
            decal_state=get("decal_state", torch.int32), decal_geom=get("decal_geom", torch.float32),
        )


def _require(tensor: torch.Tensor, name: str, dtype, shape, device) -> torch.Tensor:
    # Same error classes as the reference's tensor validation (env.py:711-728).
    if not isinstance(tensor, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if tensor.device != device:
        raise TypeError(f"{name} must be on {device}, got {tensor.device}")
    if tensor.dtype != dtype:
        raise TypeError(f"{name} must have dtype {dtype}, got {tensor.dtype}")
    if tuple(tensor.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(tensor.shape)}")
    if not tensor.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return tensor


class HipRenderer:
    """Owns a ``gd_renderer`` for one map on one device."""

    def __init__(self, smap, max_lanes: int, device="cuda:0", *, cosine_correction=None, tables=None):
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("HipRenderer needs a ROCm device; there is no CPU fallback")
        self._lib = _lib.library()
        self.tables = mapbuild.build_map_tables(smap) if tables is None else tables
        self.max_lanes = int(max_lanes)
        self.chunk_lanes = min(self.max_lanes, 4096)  # lanes per kernel launch (library working-memory chunk)
        if cosine_correction is None:
            # the same Torch ops on the same device as the ray tables and billboard depths this renderer derives per frame
            # (_lanes_desc): the stand-alone path is the reference's arithmetic on that device (engine.py:1527-1531, 2050-2054)
            cosine_correction = hostmath.cosine_correction(self.device).cpu().numpy()
        self._cosine = np.ascontiguousarray(cosine_correction, dtype=np.float32)
        if self._cosine.shape != (_abi.SCREEN_WIDTH,):
            raise ValueError("cosine_correction must hold 320 floats")
        self.ray_offsets = hostmath.native_ray_offsets(self.device)
        self.playpal = torch.as_tensor(self.tables["playpal"]).to(self.device).contiguous()
        desc, keep = _abi.host_map_desc(self.tables)
        handle = C.c_void_p()
        with torch.cuda.device(self.device):
            _lib.check(self._lib.gd_renderer_create(C.byref(desc), self._cosine.ctypes.data, self.max_lanes, C.byref(handle)))
        del keep
        self._handle = handle
        from . import ops  # noqa: PLC0415

        self.token = ops.register_renderer(self)   # names this renderer in torch.ops.gradoom_amd.render_ calls

    def close(self) -> None:
        if getattr(self, "_handle", None):
            self._lib.gd_renderer_destroy(self._handle)
            self._handle = None

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass

    def status(self) -> int:
        value = C.c_int32()
        _lib.check(self._lib.gd_renderer_status(self._handle, C.byref(value)))
        return int(value.value)

    def set_assembly(self, assembly: str) -> None:
        """``"separate"`` (kernel by kernel through a frame in device memory, the caller's or the working memory's own),
        ``"fused"`` (every frame is put together band by band in LDS and never reaches device memory unless asked for: a
        fifth less traffic in the assembly, nine tenths of the speed) or ``"auto"`` (the default: separate).  Both give the same bytes."""

        codes = {"auto": 0, "fused": 1, "separate": 2}
        if assembly not in codes:
            raise ValueError("assembly must be 'auto', 'fused' or 'separate'")
        _lib.check(self._lib.gd_renderer_set_assembly(self._handle, codes[assembly]))

    def scribble(self, value: int) -> None:
        """Fill the working memory with one byte value (diagnostic: later frames must not depend on it)."""

        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(self._lib.gd_renderer_scribble(self._handle, int(value), C.c_void_p(stream)))

    def set_overlays(self, overlays: dict) -> None:
        """Upload the weapon and status bar patches (NumPy arrays named like ``gd_overlay_desc``'s fields).

        Afterwards lanes that carry ``weapon_state`` / ``hud_state`` get the psprite over the view and
        the status bar in rows 208..239 (``engine.py:15051-15110``, ``15232-15267``).
        """

        if self._handle is None:
            raise RuntimeError("renderer is closed")
        desc, keep = _abi.host_overlay_desc(overlays)
        with torch.cuda.device(self.device):
            _lib.check(self._lib.gd_renderer_set_overlays(self._handle, C.byref(desc)))
        del keep

    def set_sector_lights(self, lights: torch.Tensor) -> None:
        """Replace the per-sector light levels (float32 [S] on the device) for later frames."""

        count = int(self.tables["sector_count"])
        _require(lights, "lights", torch.float32, (count,), self.device)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(self._lib.gd_renderer_set_sector_lights(self._handle, lights.data_ptr(), C.c_void_p(stream)))

    # ------------------------------------------------------------------ descriptors
    def _lanes_desc(self, lanes: LaneState):
        count = int(lanes.x.shape[0])
        device = self.device
        keep = []
        desc = _abi.LanesDesc()
        desc.lane_count = count
        for name in ("x", "y", "angle", "view_z"):
            setattr(desc, name, _require(getattr(lanes, name), name, torch.float32, (count,), device).data_ptr())
        for name in ("x_fixed", "y_fixed", "angle_bam", "pitch_bam", "flash_light"):
            setattr(desc, name, _require(getattr(lanes, name), name, torch.int64, (count,), device).data_ptr())
        if lanes.ray_cos is None or lanes.ray_sin is None:
            ray_cos, ray_sin = hostmath.ray_tables(lanes.angle, self.ray_offsets)
        else:
            ray_cos, ray_sin = lanes.ray_cos, lanes.ray_sin
        keep += [ray_cos, ray_sin]
        desc.ray_cos = _require(ray_cos, "ray_cos", torch.float32, (count, 320), device).data_ptr()
        desc.ray_sin = _require(ray_sin, "ray_sin", torch.float32, (count, 320), device).data_ptr()
        desc.sprite_slots = 0
        if lanes.sprite_x is not None and lanes.sprite_x.shape[1] > 0:
            slots = int(lanes.sprite_x.shape[1])
            desc.sprite_slots = slots
            for name in ("sprite_x", "sprite_y", "sprite_z"):
                setattr(desc, name, _require(getattr(lanes, name), name, torch.float32, (count, slots), device).data_ptr())
            desc.sprite_id = _require(lanes.sprite_id, "sprite_id", torch.int32, (count, slots), device).data_ptr()
            alive = lanes.sprite_alive
            if alive.dtype == torch.bool:
                alive = alive.to(torch.uint8)
            keep.append(alive)
            desc.sprite_alive = _require(alive, "sprite_alive", torch.uint8, (count, slots), device).data_ptr()
            if lanes.sprite_fullbright is not None:
                bright = lanes.sprite_fullbright
                if bright.dtype == torch.bool:
                    bright = bright.to(torch.uint8)
                keep.append(bright)
                desc.sprite_fullbright = _require(bright, "sprite_fullbright", torch.uint8, (count, slots), device).data_ptr()
            if lanes.sprite_style is not None:
                desc.sprite_style = _require(lanes.sprite_style, "sprite_style", torch.int8, (count, slots), device).data_ptr()
            depth = lanes.sprite_depth
            if depth is None:
                depth = hostmath.sprite_depth(lanes.x, lanes.y, lanes.angle, lanes.sprite_x, lanes.sprite_y)
            keep.append(depth)
            desc.sprite_depth = _require(depth, "sprite_depth", torch.float32, (count, slots), device).data_ptr()
        if lanes.weapon_state is not None:
            desc.weapon_state = _require(lanes.weapon_state, "weapon_state", torch.int64, (count, 5), device).data_ptr()
        desc.decal_slots = 0
        if lanes.decal_state is not None and lanes.decal_state.shape[1] > 0:
            slots = int(lanes.decal_state.shape[1])
            desc.decal_slots = slots
            desc.decal_state = _require(lanes.decal_state, "decal_state", torch.int32, (count, slots, 3), device).data_ptr()
            desc.decal_geom = _require(lanes.decal_geom, "decal_geom", torch.float32, (count, slots, 4), device).data_ptr()
        if lanes.screen_blend is not None:
            desc.screen_blend = _require(lanes.screen_blend, "screen_blend", torch.float32, (count, 2), device).data_ptr()
        if lanes.hud_state is not None:
            desc.hud_state = _require(lanes.hud_state, "hud_state", torch.int32, (count, 9), device).data_ptr()
        return desc, keep

    def _out_desc(self, count, indexed, obs, frames, reset_mask, rgb, stack_only_masked=False, final_frames=None, obs_source_rows=208,
                  final_layout="chw"):
        device = self.device
        out = _abi.FrameOut()
        out.stack_mode = _abi.STACK_RESET if stack_only_masked else _abi.STACK_STEP
        if obs_source_rows not in (208, 240):
            raise ValueError("obs_source_rows must be 208 (status bar masked) or 240 (status bar pooled)")
        out.obs_source_rows = int(obs_source_rows)
        keep = []
        if indexed is not None:
            out.indexed = _require(indexed, "indexed", torch.uint8, (count, 240, 320), device).data_ptr()
        if obs is not None:
            out.obs = _require(obs, "obs", torch.uint8, (count, 84, 84), device).data_ptr()
        if frames is not None:
            out.frames = _require(frames, "frames", torch.uint8, (count, 4, 84, 84), device).data_ptr()
        if reset_mask is not None:
            mask = reset_mask.to(torch.uint8) if reset_mask.dtype == torch.bool else reset_mask
            keep.append(mask)
            out.reset_mask = _require(mask, "reset_mask", torch.uint8, (count,), device).data_ptr()
        if rgb is not None:
            out.rgb = _require(rgb, "rgb", torch.uint8, (count, 240, 320, 3), device).data_ptr()
        if final_frames is not None:
            if frames is None:
                raise ValueError("final_frames needs frames")
            if final_layout not in ("chw", "hwc"):
                raise ValueError("final_layout must be 'chw' or 'hwc'")
            shape = (count, 4, 84, 84) if final_layout == "chw" else (count, 84, 84, 4)
            out.final_frames = _require(final_frames, "final_frames", torch.uint8, shape, device).data_ptr()
            out.final_frames_layout = _abi.LAYOUT_HWC if final_layout == "hwc" else _abi.LAYOUT_CHW
        return out, keep

    # ------------------------------------------------------------------ entry points
    def render(self, lanes: LaneState, *, indexed=None, obs=None, frames=None, reset_mask=None, rgb=None,
               stack_only_masked: bool = False, final_frames=None, obs_source_rows: int = 208, final_layout: str = "chw") -> None:
        """One frame for every lane, written into the given (preallocated) tensors.

        ``frames`` is rolled by one and the new observation appended (``engine.py:9545-9548``); lanes
        whose ``reset_mask`` is set get four copies instead (``engine.py:2443-2450``).  With
        ``stack_only_masked`` the unmasked lanes' stacks are left untouched (the reset call).
        ``final_frames`` also receives every lane's stack as the call leaves it: the clone that
        ``step_and_reset_device`` returns as ``final_observations`` (``env.py:915-917``), written by
        the observation kernel itself.  ``obs_source_rows=240`` pools the status bar rows into the observation
        instead of masking them black, as an environment made with ``obs_crop=None`` does (``env.py:441``,
        ``engine.py:15440``).  ``final_layout="hwc"`` makes ``final_frames`` a ``(N, 84, 84, 4)`` tensor holding
        what ``frames.permute(0, 2, 3, 1)`` shows: the buffer an ``obs_layout="hwc"`` environment hands out
        (``env.py:678-688``).
        """

        if self._handle is None:
            raise RuntimeError("renderer is closed")
        desc, keep_lanes = self._lanes_desc(lanes)
        out, keep_out = self._out_desc(desc.lane_count, indexed, obs, frames, reset_mask, rgb, stack_only_masked, final_frames, obs_source_rows,
                                       final_layout)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(self._lib.gd_render(self._handle, C.byref(desc), C.byref(out), C.c_void_p(stream)))
        del keep_lanes, keep_out

    def render_static(self, lanes: LaneState, *, indexed=None, obs=None, frames=None, reset_mask=None, rgb=None,
                      stack_only_masked: bool = False, final_frames=None, obs_source_rows: int = 208, final_layout: str = "chw") -> None:
        """``render`` through the entry point that allocates nothing (``gd_render_static``): the working memory is
        the library's fixed per-GPU array, so a renderer created with ``max_lanes=0`` can call it.  Same arguments
        as ``render``.  Calls that overlap on one GPU race; ``ValueError`` when one lane of the map does not fit the array."""

        if self._handle is None:
            raise RuntimeError("renderer is closed")
        desc, keep_lanes = self._lanes_desc(lanes)
        out, keep_out = self._out_desc(desc.lane_count, indexed, obs, frames, reset_mask, rgb, stack_only_masked, final_frames, obs_source_rows,
                                       final_layout)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(self._lib.gd_render_static(self._handle, C.byref(desc), C.byref(out), C.c_void_p(stream)))
        del keep_lanes, keep_out

    def render_timed(self, lanes: LaneState, launches: int, *, indexed=None, obs=None, frames=None) -> dict[str, float]:
        """Average milliseconds per launch of each kernel stage (HIP events on the current stream)."""

        desc, keep_lanes = self._lanes_desc(lanes)
        out, keep_out = self._out_desc(desc.lane_count, indexed, obs, frames, None, None)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        times = (C.c_float * len(STAGES))()
        _lib.check(
            self._lib.gd_render_timed(self._handle, C.byref(desc), C.byref(out), C.c_void_p(stream), int(launches), times, len(STAGES))
        )
        del keep_lanes, keep_out
        return {name: float(times[i]) for i, name in enumerate(STAGES)}

    def observe(self, indexed: torch.Tensor, *, obs=None, frames=None, reset_mask=None, stack_only_masked: bool = False) -> None:
        """Observation pipeline on an existing ``[N,208|240,320]`` indexed frame."""

        if indexed.ndim != 3 or tuple(indexed.shape[1:]) not in ((208, 320), (240, 320)):
            raise ValueError("indexed must have shape (N, 208, 320) or (N, 240, 320)")
        if indexed.dtype != torch.uint8:
            raise TypeError("indexed must be a uint8 tensor")
        count, rows = int(indexed.shape[0]), int(indexed.shape[1])
        out, keep = self._out_desc(count, None, obs, frames, reset_mask, None, stack_only_masked)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(
            self._lib.gd_observe(
                indexed.contiguous().data_ptr(), rows, self.playpal.data_ptr(), count, out.obs, out.frames, out.reset_mask,
                out.stack_mode, C.c_void_p(stream),
            )
        )
        del keep

    def expand_rgb24(self, indexed: torch.Tensor, rgb: torch.Tensor) -> None:
        count, rows = int(indexed.shape[0]), int(indexed.shape[1])
        _require(indexed, "indexed", torch.uint8, (count, rows, 320), self.device)
        _require(rgb, "rgb", torch.uint8, (count, rows, 320, 3), self.device)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _lib.check(
            self._lib.gd_expand_rgb24(indexed.data_ptr(), rows, self.playpal.data_ptr(), count, rgb.data_ptr(), C.c_void_p(stream))
        )
