"""The HIP kernels as Torch operators, the way the reference exposes its own.

The reference registers every kernel as ``torch.library.custom_op("gradoom::name", mutates_args=...)`` with a
``register_fake`` shape function, names operators that write into their arguments with a trailing underscore
(``/root/reference/src/gradoom/_triton_kernels.py:180-212``), and binds every name to a stub raising
``RuntimeError`` when the backend cannot be loaded (``/root/reference/src/gradoom/_kernels.py:8-65``).  The same
here, in the namespace ``gradoom_amd``:

* ``policy_area_grayscale(indexed, palette) -> uint8 [N, 84, 84]``  exact area pool + grayscale on palette indices
* ``render_(renderer, indexed, obs, frames, rgb, final_frames, x, y, ...) -> None``  one frame of every lane,
  written into the given tensors (every tensor the call writes is declared in ``mutates_args``)

so that callers can trace them under ``torch.compile`` / ``FakeTensorMode``.  The implementations pass device
pointers and the current stream through the C ABI (``include/gradoom_amd.h``); there is no CPU implementation.
"""

from __future__ import annotations

import ctypes as C
import weakref
from typing import Any, Callable, Optional

import torch

OBS_SIZE = 84
_RENDERERS: "weakref.WeakValueDictionary[int, Any]" = weakref.WeakValueDictionary()
_NEXT_TOKEN = [1]


def register_renderer(renderer) -> int:
    """A small integer that names ``renderer`` in ``render_`` calls (operators take no Python objects)."""

    token = _NEXT_TOKEN[0]
    _NEXT_TOKEN[0] += 1
    _RENDERERS[token] = renderer
    return token


def _unavailable(*_args: Any, **_kwargs: Any) -> Any:
    raise RuntimeError("gradoom_amd HIP kernels require libgradoom_amd.so and a ROCm-capable Torch installation")


try:
    from . import _lib

    _lib.library()
    _BACKEND_ERROR: Optional[BaseException] = None
except (RuntimeError, OSError) as exc:   # the shared library is missing or does not load: bind stubs, as _kernels.py does
    _BACKEND_ERROR = exc

if _BACKEND_ERROR is not None:
    policy_area_grayscale: Callable[..., Any] = _unavailable
    render_: Callable[..., Any] = _unavailable
else:

    @torch.library.custom_op("gradoom_amd::policy_area_grayscale", mutates_args=())
    def policy_area_grayscale(indexed: torch.Tensor, palette: torch.Tensor) -> torch.Tensor:
        """320x240 -> 84x84 area pooling and grayscale on palette indices (``_triton_kernels.py:180-203``).

        ``indexed`` uint8 ``[N, 208|240, 320]`` (208 rows: the status bar counts as black), ``palette`` uint8
        ``[256, 3]``; returns uint8 ``[N, 84, 84]`` on the same device.  Same checks and messages as the reference.
        """

        if indexed.ndim != 3 or tuple(indexed.shape[1:]) not in ((208, 320), (240, 320)):
            raise ValueError("indexed must have shape (N, 208, 320) or (N, 240, 320)")
        if indexed.dtype != torch.uint8 or palette.dtype != torch.uint8:
            raise TypeError("indexed and palette must be uint8 tensors")
        if tuple(palette.shape) != (256, 3):
            raise ValueError("palette must have shape (256, 3)")
        if indexed.device.type != "cuda" or palette.device != indexed.device:
            raise RuntimeError("policy_area_grayscale needs both tensors on one ROCm device; there is no CPU fallback")
        library = _lib.library()
        output = torch.empty((indexed.shape[0], OBS_SIZE, OBS_SIZE), device=indexed.device, dtype=torch.uint8)
        if indexed.shape[0] == 0:
            return output
        source, colours = indexed.contiguous(), palette.contiguous()
        with torch.cuda.device(indexed.device):
            stream = torch.cuda.current_stream(indexed.device).cuda_stream
            _lib.check(library.gd_observe(source.data_ptr(), int(indexed.shape[1]), colours.data_ptr(), int(indexed.shape[0]),
                                          output.data_ptr(), None, None, 0, C.c_void_p(stream)))
        return output

    @policy_area_grayscale.register_fake
    def _policy_area_grayscale_fake(indexed: torch.Tensor, palette: torch.Tensor) -> torch.Tensor:
        del palette
        return torch.empty((indexed.shape[0], OBS_SIZE, OBS_SIZE), device=indexed.device, dtype=torch.uint8)

    @torch.library.custom_op(
        "gradoom_amd::render_", mutates_args=("indexed", "obs", "frames", "rgb", "final_frames"), device_types="cuda",
    )
    def render_(
        renderer: int,
        indexed: Optional[torch.Tensor], obs: Optional[torch.Tensor], frames: Optional[torch.Tensor],
        rgb: Optional[torch.Tensor], final_frames: Optional[torch.Tensor],
        x: torch.Tensor, y: torch.Tensor, angle: torch.Tensor, view_z: torch.Tensor,
        x_fixed: torch.Tensor, y_fixed: torch.Tensor, angle_bam: torch.Tensor, pitch_bam: torch.Tensor, flash_light: torch.Tensor,
        ray_cos: Optional[torch.Tensor] = None, ray_sin: Optional[torch.Tensor] = None,
        sprite_x: Optional[torch.Tensor] = None, sprite_y: Optional[torch.Tensor] = None, sprite_z: Optional[torch.Tensor] = None,
        sprite_id: Optional[torch.Tensor] = None, sprite_alive: Optional[torch.Tensor] = None,
        sprite_fullbright: Optional[torch.Tensor] = None, sprite_style: Optional[torch.Tensor] = None,
        sprite_depth: Optional[torch.Tensor] = None,
        weapon_state: Optional[torch.Tensor] = None, hud_state: Optional[torch.Tensor] = None,
        screen_blend: Optional[torch.Tensor] = None, decal_state: Optional[torch.Tensor] = None,
        decal_geom: Optional[torch.Tensor] = None,
        reset_mask: Optional[torch.Tensor] = None, stack_only_masked: bool = False, obs_source_rows: int = 208,
        final_hwc: bool = False,
    ) -> None:
        """One frame of every lane through ``gd_render``, written into ``indexed`` / ``obs`` / ``frames`` / ``rgb`` /
        ``final_frames`` (whichever are not None; the written tensors come first and are passed by position).
        ``renderer`` is ``HipRenderer.token``.  The lane tensors carry the reference engine's attribute names
        (``renderer.LaneState``)."""

        from .renderer import LaneState

        target = _RENDERERS.get(int(renderer))
        if target is None:
            raise RuntimeError("render_: unknown or closed renderer")
        lanes = LaneState(
            x=x, y=y, angle=angle, view_z=view_z, x_fixed=x_fixed, y_fixed=y_fixed, angle_bam=angle_bam, pitch_bam=pitch_bam,
            flash_light=flash_light, sprite_x=sprite_x, sprite_y=sprite_y, sprite_z=sprite_z, sprite_id=sprite_id,
            sprite_alive=sprite_alive, sprite_fullbright=sprite_fullbright, ray_cos=ray_cos, ray_sin=ray_sin,
            sprite_depth=sprite_depth, weapon_state=weapon_state, hud_state=hud_state, sprite_style=sprite_style,
            screen_blend=screen_blend, decal_state=decal_state, decal_geom=decal_geom,
        )
        target.render(lanes, indexed=indexed, obs=obs, frames=frames, reset_mask=reset_mask, rgb=rgb,
                      stack_only_masked=stack_only_masked, final_frames=final_frames, obs_source_rows=obs_source_rows,
                      final_layout="hwc" if final_hwc else "chw")

    @render_.register_fake
    def _render_fake(renderer, indexed, obs, frames, rgb, final_frames, x, y, angle, view_z, x_fixed, y_fixed, angle_bam, pitch_bam, flash_light, ray_cos=None, ray_sin=None,
                     sprite_x=None, sprite_y=None, sprite_z=None, sprite_id=None, sprite_alive=None, sprite_fullbright=None,
                     sprite_style=None, sprite_depth=None, weapon_state=None, hud_state=None, screen_blend=None, decal_state=None,
                     decal_geom=None, reset_mask=None,
                     stack_only_masked=False, obs_source_rows=208, final_hwc=False) -> None:
        # shape contract of the outputs, checked at trace time (the kernels check it again on real tensors)
        count = x.shape[0]
        for name, tensor, shape in (
            ("indexed", indexed, (count, 240, 320)), ("obs", obs, (count, OBS_SIZE, OBS_SIZE)),
            ("frames", frames, (count, 4, OBS_SIZE, OBS_SIZE)), ("rgb", rgb, (count, 240, 320, 3)),
            ("final_frames", final_frames, (count, OBS_SIZE, OBS_SIZE, 4) if final_hwc else (count, 4, OBS_SIZE, OBS_SIZE)),
        ):
            if tensor is None:
                continue
            if tensor.dtype != torch.uint8:
                raise TypeError(f"{name} must have dtype torch.uint8, got {tensor.dtype}")
            if tuple(tensor.shape) != shape:
                raise ValueError(f"{name} must have shape {shape}, got {tuple(tensor.shape)}")
        if obs_source_rows not in (208, 240):
            raise ValueError("obs_source_rows must be 208 (status bar masked) or 240 (status bar pooled)")
        return None


def render_lanes_(token: int, lanes, *, indexed=None, obs=None, frames=None, reset_mask=None, rgb=None, stack_only_masked: bool = False,
                  final_frames=None, obs_source_rows: int = 208, final_layout: str = "chw") -> None:
    """``render_`` with the lane tensors taken from a ``LaneState``."""

    render_(
        token, indexed, obs, frames, rgb, final_frames, lanes.x, lanes.y, lanes.angle, lanes.view_z, lanes.x_fixed, lanes.y_fixed, lanes.angle_bam, lanes.pitch_bam,
        lanes.flash_light, lanes.ray_cos, lanes.ray_sin, lanes.sprite_x, lanes.sprite_y, lanes.sprite_z, lanes.sprite_id,
        lanes.sprite_alive, lanes.sprite_fullbright, lanes.sprite_style, lanes.sprite_depth, lanes.weapon_state, lanes.hud_state,
        lanes.screen_blend, lanes.decal_state, lanes.decal_geom, reset_mask,
        stack_only_masked, obs_source_rows, final_layout == "hwc",
    )
