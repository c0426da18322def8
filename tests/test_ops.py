"""The kernels as registered Torch operators (``gradoom_amd::policy_area_grayscale``, ``gradoom_amd::render_``).

Mirrors how the reference exposes its kernels (``/root/reference/src/gradoom/_triton_kernels.py:180-212``: a
``torch.library.custom_op`` with a fake implementation; ``_kernels.py:8-65``: stubs raising ``RuntimeError`` when the
backend is absent).  CPU tests cover the schemas, the fake implementations and the stub binding; the GPU test traces
both operators through ``torch.compile(fullgraph=True)`` and compares with the direct calls.
"""

from __future__ import annotations

import importlib
import sys

import numpy as np
import pytest
import torch

from conftest import lane_inputs, load_fixture


def test_schemas_declare_what_the_operators_write():
    from gradoom_amd import ops  # noqa: F401  (registers the operators)

    pool = torch.ops.gradoom_amd.policy_area_grayscale.default._schema
    assert str(pool) == "gradoom_amd::policy_area_grayscale(Tensor indexed, Tensor palette) -> Tensor"
    assert not pool.is_mutable
    render = torch.ops.gradoom_amd.render_.default._schema
    written = {argument.name for argument in render.arguments if argument.alias_info is not None and argument.alias_info.is_write}
    assert written == {"indexed", "obs", "frames", "rgb", "final_frames"}
    assert str(render.returns) == "[]" or len(render.returns) == 0


def test_fake_implementations_give_shapes_without_running_a_kernel():
    from torch._subclasses.fake_tensor import FakeTensorMode

    from gradoom_amd import ops  # noqa: F401

    with FakeTensorMode():
        palette = torch.empty((256, 3), dtype=torch.uint8)
        for rows in (208, 240):
            out = torch.ops.gradoom_amd.policy_area_grayscale(torch.empty((7, rows, 320), dtype=torch.uint8), palette)
            assert tuple(out.shape) == (7, 84, 84) and out.dtype == torch.uint8
        assert tuple(torch.ops.gradoom_amd.policy_area_grayscale(torch.empty((0, 208, 320), dtype=torch.uint8), palette).shape) == (0, 84, 84)
        f32 = lambda: torch.empty(5, dtype=torch.float32)  # noqa: E731
        i64 = lambda: torch.empty(5, dtype=torch.int64)  # noqa: E731
        pose = (f32(), f32(), f32(), f32(), i64(), i64(), i64(), i64(), i64())
        frames = torch.empty((5, 4, 84, 84), dtype=torch.uint8)
        # written tensors by position: indexed, obs, frames, rgb, final_frames
        assert torch.ops.gradoom_amd.render_(1, torch.empty((5, 240, 320), dtype=torch.uint8), None, frames, None, None, *pose) is None
        torch.ops.gradoom_amd.render_(1, None, None, frames, None, torch.empty((5, 84, 84, 4), dtype=torch.uint8), *pose, final_hwc=True)
        with pytest.raises(ValueError, match=r"obs must have shape \(5, 84, 84\)"):
            torch.ops.gradoom_amd.render_(1, None, torch.empty((4, 84, 84), dtype=torch.uint8), None, None, None, *pose)
        with pytest.raises(TypeError, match="rgb must have dtype torch.uint8"):
            torch.ops.gradoom_amd.render_(1, None, None, None, torch.empty((5, 240, 320, 3), dtype=torch.float32), None, *pose)
        with pytest.raises(ValueError, match="obs_source_rows must be 208"):
            torch.ops.gradoom_amd.render_(1, None, None, frames, None, None, *pose, obs_source_rows=200)


def test_operators_are_stubs_when_the_library_is_missing(monkeypatch):
    # _kernels.py:36-40: every name is bound to a function raising RuntimeError when the backend cannot be loaded
    from gradoom_amd import _lib

    def missing():
        raise RuntimeError("libgradoom_amd.so is missing")

    monkeypatch.setattr(_lib, "library", missing)
    monkeypatch.delitem(sys.modules, "gradoom_amd.ops", raising=False)
    try:
        stubbed = importlib.import_module("gradoom_amd.ops")
        assert stubbed._BACKEND_ERROR is not None
        for name in ("policy_area_grayscale", "render_"):
            with pytest.raises(RuntimeError, match="require libgradoom_amd.so and a ROCm-capable Torch"):
                getattr(stubbed, name)(torch.zeros(1), torch.zeros(1))
    finally:
        monkeypatch.undo()
        sys.modules.pop("gradoom_amd.ops", None)
        importlib.import_module("gradoom_amd.ops")


@pytest.mark.gpu
def test_both_operators_trace_through_torch_compile():
    from gradoom_amd import ops
    from gradoom_amd.renderer import HipRenderer, LaneState

    _meta, data, smap, tables = load_fixture("small_midtex_sprites")
    renderer = HipRenderer(smap, 8, "cuda:0", cosine_correction=data["cosine_correction"], tables=tables)
    lanes = LaneState.from_numpy(lane_inputs(data), "cuda:0")
    palette = torch.as_tensor(tables["playpal"]).to("cuda:0")
    token = renderer.token

    def frame_and_observation(x, y, angle, view_z, x_fixed, y_fixed, angle_bam, pitch_bam, flash_light, ray_cos, ray_sin,
                              sprite_x, sprite_y, sprite_z, sprite_id, sprite_alive, sprite_fullbright, sprite_depth, indexed, frames, palette):
        torch.ops.gradoom_amd.render_(
            token, indexed, None, frames, None, None, x, y, angle, view_z, x_fixed, y_fixed, angle_bam, pitch_bam, flash_light,
            ray_cos, ray_sin, sprite_x, sprite_y, sprite_z, sprite_id, sprite_alive, sprite_fullbright, None, sprite_depth,
        )
        pooled = torch.ops.gradoom_amd.policy_area_grayscale(indexed[:, :208].contiguous(), palette)
        return pooled, frames[:, 3] + 0

    arguments = (
        lanes.x, lanes.y, lanes.angle, lanes.view_z, lanes.x_fixed, lanes.y_fixed, lanes.angle_bam, lanes.pitch_bam, lanes.flash_light,
        lanes.ray_cos, lanes.ray_sin, lanes.sprite_x, lanes.sprite_y, lanes.sprite_z, lanes.sprite_id, lanes.sprite_alive,
        lanes.sprite_fullbright, lanes.sprite_depth,
    )
    indexed = torch.zeros((8, 240, 320), dtype=torch.uint8, device="cuda:0")
    frames = torch.zeros((8, 4, 84, 84), dtype=torch.uint8, device="cuda:0")
    compiled = torch.compile(frame_and_observation, fullgraph=True, backend="aot_eager")
    pooled, newest = compiled(*arguments, indexed, frames, palette)
    torch.cuda.synchronize()
    # the traced call wrote the caller's tensors (mutates_args) and equals the reference's frame
    assert np.array_equal(indexed.cpu().numpy(), data["indexed"])
    assert torch.equal(pooled, newest) and torch.equal(frames[:, 3], pooled)
    assert int(np.abs(pooled.cpu().numpy().astype(np.int16) - data["obs"].astype(np.int16)).max()) <= 1
    # and equals the direct calls
    direct_indexed = torch.zeros_like(indexed)
    direct_frames = torch.zeros_like(frames)
    ops.render_lanes_(token, lanes, indexed=direct_indexed, frames=direct_frames)
    assert torch.equal(direct_indexed, indexed) and torch.equal(direct_frames, frames)
    assert torch.equal(ops.policy_area_grayscale(direct_indexed, palette)[:, :72], pooled[:, :72])
    # a second call of the compiled function rolls the stack again (no stale capture of the outputs)
    compiled(*arguments, indexed, frames, palette)
    torch.cuda.synchronize()
    assert torch.equal(frames[:, 2], pooled) and torch.equal(frames[:, 3], pooled)
    renderer.close()
    with pytest.raises(RuntimeError, match="renderer is closed"):
        ops.render_lanes_(token, lanes, indexed=direct_indexed)
