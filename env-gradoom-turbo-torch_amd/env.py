"""Device-resident vector-env front end with the reference's render-path contract.

Mirrors the part of ``GraDoomVecEnv`` (``/root/reference/src/gradoom/env.py``) that
the render path serves:

* ``reset_device(mask, seeds) -> (observations, signals)``                      (``env.py:879-907``)
* ``step_device(actions) -> DeviceTransition``                                  (``env.py:851-877``)
* ``step_and_reset_device(actions, reset_seeds) -> DeviceAutoResetTransition``  (``env.py:909-942, 998``)
* ``render() / render_lane(i) / get_images()`` -> ``uint8 (240, 320, 3)``       (``env.py:1037-1064``)
* ``reset(seed=, options=) / step(actions)`` with ``obs_copy`` ownership         (``env.py:750-834, 678-688``)

with the same argument validation (``env.py:711-728``), the same ownership rules
(``observations`` is the renderer-owned ``frames`` stack returned by reference;
``final_*`` are fresh clones; the reset is skipped when no lane is done) and the
same error classes.  Gameplay (movement, combat, rewards) is NOT part of this
package: the lane state that the renderer draws comes from a ``LaneDynamics``
object.  ``PosePoolDynamics`` is a deterministic stand-in that teleports every
lane through a seeded pool of poses; a real engine would implement the same
three methods on top of its own state tensors.
"""

from __future__ import annotations

import dataclasses
import operator
from collections.abc import Sequence

import numpy as np
import torch

from . import hostmath, synthmap
from .renderer import HipRenderer, LaneState

SIGNAL_COUNT = 27  # len(DEVICE_SIGNAL_NAMES), engine.py:509-539
INDEX_DTYPES = (torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8)


@dataclasses.dataclass(frozen=True)
class DeviceTransition:  # env.py:181-190
    observations: torch.Tensor
    rewards: torch.Tensor
    terminated: torch.Tensor
    truncated: torch.Tensor
    signals: torch.Tensor
    info_histories: torch.Tensor


@dataclasses.dataclass(frozen=True)
class DeviceAutoResetTransition:  # env.py:193-205
    observations: torch.Tensor
    rewards: torch.Tensor
    terminated: torch.Tensor
    truncated: torch.Tensor
    signals: torch.Tensor
    info_histories: torch.Tensor
    final_observations: torch.Tensor
    final_signals: torch.Tensor
    final_info_histories: torch.Tensor


def _normalize_seed(seed, num_envs: int):  # env.py:101-113
    if seed is None:
        return [None] * num_envs
    if isinstance(seed, Sequence) and not isinstance(seed, (str, bytes, bytearray)):
        values = [None if value is None else int(value) for value in seed]
        if len(values) != num_envs:
            raise ValueError("seed sequence length must match num_envs")
        return values
    return [int(seed) + lane for lane in range(num_envs)]


class PosePoolDynamics:
    """Deterministic lane state source: lane ``i`` at time ``t`` shows pose ``(seed_i + t) mod pool``."""

    def __init__(self, smap, num_envs: int, device, *, pool: int = 64, sprites: int = 0, episode_timeout: int = 32, seed: int = 0):
        self.device = torch.device(device)
        self.num_envs = num_envs
        self.episode_timeout = int(episode_timeout)
        poses = synthmap.generate_poses_batch(smap, pool, seed, flash=True)
        to = lambda array, dtype: torch.as_tensor(np.ascontiguousarray(array)).to(device=self.device, dtype=dtype)  # noqa: E731
        self._pool = dict(
            x=to(poses.x, torch.float32), y=to(poses.y, torch.float32), view_z=to(poses.view_z, torch.float32),
            angle_bam=to(poses.angle_bam, torch.int64), pitch_bam=to(poses.pitch_bam, torch.int64),
            flash_light=to(poses.flash_light, torch.int64),
        )
        self._pool_size = pool
        self._sprites = None
        if sprites:
            spr = synthmap.generate_sprites_batch(smap, pool, sprites, seed)
            self._sprites = dict(
                sprite_x=to(spr.x, torch.float32), sprite_y=to(spr.y, torch.float32), sprite_z=to(spr.z, torch.float32),
                sprite_id=to(spr.sprite, torch.int32), sprite_alive=to(spr.alive.astype(np.uint8), torch.uint8),
                sprite_fullbright=to(spr.fullbright.astype(np.uint8), torch.uint8),
            )
        self.phase = torch.zeros(num_envs, dtype=torch.int64, device=self.device)
        self.episode_time = torch.zeros(num_envs, dtype=torch.int64, device=self.device)

    def reset(self, mask: torch.Tensor, seeds: torch.Tensor) -> None:
        self.phase.copy_(torch.where(mask, torch.remainder(seeds, self._pool_size), self.phase))
        self.episode_time.copy_(torch.where(mask, torch.zeros_like(self.episode_time), self.episode_time))

    def step(self, actions: torch.Tensor):
        self.phase.copy_(torch.remainder(self.phase + 1 + actions, self._pool_size))
        self.episode_time.add_(1)
        rewards = torch.zeros(self.num_envs, dtype=torch.float32, device=self.device)
        terminated = torch.zeros(self.num_envs, dtype=torch.bool, device=self.device)
        truncated = self.episode_time >= self.episode_timeout
        return rewards, terminated, truncated

    def lane_state(self) -> LaneState:
        index = self.phase
        pool = self._pool
        x, y = pool["x"][index], pool["y"][index]
        bam = pool["angle_bam"][index]
        fields = dict(
            x=x, y=y, angle=hostmath.angle_from_bam(bam), view_z=pool["view_z"][index],
            x_fixed=torch.round(x * 65536).to(torch.int64), y_fixed=torch.round(y * 65536).to(torch.int64),
            angle_bam=bam, pitch_bam=pool["pitch_bam"][index], flash_light=pool["flash_light"][index],
        )
        if self._sprites is not None:
            fields.update({name: value[index].contiguous() for name, value in self._sprites.items()})
        return LaneState(**{name: value.contiguous() for name, value in fields.items()})


class GraDoomVecEnv:
    """Render-path subset of the reference's vector environment (device API only)."""

    frame_stack = 4

    def __init__(
        self,
        smap,
        num_envs: int,
        *,
        device="cuda:0",
        render_mode: str | None = None,
        obs_layout: str = "chw",
        obs_copy: str = "safe_view",
        dynamics=None,
        renderer=None,
        episode_timeout: int = 32,
        sprites: int = 0,
        action_count: int = 17,
    ):
        if num_envs <= 0:
            raise ValueError("num_envs must be positive")
        if obs_layout not in ("chw", "hwc"):
            raise ValueError("obs_layout must be 'chw' or 'hwc'")
        if obs_copy not in ("copy", "safe_view", "unsafe_view"):  # env.py:344-345
            raise ValueError("obs_copy must be copy, safe_view, or unsafe_view")
        if render_mode not in (None, "rgb_array"):
            raise ValueError("render_mode must be None or 'rgb_array'")
        self.num_envs = int(num_envs)
        self.device = torch.device(device)
        self._resident_device = self.device
        self.render_mode = render_mode
        self.obs_layout = obs_layout
        self.obs_copy = obs_copy
        self.observation_ownership = {"copy": "owned", "safe_view": "safe_view", "unsafe_view": "unsafe_view"}[obs_copy]  # env.py:377-382
        self.observation_buffer_depth = {"copy": None, "safe_view": 2, "unsafe_view": 1}[obs_copy]
        self.observation_renderer = "reference"
        self.closed = False
        self.action_count = int(action_count)   # len(action_table); 17 in the reference's pinned table (actions.py:33-51)
        if self.action_count <= 0:
            raise ValueError("action table must contain at least one action")
        self._renderer = renderer if renderer is not None else HipRenderer(smap, self.num_envs, self.device)
        self._dynamics = dynamics if dynamics is not None else PosePoolDynamics(
            smap, self.num_envs, self.device, sprites=sprites, episode_timeout=episode_timeout
        )
        n = self.num_envs
        # engine-owned buffers (engine.py:1927-1934)
        self.frames = torch.zeros((n, self.frame_stack, 84, 84), dtype=torch.uint8, device=self.device)
        self.signal_buffer = torch.zeros((n, SIGNAL_COUNT), dtype=torch.float32, device=self.device)
        self._info_history = torch.zeros((n, 0, self.frame_stack), dtype=torch.float32, device=self.device)
        self._initialized = torch.zeros(n, dtype=torch.bool, device=self.device)
        self.pending_reset = torch.ones(n, dtype=torch.bool, device=self.device)   # engine.py:1661
        self._latest_reset_seeds = torch.zeros(n, dtype=torch.int64, device=self.device)
        self._all_lanes = torch.ones(n, dtype=torch.uint8, device=self.device)
        # obs_copy="safe_view": two buffers handed out in turn, so that the observation of the step before stays
        # valid while this step's is written (env.py:459-472).  The renderer's observation kernel fills them.
        view_shape = (n, self.frame_stack, 84, 84) if obs_layout == "chw" else (n, 84, 84, self.frame_stack)
        self._view_shape = view_shape
        self._safe_obs_buffers = (
            tuple(torch.empty(view_shape, dtype=torch.uint8, device=self.device) for _ in range(2)) if obs_copy == "safe_view" else ()
        )
        self._safe_obs_index = 0
        self._seed_values = [None] * n
        self._deferred_actions = None   # the one-element tuple step_async leaves for step_wait
        self._reset_rngs = [np.random.default_rng() for _ in range(n)]

    # ------------------------------------------------------------------ helpers
    def _require_device_tensor(self, value, name, *, shape, dtypes):  # env.py:711-728
        if not isinstance(value, torch.Tensor):
            raise TypeError(f"{name} must be a Torch tensor")
        if value.device != self._resident_device:
            raise TypeError(f"{name} must be on device {self._resident_device}")
        if value.shape != shape:
            raise ValueError(f"{name} must have shape {shape}")
        if value.dtype not in dtypes:
            expected = ", ".join(str(dtype) for dtype in dtypes)
            raise TypeError(f"{name} must have dtype {expected}")
        return value

    def _device_observations(self, observations: torch.Tensor) -> torch.Tensor:  # env.py:690-691
        return observations.permute(0, 2, 3, 1) if self.obs_layout == "hwc" else observations

    def _update_signals(self) -> None:
        self.signal_buffer[:, 17].copy_(self._dynamics.episode_time)  # episode_time, engine.py:15469
        self.signal_buffer[:, 20].copy_(self.pending_reset)           # engine.py:15472

    # ------------------------------------------------------------------ device API
    def reset_device(self, mask: torch.Tensor, seeds: torch.Tensor):
        return self._reset(mask, seeds, None)

    def _reset(self, mask: torch.Tensor, seeds: torch.Tensor, view):
        if self.closed:
            raise RuntimeError("cannot reset a closed environment")
        device_mask = self._require_device_tensor(mask, "mask", shape=(self.num_envs,), dtypes=(torch.bool,))
        device_seeds = self._require_device_tensor(seeds, "seeds", shape=(self.num_envs,), dtypes=INDEX_DTYPES).to(torch.int64)
        self._dynamics.reset(device_mask, device_seeds)
        # engine.reset renders every lane and fills the stack of the masked ones with four copies
        # (engine.py:2443-2450); unmasked lanes keep their stack, which the fused epilogue does by
        # writing only under the mask.
        self._renderer.render(self._dynamics.lane_state(), frames=self.frames, reset_mask=device_mask, obs=None, stack_only_masked=True,
                              final_frames=view, final_layout=self.obs_layout)
        self._latest_reset_seeds.copy_(torch.where(device_mask, device_seeds, self._latest_reset_seeds))
        self._initialized |= device_mask
        self.pending_reset.masked_fill_(device_mask, False)   # engine.py:2409
        self._update_signals()
        return self._device_observations(self.frames), self.signal_buffer

    def step_device(self, actions: torch.Tensor) -> DeviceTransition:
        return self._step(actions, None)

    def _step(self, actions: torch.Tensor, final_frames, final_layout: str = "chw") -> DeviceTransition:
        if self.closed:
            raise RuntimeError("cannot step a closed environment")
        indices = self._require_device_tensor(actions, "actions", shape=(self.num_envs,), dtypes=INDEX_DTYPES).to(torch.int64)
        rewards, terminated, truncated = self._dynamics.step(indices)
        self.pending_reset.copy_(terminated | truncated)      # engine.py:9542
        self._renderer.render(self._dynamics.lane_state(), frames=self.frames, final_frames=final_frames, final_layout=final_layout)
        self._update_signals()
        return DeviceTransition(
            observations=self._device_observations(self.frames), rewards=rewards, terminated=terminated, truncated=truncated,
            signals=self.signal_buffer, info_histories=self._info_history,
        )

    def step_and_reset_device(self, actions: torch.Tensor, reset_seeds: torch.Tensor) -> DeviceAutoResetTransition:
        # the final-observation clone (env.py:915) is written by the observation kernel of the step
        final_frames = torch.empty_like(self.frames)
        transition = self._step(actions, final_frames)
        final_observations = self._device_observations(final_frames)
        final_signals = transition.signals.clone()
        final_info_histories = transition.info_histories.clone()
        done = transition.terminated | transition.truncated
        any_done = bool(torch.any(done))  # env.py:919: one host sync for the reference renderer
        self.check_renderer_status()      # the device is idle here anyway
        if not any_done:
            return DeviceAutoResetTransition(
                transition.observations, transition.rewards, transition.terminated, transition.truncated,
                transition.signals, transition.info_histories, final_observations, final_signals, final_info_histories,
            )
        observations, signals = self.reset_device(done, reset_seeds)
        return DeviceAutoResetTransition(
            observations, transition.rewards, transition.terminated, transition.truncated, signals, self._info_history,
            final_observations, final_signals, final_info_histories,
        )

    def device_signals(self) -> torch.Tensor:
        return self.signal_buffer

    def check_renderer_status(self) -> None:
        """Raise if the renderer had to drop a linedef from a column's candidate list.

        A column keeps 64 linedefs in its own slots and up to 256 in the spill pool, which holds one column in 32 of a large
        batch (every column of up to eight lanes).

        Such a frame may differ from the reference's, which has no such bound, so it must not pass for a good one.
        Synchronises the device: called where the environment already waits for it.
        """
        status = getattr(self._renderer, "status", None)
        flags = status() if status is not None else 0
        if flags & 1:
            raise RuntimeError(
                "the renderer truncated a screen column's candidate list (more than 256 linedefs overlap one column of one "
                "lane's view, or more columns than the spill pool holds see more than 64): frames of this environment are "
                "not trustworthy on this map"
            )
        if flags & 2:
            raise RuntimeError(
                "the renderer truncated a screen column's list of drawsegs (a column crossed more than 255 portals): frames of "
                "this environment are not trustworthy on this map"
            )

    # ------------------------------------------------------------------ host-facing API (env.py:750-834)
    def _view_target(self):
        """The tensor this call's observation copy goes to, or None for ``unsafe_view`` (env.py:678-688)."""
        if self.obs_copy == "copy":
            return torch.empty(self._view_shape, dtype=torch.uint8, device=self.device)
        if self.obs_copy == "safe_view":
            buffer = self._safe_obs_buffers[self._safe_obs_index]
            self._safe_obs_index = (self._safe_obs_index + 1) % len(self._safe_obs_buffers)
            return buffer
        return None

    def seed(self, seed=None):
        self._seed_values = _normalize_seed(seed, self.num_envs)
        return list(self._seed_values)

    def reset(self, *, seed=None, options=None):
        if self.closed:
            raise RuntimeError("cannot reset a closed environment")
        reset_options = dict(options or {})
        raw_mask = reset_options.pop("reset_mask", None)
        if raw_mask is None:
            mask = torch.ones(self.num_envs, device=self.device, dtype=torch.bool)
        else:
            mask = self._require_device_tensor(raw_mask, "options['reset_mask']", shape=(self.num_envs,), dtypes=(torch.bool,))
        if not bool(torch.any(mask)):
            raise ValueError("options['reset_mask'] must select at least one lane")
        if reset_options:
            raise ValueError(f"unsupported reset options: {sorted(reset_options)}")
        seed_values = _normalize_seed(seed, self.num_envs) if seed is not None else self._seed_values
        game_seeds = [0] * self.num_envs
        for lane in torch.nonzero(mask, as_tuple=False).flatten().to("cpu").tolist():
            if seed_values[lane] is not None:
                self._reset_rngs[lane] = np.random.default_rng(seed_values[lane])
            game_seeds[lane] = int(self._reset_rngs[lane].integers(0, np.iinfo(np.uint32).max + 1, dtype=np.uint32))
        self._seed_values = [None] * self.num_envs
        seeds = torch.tensor(game_seeds, device=self.device, dtype=torch.int64)
        view = self._view_target()
        observations, _ = self._reset(mask, seeds, view)
        return (observations if view is None else view), {}

    def step(self, actions: torch.Tensor):
        if self.closed:
            raise RuntimeError("cannot step a closed environment")
        if not bool(torch.all(self._initialized)):
            raise RuntimeError("all lanes must be reset before the first step")
        if bool(torch.any(self.pending_reset)):   # env.py:819-821
            lanes = torch.nonzero(self.pending_reset).flatten().to("cpu").tolist()
            raise RuntimeError(f"terminal lanes must be reset before step: {lanes}")
        # every argument is checked before the observation buffer is taken: a refused call must not advance the
        # safe_view rotation, or the next step would write into the buffer the caller still holds (env.py:459-472)
        indices = self._require_device_tensor(actions, "actions", shape=(self.num_envs,), dtypes=INDEX_DTYPES).to(torch.int64)
        if bool(torch.any((indices < 0) | (indices >= self.action_count))):   # env.py:828-829
            raise ValueError("actions fall outside the declared action space")
        view = self._view_target()
        transition = self._step(indices, view, self.obs_layout)
        observations = transition.observations if view is None else view
        return observations, transition.rewards, transition.terminated, transition.truncated, {}

    def step_async(self, actions: torch.Tensor) -> None:  # env.py:839-842
        """Hand in the actions of a step that ``step_wait`` will run; nothing is checked or rendered yet."""
        if self._deferred_actions is not None:
            raise RuntimeError("an asynchronous step is already pending")
        self._deferred_actions = (actions,)

    def step_wait(self):  # env.py:844-849
        if self._deferred_actions is None:
            raise RuntimeError("no asynchronous step is pending")
        (actions,), self._deferred_actions = self._deferred_actions, None
        return self.step(actions)

    # ------------------------------------------------------------------ RGB frames
    def _rgb_frames(self, lane: int | None = None) -> torch.Tensor:
        state = self._dynamics.lane_state()
        if lane is not None:   # one lane's frame: only that lane is rendered
            state = state.select(slice(lane, lane + 1))
        rgb = torch.empty((state.x.shape[0], 240, 320, 3), dtype=torch.uint8, device=self.device)
        self._renderer.render(state, rgb=rgb)
        return rgb

    def render_lane(self, lane: int):  # env.py:1037-1053
        if self.closed:
            raise RuntimeError("cannot render a closed environment")
        if isinstance(lane, (bool, np.bool_)):
            raise TypeError("lane must be an integer")
        lane_index = operator.index(lane)
        if not 0 <= lane_index < self.num_envs:
            raise IndexError(f"lane must be in [0, {self.num_envs - 1}]")
        if self.render_mode != "rgb_array":
            return None
        frame = self._rgb_frames(lane_index)[0].detach().to("cpu").numpy().copy()
        self.check_renderer_status()
        return frame

    def render(self):
        return self.render_lane(0)

    def get_images(self):  # env.py:1058-1064
        if self.closed:
            raise RuntimeError("cannot render a closed environment")
        if self.render_mode != "rgb_array":
            return [None for _ in range(self.num_envs)]
        frames = self._rgb_frames().detach().to("cpu").numpy()
        self.check_renderer_status()
        return [frame.copy() for frame in frames]

    def close(self) -> None:
        if not self.closed:
            self.closed = True
            try:
                self.check_renderer_status()
            finally:
                self._close_renderer()

    def _close_renderer(self) -> None:
        close = getattr(self._renderer, "close", None)
        if close is not None:
            close()
