"""Host logic of the vector-env front end with a recording stand-in for the renderer (CPU only)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import load_fixture


class RecordingRenderer:
    """Writes a lane-dependent constant so ownership and masking can be observed without a GPU."""

    def __init__(self):
        self.calls = []

    status_value = 0

    def status(self):
        return self.status_value

    def render(self, lanes, *, indexed=None, obs=None, frames=None, reset_mask=None, rgb=None, stack_only_masked=False, final_frames=None,
               final_layout="chw"):
        self.calls.append(dict(reset=stack_only_masked, mask=None if reset_mask is None else reset_mask.clone(), final=final_frames, layout=final_layout))
        value = (lanes.x.abs().to(torch.int64) % 251).to(torch.uint8)
        if frames is not None:
            new = value[:, None, None].expand(-1, 84, 84)
            for lane in range(frames.shape[0]):
                if reset_mask is not None and bool(reset_mask[lane]):
                    frames[lane] = new[lane]
                elif not stack_only_masked:
                    frames[lane] = torch.roll(frames[lane], -1, 0)
                    frames[lane, -1] = new[lane]
            if final_frames is not None:
                final_frames.copy_(frames if final_layout == "chw" else frames.permute(0, 2, 3, 1))
        if rgb is not None:
            rgb.copy_(value[:, None, None, None].expand_as(rgb))

    def close(self):
        self.closed = True


@pytest.fixture
def env():
    from gradoom_amd.env import GraDoomVecEnv

    _meta, _data, smap, _tables = load_fixture("tiny_stages")
    return GraDoomVecEnv(smap, 4, device="cpu", render_mode="rgb_array", renderer=RecordingRenderer(), episode_timeout=3)


def test_argument_validation_matches_reference_error_classes(env):
    mask = torch.ones(4, dtype=torch.bool)
    seeds = torch.arange(4)
    with pytest.raises(TypeError, match="mask must be a Torch tensor"):
        env.reset_device([True] * 4, seeds)
    with pytest.raises(TypeError, match="mask must have dtype torch.bool"):
        env.reset_device(mask.to(torch.uint8), seeds)
    with pytest.raises(ValueError, match="seeds must have shape"):
        env.reset_device(mask, seeds[:3])
    with pytest.raises(TypeError, match="seeds must have dtype"):
        env.reset_device(mask, seeds.to(torch.float32))
    with pytest.raises(TypeError, match="actions must have dtype"):
        env.step_device(torch.zeros(4))


def test_observations_are_the_engine_owned_stack_and_finals_are_clones(env):
    obs, signals = env.reset_device(torch.ones(4, dtype=torch.bool), torch.arange(4))
    assert obs.data_ptr() == env.frames.data_ptr() and signals.data_ptr() == env.signal_buffer.data_ptr()
    assert obs.shape == (4, 4, 84, 84) and obs.dtype == torch.uint8
    # reset fills four identical frames (engine.py:2443-2450)
    assert torch.equal(obs[:, 0], obs[:, 3])
    transition = env.step_and_reset_device(torch.zeros(4, dtype=torch.int64), torch.arange(4))
    assert transition.observations.data_ptr() == env.frames.data_ptr()
    assert transition.final_observations.data_ptr() != env.frames.data_ptr()
    assert torch.equal(transition.final_observations, transition.observations)
    assert not bool(transition.truncated.any())
    # no lane done -> no reset render (tests/test_env.py:187-210)
    assert [call["reset"] for call in env._renderer.calls] == [True, False]


def test_done_lanes_are_reset_and_terminal_observation_is_retained(env):
    env.reset_device(torch.ones(4, dtype=torch.bool), torch.arange(4))
    actions = torch.zeros(4, dtype=torch.int64)
    env.step_and_reset_device(actions, torch.arange(4))
    env.step_and_reset_device(actions, torch.arange(4))
    env._dynamics.episode_time[2:] = 0  # only lanes 0 and 1 reach the timeout next step
    transition = env.step_and_reset_device(actions, torch.tensor([9, 8, 7, 6]))
    assert transition.truncated.tolist() == [True, True, False, False]
    last = env._renderer.calls[-1]
    assert last["reset"] and last["mask"].tolist() == [True, True, False, False]
    # reset lanes show four copies of their new frame, the others kept their rolled stack
    assert torch.equal(transition.observations[0, 0], transition.observations[0, 3])
    assert torch.equal(transition.observations[2], transition.final_observations[2])
    assert not torch.equal(transition.observations[0], transition.final_observations[0])
    assert env._latest_reset_seeds.tolist()[:2] == [9, 8]


def test_hwc_layout_is_a_permuted_view():
    from gradoom_amd.env import GraDoomVecEnv

    _meta, _data, smap, _tables = load_fixture("tiny_stages")
    env = GraDoomVecEnv(smap, 2, device="cpu", obs_layout="hwc", renderer=RecordingRenderer())
    obs, _ = env.reset_device(torch.ones(2, dtype=torch.bool), torch.zeros(2, dtype=torch.int64))
    assert obs.shape == (2, 84, 84, 4) and obs.data_ptr() == env.frames.data_ptr()


def test_render_contract(env):
    env.reset_device(torch.ones(4, dtype=torch.bool), torch.arange(4))
    image = env.render()
    assert isinstance(image, np.ndarray) and image.shape == (240, 320, 3) and image.dtype == np.uint8
    assert len(env.get_images()) == 4
    with pytest.raises(TypeError):
        env.render_lane(True)
    with pytest.raises(IndexError):
        env.render_lane(4)
    env.close()
    with pytest.raises(RuntimeError, match="closed"):
        env.render()
    with pytest.raises(RuntimeError, match="closed"):
        env.step_device(torch.zeros(4, dtype=torch.int64))


def test_render_mode_none_returns_none():
    from gradoom_amd.env import GraDoomVecEnv

    _meta, _data, smap, _tables = load_fixture("tiny_stages")
    env = GraDoomVecEnv(smap, 2, device="cpu", renderer=RecordingRenderer())
    assert env.render() is None and env.get_images() == [None, None]


def _host_env(obs_copy, obs_layout="chw"):
    from gradoom_amd.env import GraDoomVecEnv

    _meta, _data, smap, _tables = load_fixture("tiny_stages")
    renderer = RecordingRenderer()
    env = GraDoomVecEnv(smap, 4, device="cpu", renderer=renderer, episode_timeout=50, obs_copy=obs_copy, obs_layout=obs_layout)
    return env, renderer


def test_obs_copy_modes_follow_the_reference_ownership_rules():
    # env.py:678-688: "copy" hands out a fresh tensor, "safe_view" two buffers in turn, "unsafe_view" the stack itself
    from gradoom_amd.env import GraDoomVecEnv

    with pytest.raises(ValueError, match="obs_copy must be copy, safe_view, or unsafe_view"):
        GraDoomVecEnv(load_fixture("tiny_stages")[2], 4, device="cpu", renderer=RecordingRenderer(), obs_copy="view")
    actions = torch.zeros(4, dtype=torch.int64)

    env, renderer = _host_env("safe_view")
    assert (env.observation_ownership, env.observation_buffer_depth) == ("safe_view", 2)
    first, info = env.reset(seed=3)
    assert info == {} and first.data_ptr() != env.frames.data_ptr() and torch.equal(first, env.frames)
    held = first.clone()
    second = env.step(actions)[0]
    assert second.data_ptr() != first.data_ptr() and torch.equal(first, held), "the observation of the step before stays valid"
    third = env.step(actions)[0]
    assert third.data_ptr() == first.data_ptr() and torch.equal(third, env.frames)
    assert all(call["final"] is not None for call in renderer.calls), "the renderer writes the view itself: no copy pass"

    env, renderer = _host_env("copy")
    assert (env.observation_ownership, env.observation_buffer_depth) == ("owned", None)
    first = env.reset(seed=3)[0]
    second = env.step(actions)[0]
    third = env.step(actions)[0]
    assert len({first.data_ptr(), second.data_ptr(), third.data_ptr(), env.frames.data_ptr()}) == 4

    env, renderer = _host_env("unsafe_view")
    assert (env.observation_ownership, env.observation_buffer_depth) == ("unsafe_view", 1)
    first = env.reset(seed=3)[0]
    assert first.data_ptr() == env.frames.data_ptr() and renderer.calls[-1]["final"] is None
    assert env.step(actions)[0].data_ptr() == env.frames.data_ptr()


def test_host_api_layout_seeds_and_errors():
    env, renderer = _host_env("safe_view", "hwc")
    actions = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="all lanes must be reset before the first step"):
        env.step(actions)
    with pytest.raises(ValueError, match="must select at least one lane"):
        env.reset(options={"reset_mask": torch.zeros(4, dtype=torch.bool)})
    with pytest.raises(ValueError, match="unsupported reset options"):
        env.reset(options={"difficulty": 3})
    with pytest.raises(ValueError, match="seed sequence length must match num_envs"):
        env.reset(seed=[1, 2])
    observations, _ = env.reset(seed=11)
    assert observations.shape == (4, 84, 84, 4) and renderer.calls[-1]["layout"] == "hwc"
    assert torch.equal(observations, env.frames.permute(0, 2, 3, 1))
    phases = env._dynamics.phase.clone()
    env.reset(seed=11)
    assert torch.equal(env._dynamics.phase, phases), "the same seed resets to the same lane state (env.py:785-797)"
    assert env.seed(5) == [5, 6, 7, 8]
    env.reset()
    after_seed_call = env._dynamics.phase.clone()
    env.reset(seed=5)
    assert torch.equal(env._dynamics.phase, after_seed_call)
    observations = env.step(actions)[0]
    assert observations.shape == (4, 84, 84, 4) and torch.equal(observations, env.frames.permute(0, 2, 3, 1))
    env.close()
    with pytest.raises(RuntimeError, match="cannot step a closed environment"):
        env.step(actions)
    with pytest.raises(RuntimeError, match="cannot reset a closed environment"):
        env.reset()


def test_truncated_candidate_list_raises_instead_of_passing_a_bad_frame():
    env, renderer = _host_env("unsafe_view")
    mask = torch.ones(4, dtype=torch.bool)
    env.reset_device(mask, torch.arange(4))
    actions = torch.zeros(4, dtype=torch.int64)
    env.step_and_reset_device(actions, torch.arange(4))
    renderer.status_value = 1
    with pytest.raises(RuntimeError, match="truncated a screen column's candidate list"):
        env.step_and_reset_device(actions, torch.arange(4))
    with pytest.raises(RuntimeError, match="truncated"):
        env.close()
    assert env.closed and renderer.closed


def test_step_preconditions_follow_the_reference():
    # env.py:815-829: terminal lanes must be reset before the next host step; actions outside the table are refused
    from gradoom_amd.env import GraDoomVecEnv

    smap = load_fixture("tiny_stages")[2]
    renderer = RecordingRenderer()
    env = GraDoomVecEnv(smap, 4, device="cpu", renderer=renderer, episode_timeout=2, obs_copy="safe_view")
    assert env.action_count == 17 and bool(env.pending_reset.all())
    first = env.reset(seed=1)[0]
    assert not bool(env.pending_reset.any()) and not bool(env.signal_buffer[:, 20].any())
    actions = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(ValueError, match="actions fall outside the declared action space"):
        env.step(torch.full((4,), 17, dtype=torch.int64))
    with pytest.raises(ValueError, match="actions fall outside the declared action space"):
        env.step(torch.tensor([0, -1, 0, 0], dtype=torch.int8))
    with pytest.raises(TypeError, match="actions must have dtype"):
        env.step(torch.zeros(4))
    # a refused call takes no observation buffer: the next good step must not write into the one handed out last
    held = first.clone()
    second = env.step(actions)[0]
    assert second.data_ptr() != first.data_ptr() and torch.equal(first, held)
    truncated = env.step(actions)[3]
    assert bool(truncated.all()) and bool(env.pending_reset.all()) and bool(env.signal_buffer[:, 20].all())
    with pytest.raises(RuntimeError, match=r"terminal lanes must be reset before step: \[0, 1, 2, 3\]"):
        env.step(actions)
    mask = torch.tensor([True, False, True, False])
    env.reset(options={"reset_mask": mask})
    assert env.pending_reset.tolist() == [False, True, False, True]
    with pytest.raises(RuntimeError, match=r"terminal lanes must be reset before step: \[1, 3\]"):
        env.step(actions)
    with pytest.raises(ValueError, match="action table must contain at least one action"):
        GraDoomVecEnv(smap, 4, device="cpu", renderer=RecordingRenderer(), action_count=0)


def test_render_lane_renders_only_the_lane_asked_for():
    from gradoom_amd.env import GraDoomVecEnv

    smap = load_fixture("tiny_stages")[2]
    shapes = []

    class ShapeRenderer(RecordingRenderer):
        def render(self, lanes, **kwargs):
            shapes.append(tuple(lanes.x.shape))
            super().render(lanes, **kwargs)

    env = GraDoomVecEnv(smap, 4, device="cpu", render_mode="rgb_array", renderer=ShapeRenderer())
    env.reset_device(torch.ones(4, dtype=torch.bool), torch.arange(4))
    state = env._dynamics.lane_state()
    frame = env.render_lane(2)
    assert shapes[-1] == (1,) and frame.shape == (240, 320, 3)
    assert int(frame[0, 0, 0]) == int(state.x[2].abs().to(torch.int64) % 251)
    assert len(env.get_images()) == 4 and shapes[-1] == (4,)


def test_deferred_step_runs_when_waited_for(env):
    # tests/test_turbo_api_contract.py:345-347 and env.py:839-849: one step may be pending; waiting without one is an error
    env.reset(seed=5)
    with pytest.raises(RuntimeError, match="no asynchronous step is pending"):
        env.step_wait()
    calls = len(env._renderer.calls)
    env.step_async(torch.zeros(4, dtype=torch.int64))
    assert len(env._renderer.calls) == calls   # nothing rendered yet
    with pytest.raises(RuntimeError, match="already pending"):
        env.step_async(torch.zeros(4, dtype=torch.int64))
    transition = env.step_wait()
    assert len(env._renderer.calls) == calls + 1
    assert all(isinstance(value, torch.Tensor) for value in transition[:4]) and transition[0].shape == (4, 4, 84, 84)
    with pytest.raises(RuntimeError, match="no asynchronous step is pending"):
        env.step_wait()
    env.step_async(torch.zeros(4))   # a bad argument is refused when the step runs, and leaves nothing pending
    with pytest.raises(TypeError, match="actions must have dtype"):
        env.step_wait()
    env.step_async(torch.zeros(4, dtype=torch.int64))
    env.step_wait()
