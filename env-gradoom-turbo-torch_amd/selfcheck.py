"""One small end-to-end invocation of the HIP path, checked against the CPU oracle."""

from __future__ import annotations

import os
import sys

import numpy as np
import torch

from . import hostmath, mapbuild, synthmap
from .renderer import HipRenderer, LaneState


def make_lane_arrays(smap, poses, sprites=None) -> dict:
    """NumPy lane inputs with the Torch-CPU float32 tables, as the golden fixtures carry them."""

    bam = torch.as_tensor(poses.angle_bam, dtype=torch.int64)
    angle = hostmath.angle_from_bam(bam)
    x = torch.as_tensor(poses.x)
    y = torch.as_tensor(poses.y)
    ray_cos, ray_sin = hostmath.ray_tables(angle, hostmath.native_ray_offsets("cpu"))
    arrays = dict(
        x=poses.x, y=poses.y, angle=angle.numpy(), view_z=poses.view_z,
        x_fixed=np.rint(poses.x.astype(np.float64) * 65536).astype(np.int64),
        y_fixed=np.rint(poses.y.astype(np.float64) * 65536).astype(np.int64),
        angle_bam=poses.angle_bam, pitch_bam=poses.pitch_bam, flash_light=poses.flash_light,
        ray_cos=ray_cos.numpy(), ray_sin=ray_sin.numpy(),
    )
    if sprites is not None and sprites.x.shape[1] > 0:
        arrays.update(
            sprite_x=sprites.x, sprite_y=sprites.y, sprite_z=sprites.z, sprite_id=sprites.sprite,
            sprite_alive=sprites.alive.astype(np.uint8), sprite_fullbright=sprites.fullbright.astype(np.uint8),
            sprite_depth=hostmath.sprite_depth(x, y, angle, torch.as_tensor(sprites.x), torch.as_tensor(sprites.y)).numpy(),
        )
    return arrays


def smoke() -> None:
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, os.path.join(root, "oracle"))
    import oracle  # test infrastructure: the checker, not the thing under test

    if not torch.cuda.is_available():
        raise RuntimeError("smoke() needs a ROCm device")
    lanes = 6
    smap = synthmap.generate_map(31, grid=(6, 5), sectors=26, linedefs=160, midtex=0.2)
    tables = mapbuild.build_map_tables(smap)
    poses = synthmap.generate_poses(smap, lanes, 5, pitch=True, flash=True)
    sprites = synthmap.generate_sprites(smap, lanes, 24, 5)
    arrays = make_lane_arrays(smap, poses, sprites)
    cosine = hostmath.cosine_correction("cpu").numpy()
    expected = oracle.render(tables, arrays, cosine, frames=np.zeros((lanes, 4, 84, 84), np.uint8), reset_mask=np.ones(lanes, np.uint8))
    renderer = HipRenderer(smap, lanes, "cuda:0", cosine_correction=cosine, tables=tables)
    state = LaneState.from_numpy(arrays, "cuda:0")
    indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device="cuda:0")
    obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device="cuda:0")
    frames = torch.zeros((lanes, 4, 84, 84), dtype=torch.uint8, device="cuda:0")
    mask = torch.ones(lanes, dtype=torch.uint8, device="cuda:0")
    renderer.render(state, indexed=indexed, obs=obs, frames=frames, reset_mask=mask)
    torch.cuda.synchronize()
    if renderer.status() != 0:
        raise RuntimeError("renderer reported a truncated column list")
    if not np.array_equal(indexed.cpu().numpy(), expected["indexed"]):
        raise RuntimeError("HIP indexed frame differs from the CPU oracle")
    if not np.array_equal(frames.cpu().numpy(), expected["frames"]):
        raise RuntimeError("HIP observation stack differs from the CPU oracle")
    renderer.close()
    print(f"smoke ok: {lanes} lanes, 320x240 indexed + 84x84x4 observation match the oracle bit for bit")
