"""Float32 transcendentals the renderer takes as inputs, computed with Torch.

The reference evaluates a handful of ``cos/sin/atan/atan2/sqrt`` expressions
with Torch ops on the engine's device; their bit patterns are a property of the
Torch build, not of the algorithm.  The kernels therefore receive these values
as inputs, produced here by the very same Torch expressions on whichever device
the lane tensors live on:

* ``native_ray_offsets = -atan((x - 160) / 160)``      (``engine.py:2050-2054``)
* ``cosine_correction  = cos(native_ray_offsets)``      (``engine.py:10967``)
* ``ray_cos/ray_sin    = cos/sin(angle + offsets)``     (``engine.py:10966-10974``)
* ``sprite depth       = clamp_min(sqrt(dx²+dy²),1) * cos(wrap(atan2(dy,dx) - angle))``
  (``engine.py:14684-14688``)
* retained view angle ``bam.float() * (2π / 2³²)``      (``engine.py:10651``)
"""

from __future__ import annotations

import math

import torch

SCREEN_WIDTH = 320
BAM_TO_RADIANS = 2.0 * math.pi / float(1 << 32)


def native_ray_offsets(device) -> torch.Tensor:
    columns = torch.arange(SCREEN_WIDTH, device=device, dtype=torch.float32) - SCREEN_WIDTH / 2.0
    return -torch.atan(columns / (SCREEN_WIDTH / 2.0))


def cosine_correction(device) -> torch.Tensor:
    return torch.cos(native_ray_offsets(device))


def ray_tables(angle: torch.Tensor, offsets: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    ray_angles = angle[:, None] + offsets[None, :]
    return torch.cos(ray_angles).contiguous(), torch.sin(ray_angles).contiguous()


def angle_from_bam(angle_bam: torch.Tensor) -> torch.Tensor:
    return angle_bam.to(torch.float32) * BAM_TO_RADIANS


def sprite_depth(x, y, angle, sprite_x, sprite_y) -> torch.Tensor:
    dx = sprite_x - x[:, None]
    dy = sprite_y - y[:, None]
    distance = torch.sqrt(dx * dx + dy * dy).clamp_min(1)
    relative = torch.remainder(torch.atan2(dy, dx) - angle[:, None] + math.pi, 2 * math.pi) - math.pi
    return (distance * torch.cos(relative)).contiguous()
