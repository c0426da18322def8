"""Headline benchmark: rendered lane-frames/s (320x240 indexed + 84x84x4 observation) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--workload config4] [--heights uniform|quantised]
                    [--lanes N] [--mode full|obs-only|rgb] [--assembly auto|fused|separate] [--no-cpu]

A step is one pass of the whole hot path over one batch of lanes whose inputs already sit in
HBM: sector-light flicker update, the Torch float32 ray / sprite-depth tables, the render
kernel chain and the fused observation + frame-stack update.  Camera poses and sprite lists
change every step.  After W warm-up steps, R repeats of K steps each are timed (device synchronised around every
repeat); the value is the median repeat and every sample is listed.  One JSON line is printed: metric, value,
timing, the roofline of the slowest kernel (algorithmic bytes over its launch duration, measured here with HIP
events) and a CPU baseline (the scalar C++ restatement of the reference algorithm on every host core).
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
POSE_SETS = 4
# HBM bytes one launch of a kernel moves: rocprofv3 FETCH_SIZE + WRITE_SIZE of a launch, each scaled by what the
# same counter reads for a 1 GiB copy in the same run.  Measured offline with the commands the summaries under
# profiles/ give and kept, per (workload, heights, mode, kernel), in profiles/hbm_traffic.json; a workload that was
# not measured reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic_per_lane(workload: str, heights: str, mode: str, kernel: str):
    try:
        with open(TRAFFIC_FILE) as handle:
            table = json.load(handle)["bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return None
    entry = table.get(f"{workload}/{heights}/{mode}/{kernel}")
    return None if entry is None else entry["bytes"] / entry["lanes"]


def algorithmic_bytes_per_lane_frame(sprites: int, map_bytes: int, lanes: int, mode: str) -> float:
    # 320x240 u8 frame write + 4x84x84 stack write + 3 older stack frames read
    # + lane pose (64 B) + 24 B per sprite + the shared map/atlas bytes once per launch.
    state = 64 + 24 * sprites + map_bytes / lanes
    if mode == "obs-only":      # no 320x240 frame handed out
        return 28224 + 21168 + state
    if mode == "rgb":           # palette-expanded RGB24 frame beside the indexed one
        return 230400 + 76800 + state
    return 76800 + 28224 + 21168 + state


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=100)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--repeats", type=int, default=5, help="timed repeats of --steps steps each; the median is reported")
    parser.add_argument("--workload", default="config4")
    parser.add_argument("--heights", choices=("uniform", "quantised"), default="uniform",
                        help="sector heights: uniform (floors 0..255, ceilings 64..256 above, whole units: a plane level per sector; the "
                             "benchmark's distribution) or quantised (floors 0..96 and ceilings 160..256 in steps of 8: 13 plane levels each way)")
    parser.add_argument("--lanes", type=int, default=None)
    parser.add_argument("--mode", choices=("full", "obs-only", "rgb"), default="full",
                        help="full: indexed frame + observation stack (the headline metric); obs-only: observation stack "
                             "only, no 320x240 frame handed to the caller; rgb: indexed + RGB24 frame, no observation")
    parser.add_argument("--assembly", choices=("auto", "fused", "separate"), default="auto",
                        help="how frames are put together after the walls: kernel by kernel through a frame in device memory "
                             "(separate, what auto picks) or band by band in LDS (fused: no frame reaches device memory unless asked for)")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    parser.add_argument("--cpu-lanes", type=int, default=0, help="lanes of the same workload the CPU baseline renders (0: 24 per thread)")
    parser.add_argument("--cpu-threads", type=int, default=0, help="host threads of the CPU baseline (0: every core this process may use, at most 16)")
    parser.add_argument("--copy-probe-mib", type=int, default=0,
                        help="after the timed region, copy this many MiB device to device once (a kernel of known "
                             "traffic that scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = parser.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: lanes are independent and this build has no multi-GPU path; run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    import __graft_entry__ as entry

    entry.load_package()
    from gradoom_amd import hostmath, mapbuild, synthmap
    from gradoom_amd.renderer import STAGES, HipRenderer, LaneState
    from gradoom_amd.selfcheck import make_lane_arrays

    if not torch.cuda.is_available():
        print("bench.py needs a ROCm device", file=sys.stderr)
        return 2
    device = torch.device("cuda:0")
    cfg = synthmap.CONFIGS[args.workload]
    lanes = args.lanes or cfg["lanes"]
    sprites = cfg["sprites"]
    smap = synthmap.generate_config_map(args.workload)
    if args.heights == "uniform":
        smap = synthmap.with_variant(smap, 5, heights="uniform")
    tables = mapbuild.build_map_tables(smap)
    cosine = hostmath.cosine_correction("cpu").numpy()
    renderer = HipRenderer(smap, lanes, device, cosine_correction=cosine, tables=tables)
    renderer.set_assembly(args.assembly)

    # Resident inputs: a few pose/sprite sets cycled step by step, plus flicker light vectors.
    states = []
    for k in range(POSE_SETS):
        poses = synthmap.generate_poses_batch(smap, lanes, 100 + k, flash=True)
        spr = synthmap.generate_sprites_batch(smap, lanes, sprites, 100 + k) if sprites else None
        bam = torch.as_tensor(poses.angle_bam, dtype=torch.int64)
        arrays = dict(
            x=poses.x, y=poses.y, angle=hostmath.angle_from_bam(bam).numpy(), view_z=poses.view_z,
            x_fixed=np.rint(poses.x.astype(np.float64) * 65536).astype(np.int64),
            y_fixed=np.rint(poses.y.astype(np.float64) * 65536).astype(np.int64),
            angle_bam=poses.angle_bam, pitch_bam=poses.pitch_bam, flash_light=poses.flash_light,
        )
        if spr is not None:
            arrays.update(sprite_x=spr.x, sprite_y=spr.y, sprite_z=spr.z, sprite_id=spr.sprite,
                          sprite_alive=spr.alive.astype(np.uint8), sprite_fullbright=spr.fullbright.astype(np.uint8))
        states.append(LaneState.from_numpy(arrays, device))
    rng = np.random.default_rng(7)
    base_lights = tables["sector_lights"]
    flicker = [
        torch.as_tensor(np.clip(base_lights + rng.integers(-16, 17, len(base_lights)), 0, 255).astype(np.float32)).to(device)
        for _ in range(POSE_SETS)
    ]
    indexed = obs = frames = rgb = None
    if args.mode != "obs-only":
        indexed = torch.zeros((lanes, 240, 320), dtype=torch.uint8, device=device)
    if args.mode != "rgb":
        obs = torch.zeros((lanes, 84, 84), dtype=torch.uint8, device=device)
        frames = torch.zeros((lanes, 4, 84, 84), dtype=torch.uint8, device=device)
    else:
        rgb = torch.zeros((lanes, 240, 320, 3), dtype=torch.uint8, device=device)

    def step(k: int) -> None:
        renderer.set_sector_lights(flicker[k % POSE_SETS])
        renderer.render(states[k % POSE_SETS], indexed=indexed, obs=obs, frames=frames, rgb=rgb)

    for k in range(args.warmup):
        step(k)
    torch.cuda.synchronize()
    repeat_seconds = []
    for repeat in range(max(1, args.repeats)):
        started = time.perf_counter()
        for k in range(args.steps):
            step(args.warmup + repeat * args.steps + k)
        torch.cuda.synchronize()
        repeat_seconds.append(time.perf_counter() - started)
    if renderer.status() != 0:
        print("renderer reported truncated column lists: result invalid", file=sys.stderr)
        return 1
    elapsed = float(np.median(repeat_seconds))
    value = lanes * args.steps / elapsed
    samples = [round(lanes * args.steps / seconds, 1) for seconds in repeat_seconds]

    # Per-kernel durations with HIP events on the launch stream, same inputs, same region.
    stage_launches = max(2, min(args.steps, 5))
    stage_ms = renderer.render_timed(states[0], stage_launches, indexed=indexed, obs=obs, frames=frames)
    torch.cuda.synchronize()
    dominant = max(stage_ms, key=stage_ms.get)
    chunk = renderer.chunk_lanes
    chunks = (lanes + chunk - 1) // chunk
    map_bytes = sum(int(np.asarray(v).nbytes) for v in tables.values() if isinstance(v, np.ndarray))
    bytes_per_lane = algorithmic_bytes_per_lane_frame(sprites, map_bytes, lanes, args.mode)
    # render_timed sums a stage over the chunks of one frame; one launch handles `chunk` lanes
    launch_ms = stage_ms[dominant] / chunks
    achieved = bytes_per_lane * chunk / (launch_ms * 1e-3) / 1e9 if launch_ms > 0 else 0.0
    per_lane_traffic = measured_traffic_per_lane(args.workload, args.heights, args.mode, dominant + "_kernel") if lanes >= chunk else None
    traffic = None if per_lane_traffic is None else round(per_lane_traffic * chunk)
    roofline = dict(
        bound="hbm", kernel=dominant + "_kernel", achieved=round(achieved, 3), peak=HBM_PEAK_GBPS, unit="GB/s",
        frac=round(achieved / HBM_PEAK_GBPS, 6), traffic=traffic, launch_ms=round(launch_ms, 4),
        stage_ms_per_frame={name: round(ms, 4) for name, ms in stage_ms.items()},
        whole_path_frac=round(value * bytes_per_lane / 1e9 / HBM_PEAK_GBPS, 6),
        bytes_per_lane_frame=round(bytes_per_lane, 1),
    )

    if args.copy_probe_mib > 0:
        probe_src = torch.ones(args.copy_probe_mib << 20, dtype=torch.uint8, device=device)
        probe_dst = torch.empty_like(probe_src)
        probe_dst.copy_(probe_src)
        torch.cuda.synchronize()

    cpu_baseline = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle  # CPU restatement of the reference algorithm: the reported baseline only

        threads = args.cpu_threads or min(len(os.sched_getaffinity(0)), 16)
        sample = max(1, min(args.cpu_lanes or 24 * threads, lanes))
        poses = synthmap.generate_poses_batch(smap, sample, 100, flash=True)
        spr = synthmap.generate_sprites_batch(smap, sample, sprites, 100) if sprites else None
        arrays = make_lane_arrays(smap, poses, spr)
        oracle.library()
        cpu_started = time.perf_counter()
        oracle.render_parallel(tables, arrays, cosine, threads)
        cpu_elapsed = time.perf_counter() - cpu_started
        cpu_baseline = dict(
            value=round(sample / cpu_elapsed, 3), unit="lane-frames/s", cores=threads, kind="port",
            sample=f"{sample} lanes of {args.workload} (one frame each: indexed frame, observation, stack), scalar C++ restatement of the "
                   f"reference algorithm on {threads} host threads, {cpu_elapsed:.1f} s",
        )

    line = dict(
        metric={"full": "rendered lane-frames/sec (320x240 + 84x84x4 obs)", "obs-only": "rendered lane-frames/sec (84x84x4 obs only)",
                "rgb": "rendered lane-frames/sec (320x240 indexed + RGB24)"}[args.mode], value=round(value, 1), unit="lane-frames/s", n_gpus=1,
        steps=args.steps, warmup=args.warmup, repeats=len(repeat_seconds), samples=samples,
        ms_per_step=round(elapsed / args.steps * 1e3, 3), higher_is_better=True,
        scaling="weak", vs_baseline=None, dtype="int64+f32", data="synthetic",
        config=dict(mode=args.mode, assembly=args.assembly, workload=f"{args.workload}: {lanes} lanes, {cfg['sectors']} sectors, {cfg['linedefs']} linedefs, "
                    f"{sprites} sprites/lane, masked midtex p={cfg['midtex']}, per-step sector-light flicker, "
                    + ("sector heights quantised (floors 0..96, ceilings 160..256, steps of 8)" if args.heights == "quantised"
                       else "sector heights uniform (floors 0..255, ceilings 64..256 above, whole units)")),
        roofline=roofline, cpu_baseline=cpu_baseline,
    )
    print(json.dumps(line))
    renderer.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
