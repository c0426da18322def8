"""Compare the CPU oracle with the reference's own Torch CPU render path on seeded random cases (build container only).

Usage:  python tests/golden/reference_sweep.py FIRST_SEED COUNT [doors|billboards|layers|actors] [--keep]

Each case is a recipe of ``tests/random_cases.py`` (8 lanes), rendered by the reference through ``make_golden.build_case``
and by the oracle from the same lane inputs.  Indexed frames must be equal and observations within one, the bar of
``tests/test_oracle_golden.py``.  A lane that holds two live billboards of exactly the same depth is left out: the
reference's order among those is ``torch.topk``'s and not defined.  ``--keep`` writes the fixture of a differing case to
``tests/golden/fixtures/sweep_<seed>.npz`` so that it can be studied and kept as a golden case.
"""

from __future__ import annotations

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for path in (ROOT, os.path.dirname(HERE), HERE, os.path.join(ROOT, "oracle")):
    sys.path.insert(0, path)

import conftest  # noqa: E402
import make_golden  # noqa: E402
import oracle  # noqa: E402
import random_cases  # noqa: E402
from gradoom_amd import mapbuild  # noqa: E402

LANES = 8


def main() -> int:
    first, count = int(sys.argv[1]), int(sys.argv[2])
    kind = sys.argv[3] if len(sys.argv) > 3 and not sys.argv[3].startswith("--") else "doors"
    keep = "--keep" in sys.argv
    torch.set_num_threads(1)
    differing = 0
    for seed in range(first, first + count):
        rng = np.random.default_rng(seed)
        layers = {}
        if kind in ("doors", "layers", "actors"):
            recipe = dict(seed=seed, mixed=True, variants=True, eye_any=True, inverted=bool(rng.random() < 0.3))
            if kind == "layers":   # weapon, status bar and bullet chips over the view, projectiles and puffs that blend
                layers = dict(overlays=seed % 50 + 1, decals=seed % 97 + 1, effects=24)
            if kind == "actors":   # every kind of actor from randomised gameplay tensors, packed by actor_inputs.pack_actors
                layers = dict(actors=seed % 1000 + 1)
        else:
            recipe = dict(kind="awkward_billboards", seed=seed, ties=False)
        try:
            data = make_golden.build_case(f"sweep_{seed}", dict(recipe=recipe, lanes=LANES, **layers), False)
        except ValueError as error:   # a map the pose generator refuses
            print("seed", seed, "skipped:", error, flush=True)
            continue
        tables = mapbuild.build_map_tables(random_cases.build_parts(recipe, LANES)[0])
        arrays = conftest.lane_inputs(data)
        if layers.get("overlays"):
            from gradoom_amd import synthmap

            oracle.set_overlays(synthmap.generate_overlays(layers["overlays"]))
        result = oracle.render(tables, arrays, data["cosine_correction"])
        oracle.set_overlays(None)
        tied = np.zeros(LANES, dtype=bool)
        for lane in range(LANES):
            depths = arrays["sprite_depth"][lane][arrays["sprite_alive"][lane] != 0]
            tied[lane] = len(np.unique(depths)) < len(depths)
        pixels = (result["indexed"] != data["indexed"]).reshape(LANES, -1).sum(1)
        obs = np.abs(result["obs"].astype(int) - data["obs"].astype(int)).reshape(LANES, -1).max(1)
        wrong = ((pixels > 0) | (obs > 1)) & ~tied
        if wrong.any():
            differing += 1
            print("DIFFERS seed", seed, kind, "pixels per lane", pixels.tolist(), "observation", obs.tolist(), flush=True)
            if keep:
                np.savez_compressed(os.path.join(make_golden.FIXTURES, f"sweep_{seed}.npz"), **data)
        elif (pixels > 0).any():
            print("seed", seed, "differs only in lanes with billboards of equal depth:", np.nonzero(pixels)[0].tolist(), flush=True)
    print("sweep done", first, count, kind, "differing", differing, flush=True)
    return 1 if differing else 0


if __name__ == "__main__":
    sys.exit(main())
