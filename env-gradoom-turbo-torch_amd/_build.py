"""Compile the HIP sources into ``libgradoom_amd.so`` next to this file (gfx950 only)."""

from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(HERE, "csrc", "gd_render.hip")]
LIBRARY = os.path.join(HERE, "libgradoom_amd.so")

# -ffp-contract=off: the reference evaluates float32 expressions one rounded op at a time.
# The packed-fp32 feature is switched off for every device function.
FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def needs_build() -> bool:
    if not os.path.exists(LIBRARY):
        return True
    built = os.path.getmtime(LIBRARY)
    header = os.path.join(os.path.dirname(HERE), "include", "gradoom_amd.h")
    return any(os.path.getmtime(path) > built for path in SOURCES + [header])


def build_library(force: bool = False) -> str:
    if not force and not needs_build():
        return LIBRARY
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    command = [hipcc, *FLAGS, "-o", LIBRARY, *SOURCES]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + result.stdout + result.stderr)
    return LIBRARY


if __name__ == "__main__":
    print(build_library(force=True))
