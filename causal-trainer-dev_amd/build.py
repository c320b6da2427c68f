"""Build recipe for libct_hotpath.so (HIP, gfx950 only).

Run ``python causal-trainer-dev_amd/build.py`` (or call :func:`build`) on any
machine with hipcc; no GPU is needed to compile. The shared library is placed
next to this file and is what :mod:`_lib` loads through ctypes.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC = PACKAGE_DIR / "csrc"
LIBRARY = PACKAGE_DIR / "libct_hotpath.so"
SOURCES = ("ct_error.hip", "ct_attn.hip", "ct_cutce.hip", "ct_prep.hip", "ct_layer.hip", "ct_logits_ce.hip")

# -packed-fp32-ops is switched off on purpose: hipcc must not form packed FP32
# instructions from scalar float code on this target.
HIP_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
    "-Wno-inline-asm",
)


def hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; libct_hotpath.so needs the ROCm toolchain")
    return found


def _run(cmd: list[str]) -> None:
    result = subprocess.run(cmd, capture_output=True, text=True)
    if result.returncode != 0:
        sys.stderr.write(result.stdout + result.stderr)
        raise RuntimeError("command failed: " + " ".join(cmd))


def build(verbose: bool = False, extra_flags: tuple[str, ...] = ()) -> Path:
    """Compile every HIP source and link libct_hotpath.so. Always recompiles."""

    compiler = hipcc()
    build_dir = PACKAGE_DIR / "build"
    build_dir.mkdir(exist_ok=True)
    sources = [name for name in SOURCES if (CSRC / name).exists()]
    objects = [build_dir / (Path(name).stem + ".o") for name in sources]

    def compile_one(pair):
        name, obj = pair
        cmd = [compiler, *HIP_FLAGS, *extra_flags, "-c", str(CSRC / name), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)

    with ThreadPoolExecutor(max_workers=min(4, len(sources))) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    link = [compiler, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
            *map(str, objects), "-o", str(LIBRARY)]
    if verbose:
        print(" ".join(link), flush=True)
    _run(link)
    return LIBRARY


if __name__ == "__main__":
    print(build(verbose=True))
