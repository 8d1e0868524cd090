"""Build libtaac_hip.so (the C-ABI library of hand-written gfx950 kernels) in-tree with hipcc.

Usage: ``python -m taac_2026_amd.build`` (or ``build_library()`` from Python). hipcc cross-compiles for gfx950
without a GPU being present. The shared library is written next to this file so that it travels with the source
tree; nothing is installed into site-packages.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / "csrc"
BUILD_DIR = PACKAGE_DIR / "csrc" / "build"
LIBRARY_PATH = PACKAGE_DIR / "libtaac_hip.so"

SOURCES = ("runtime.hip", "norm.hip", "attention.hip", "linear.hip", "ffn.hip", "fp8.hip", "fp8_ts.hip", "ffn_fp8.hip", "backbone.hip", "embedding.hip", "attention_bwd.hip", "readout.hip", "linear_bwd.hip", "ffn_bwd.hip")

# -packed-fp32-ops: keep the compiler from forming packed-fp32 VALU instructions from scalar float code.
HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-value",
)

# Per-source extras. -amdgpu-mfma-vgpr-form: keep MFMA accumulators in ordinary VGPRs where the kernel interleaves
# MFMAs with VALU work on the same values (softmax), instead of copying them to and from the accumulator registers.
EXTRA_FLAGS = {
    "attention.hip": ("-mllvm", "-amdgpu-mfma-vgpr-form=1"),
    "attention_bwd.hip": ("-mllvm", "-amdgpu-mfma-vgpr-form=1"),
}


def find_hipcc() -> str:
    candidate = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(candidate).exists():
        raise RuntimeError("hipcc not found: set HIPCC or add /opt/rocm/bin to PATH")
    return candidate


def _run(cmd: list[str]) -> None:
    result = subprocess.run(cmd, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"command failed ({result.returncode}): {' '.join(cmd)}\n{result.stdout}\n{result.stderr}")


def build_library(*, verbose: bool = False, jobs: int | None = None) -> Path:
    """Compile every kernel source for gfx950 and link libtaac_hip.so. Always recompiles."""
    hipcc = find_hipcc()
    BUILD_DIR.mkdir(parents=True, exist_ok=True)
    objects = []
    commands = []
    for source in SOURCES:
        obj = BUILD_DIR / (Path(source).stem + ".o")
        objects.append(str(obj))
        commands.append([hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(source, ()), "-c", str(CSRC_DIR / source), "-o", str(obj)])
    workers = jobs or min(len(commands), max(1, (os.cpu_count() or 2) // 2), 8)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for cmd, _ in zip(commands, pool.map(_run, commands)):
            if verbose:
                print("built", cmd[-1], file=sys.stderr)
    tmp = LIBRARY_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *objects])
    os.replace(tmp, LIBRARY_PATH)
    if verbose:
        print("linked", LIBRARY_PATH, file=sys.stderr)
    return LIBRARY_PATH


if __name__ == "__main__":
    build_library(verbose=True)
