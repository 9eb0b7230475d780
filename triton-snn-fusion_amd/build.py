"""Builds libsnnf.so (hand-written HIP kernels for gfx950 + their C ABI) with hipcc, in tree.

    python triton-snn-fusion_amd/build.py [--jobs N] [--keep-objects]

hipcc cross-compiles gfx950 code objects without a GPU, so this runs on any host that has ROCm installed. The shared
library is written to triton-snn-fusion_amd/lib/libsnnf.so, next to the Python modules that load it through ctypes.
"""
from __future__ import annotations

import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path
from typing import List

PKG_DIR = Path(__file__).resolve().parent
REPO_ROOT = PKG_DIR.parent
CSRC_DIR = PKG_DIR / "csrc"
INCLUDE_DIR = REPO_ROOT / "include"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = CSRC_DIR / "_obj"
LIB_PATH = LIB_DIR / "libsnnf.so"

OFFLOAD_ARCH = "gfx950"

# -packed-fp32-ops is switched off: the compiler must not form v_pk_{add,mul,fma}_f32 from scalar float code.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-attributes",
    f"-I{INCLUDE_DIR}",
    f"-I{CSRC_DIR}",
]


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return candidate
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def sources() -> List[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


# Compiler warnings that are known and accepted: (file the warning points into, text it contains). Anything else fails
# the build, so that a new warning (an unroll request the compiler refuses leaves a loop over a register array rolled,
# an unused variable marks dead code) is seen when it appears and not after the kernels have slowed down.
ALLOWED_WARNINGS = (
    # outer epilogue loop of the 4-wave fallback kernel: too large to unroll for its widest tiles; measured as is
    ("snnf_conv_kernel.h", "loop not unrolled"),
)
_NOISE = ("is not a recognized feature for this target", "warning generated", "warnings generated")


def _split_warnings(stderr: str):
    """(allowed, unexpected) warning lines of one compiler run; the host pass's note about the packed-fp32 feature and
    the summary lines are dropped."""
    allowed, unexpected = [], []
    for line in stderr.splitlines():
        if "warning:" not in line or any(n in line for n in _NOISE):
            continue
        if any(name in line and text in line for name, text in ALLOWED_WARNINGS):
            allowed.append(line)
        else:
            unexpected.append(line)
    return allowed, unexpected


def _compile_one(hipcc: str, src: Path):
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    allowed, unexpected = _split_warnings(proc.stderr)
    if unexpected:
        sys.stderr.write(f"[build] {src.name}:\n{proc.stderr}\n")
    return obj, len(allowed), unexpected


def build_library(jobs: int = 4, keep_objects: bool = False, verbose: bool = True, allow_new_warnings: bool = False) -> Path:
    """Compiles every csrc/*.hip for gfx950 and links lib/libsnnf.so. Always recompiles."""
    hipcc = _hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC_DIR}")
    if verbose:
        print(f"[build] hipcc={hipcc} arch={OFFLOAD_ARCH} sources={[s.name for s in srcs]}", flush=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        results = list(pool.map(lambda s: _compile_one(hipcc, s), srcs))
    objs = [r[0] for r in results]
    n_allowed = sum(r[1] for r in results)
    unexpected = [line for r in results for line in r[2]]
    if verbose:
        print(f"[build] compiler warnings: {n_allowed + len(unexpected)} ({n_allowed} known, {len(unexpected)} new)", flush=True)
    if unexpected and not allow_new_warnings:
        raise RuntimeError("new compiler warnings (fix them or list them in ALLOWED_WARNINGS):\n" + "\n".join(unexpected))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if not keep_objects:
        shutil.rmtree(OBJ_DIR, ignore_errors=True)
    if verbose:
        print(f"[build] wrote {LIB_PATH} ({LIB_PATH.stat().st_size} bytes)", flush=True)
    return LIB_PATH


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("--keep-objects", action="store_true")
    ap.add_argument("--allow-new-warnings", action="store_true", help="do not fail on compiler warnings outside ALLOWED_WARNINGS")
    args = ap.parse_args()
    build_library(jobs=args.jobs, keep_objects=args.keep_objects, allow_new_warnings=args.allow_new_warnings)


if __name__ == "__main__":
    main()
