"""Builds libaimet_amd.so (gfx950) from the HIP sources in this directory.

    python -m aimet_amd.csrc.build            # compile every translation unit and link
    python -m aimet_amd.csrc.build --changed  # recompile only sources newer than their objects

Flags that matter for parity:
  -ffp-contract=off -fno-fast-math   no fused multiply-add and no reassociation: the kernels reproduce the reference
                                     arithmetic operation by operation
  -packed-fp32-ops disabled          keeps hipcc from forming packed fp32 instructions
"""

from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(PKG, "libaimet_amd.so")

SOURCES = ["capi.hip", "qdq.hip", "qdq_bwd.hip", "reduce.hip", "hist.hip", "sqnr.hip", "dlq.hip", "encodings.hip", "diag.hip"]
HEADERS = ["ahq_device.h", "ahq_host.h", "layout.h", "tiling.h", "qdq_common.h", os.path.join("..", "..", "include", "aimet_amd.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-option-ignored",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def _stale(src: str, obj: str) -> bool:
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + [os.path.join(HERE, h) for h in HEADERS]
    return any(os.path.exists(d) and os.path.getmtime(d) > t for d in deps)


def _compile(src: str, obj: str) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {os.path.basename(src)}:\n{r.stdout}\n{r.stderr}")


def build(only_changed: bool = False, jobs: int | None = None, verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    work = []
    objs = []
    for s in sources:
        src = os.path.join(HERE, s)
        obj = os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o")
        objs.append(obj)
        if not only_changed or _stale(src, obj):
            work.append((src, obj))
    jobs = jobs or min(8, max(1, len(work)))
    if verbose:
        print(f"[aimet_amd] compiling {len(work)} of {len(sources)} HIP sources for gfx950", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for _ in ex.map(lambda so: _compile(*so), work):
            pass
    if work or not os.path.exists(LIB_PATH):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
        r = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"[aimet_amd] built {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--changed", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    args = ap.parse_args()
    try:
        build(only_changed=args.changed, jobs=args.j)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
