"""Ahead-of-time build of libck_mi355.so (HIP, gfx950 only) into the Python package directory.

    python cute-kernels_amd/build.py [--jobs N] [--force]

Every translation unit under csrc/ is compiled with hipcc to an object file (in parallel) and linked into
cute_kernels/libck_mi355.so. Nothing is compiled at import time: the package only ever dlopens the result.
"""

from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
INCLUDE = os.path.join(os.path.dirname(ROOT), "include")
OBJ_DIR = os.path.join(ROOT, "build")
LIB_PATH = os.path.join(ROOT, "cute_kernels", "libck_mi355.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU forms are switched off for every kernel in this library
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-I", CSRC, "-I", INCLUDE, "-Wno-unused-command-line-argument"]


def _sources() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _newest_header_mtime() -> float:
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE) if f.endswith(".h")]
    return max(os.path.getmtime(h) for h in headers)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, src + ".o")
    src_path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj):
        if os.path.getmtime(obj) >= max(os.path.getmtime(src_path), _newest_header_mtime()):
            return obj
    cmd = [HIPCC, *COMMON_FLAGS]
    if src.endswith(".hip"):
        cmd += DEVICE_FLAGS
    cmd += ["-c", src_path, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    return obj


def build(jobs: int = 8, force: bool = False) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), _sources()))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    ap.add_argument("--force", action="store_true")
    args = ap.parse_args()
    print(build(args.jobs, args.force))
    sys.exit(0)
