"""Ahead-of-time build of libck_mi355.so (HIP, gfx950 only) into the Python package directory.

    python cute-kernels_amd/build.py [--jobs N] [--force] [--define NAME=VALUE ...] [--output FILE.so]

Every translation unit under csrc/ is compiled with hipcc to an object file (in parallel) and linked into
cute_kernels/libck_mi355.so. Nothing is compiled at import time: the package only ever dlopens the result.

Measurement builds: `--define CK_ABLATE=2 --output /some/dir/libck_ablate2.so` compiles the same sources with the given
preprocessor definitions into an object directory of their own and links the library where --output says (outside
the package: only the product library lives in cute_kernels/, and it is untouched). `bench.py --lib FILE.so` loads
such a build; the switches are documented where they are used (CK_ABLATE, CK_STAMP in csrc/grouped_gemm_line.hip and
csrc/grouped_gemm_fp8.hip).
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


def _compile(src: str, force: bool, defines: tuple[str, ...] = (), obj_dir: str = OBJ_DIR) -> str:
    obj = os.path.join(obj_dir, src + ".o")
    src_path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj):
        if os.path.getmtime(obj) >= max(os.path.getmtime(src_path), _newest_header_mtime()):
            return obj
    cmd = [HIPCC, *COMMON_FLAGS, *(f"-D{d}" for d in defines)]
    if src.endswith(".hip"):
        cmd += DEVICE_FLAGS
    cmd += ["-c", src_path, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    return obj


def build(jobs: int = 8, force: bool = False, defines: tuple[str, ...] = (), output: str | None = None) -> str:
    if defines and not output:
        raise ValueError("a build with --define needs its own --output name: the product library takes no definitions")
    lib_path = LIB_PATH if not output else os.path.abspath(output)
    if output and os.path.dirname(lib_path) == os.path.dirname(LIB_PATH):
        raise ValueError("--output must lie outside the package directory: only the product library lives there")
    obj_dir = OBJ_DIR if not output else os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(output))[0])
    os.makedirs(os.path.dirname(lib_path), exist_ok=True)
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(lambda s: _compile(s, force, tuple(defines), obj_dir), _sources()))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib_path, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return lib_path


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--define", action="append", default=[], metavar="NAME=VALUE")
    ap.add_argument("--output", default=None, metavar="FILE.so")
    args = ap.parse_args()
    print(build(args.jobs, args.force, tuple(args.define), args.output))
    sys.exit(0)
