"""Builds oracle/_ref-free test infrastructure: the C restatement of the integer stages -> oracle/libck_oracle.so.

    python oracle/build.py

The reference itself is Python and is read, not built: there is no oracle/_ref for this path.
"""

from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libck_oracle.so")


def build() -> str:
    cmd = ["gcc", "-O2", "-std=c11", "-shared", "-fPIC", "-Wall", "-Wextra", "-o", LIB_PATH, os.path.join(HERE, "ck_oracle.c"), "-lm"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"gcc failed:\n{proc.stdout}\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build())
