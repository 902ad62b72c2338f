"""Compiles libjitllm_hip.so for gfx950 with hipcc (jitllm_amd/csrc/Makefile)."""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib", "libjitllm_hip.so")


def build(force: bool = True, jobs: int = 8) -> str:
    """Runs the Makefile; ``force`` rebuilds every object.  Returns the library path."""
    cmd = ["make", "-C", CSRC, f"-j{jobs}"] + (["-B"] if force else [])
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libjitllm_hip.so failed:\n" + proc.stdout[-8000:])
    return LIB


if __name__ == "__main__":
    print(build())
