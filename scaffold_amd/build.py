"""Builds ``libscaffold_hip.so`` in-tree with hipcc for gfx950 (``make -C scaffold_amd/csrc``)."""

from __future__ import annotations

import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(jobs: int = 8, force: bool = False) -> str:
    """Compile every HIP source and link the shared library; returns its path."""
    csrc = os.path.join(_HERE, "csrc")
    if force:
        subprocess.run(["make", "-C", csrc, "clean"], check=True, stdout=subprocess.DEVNULL)
    proc = subprocess.run(["make", "-C", csrc, f"-j{int(jobs)}"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libscaffold_hip.so failed:\n" + proc.stdout[-8000:])
    path = os.path.join(_HERE, "libscaffold_hip.so")
    if not os.path.exists(path):
        raise RuntimeError(f"make succeeded but {path} is missing")
    return path


if __name__ == "__main__":
    print(build())
