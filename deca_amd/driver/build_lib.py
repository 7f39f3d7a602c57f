"""Builds libdeca_hip.so (the C-ABI loader/launcher) in-tree with hipcc."""

from __future__ import annotations

import os
import subprocess

PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REPO_ROOT = os.path.dirname(PKG_ROOT)
LIB_PATH = os.path.join(PKG_ROOT, "libdeca_hip.so")
SOURCE = os.path.join(PKG_ROOT, "csrc", "deca_hip.cpp")
INCLUDE_DIR = os.path.join(REPO_ROOT, "include")


def build_library(force: bool = True) -> str:
    if not force and os.path.exists(LIB_PATH):
        return LIB_PATH
    from deca_amd.kernels.build import hipcc_path

    tmp = f"{LIB_PATH}.tmp{os.getpid()}"
    cmd = [
        hipcc_path(), "-O2", "-std=c++17", "-fPIC", "-shared", f"-I{INCLUDE_DIR}",
        SOURCE, "-o", tmp,
    ]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building libdeca_hip.so failed:\n{proc.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
