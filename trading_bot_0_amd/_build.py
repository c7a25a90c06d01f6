"""Build recipe for libssd_hip.so (hipcc, gfx950 only).  The library is built in-tree, next to
this file, so a checkout carries it wherever the tree is copied."""
from __future__ import annotations

import shutil
import subprocess
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_DIR = PKG_DIR.parent
LIB_PATH = PKG_DIR / "libssd_hip.so"
SOURCES = [PKG_DIR / "csrc" / "ssd_kernels.hip", PKG_DIR / "csrc" / "ssd_api.cpp"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # hipcc forms packed-fp32 instructions from ordinary float code on its own; keep them off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; libssd_hip.so cannot be built")
    return exe


def build_library(verbose: bool = False) -> Path:
    cmd = [hipcc_path(), *HIPCC_FLAGS, f"-I{REPO_DIR / 'include'}", *map(str, SOURCES), "-o", str(LIB_PATH)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(" ".join(cmd))
        # the host pass does not know the device-only target feature and says so; drop that line
        print("\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if "packed-fp32-ops" not in l))
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}")
    return LIB_PATH
