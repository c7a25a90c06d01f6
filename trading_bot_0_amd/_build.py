"""Build recipe for libssd_hip.so (hipcc, gfx950 only).  The library is built in-tree, next to
this file, so a checkout carries it wherever the tree is copied."""
from __future__ import annotations

import shutil
import subprocess
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_DIR = PKG_DIR.parent
LIB_PATH = PKG_DIR / "libssd_hip.so"
CSRC = PKG_DIR / "csrc"
SOURCES = [CSRC / "ssd_stream_kernels.hip", CSRC / "ssd_chunk_state.hip", CSRC / "ssd_chunk_state_scan.hip",
           CSRC / "ssd_chunk_scan_f32.hip",
           CSRC / "ssd_chunk_scan_bf16.hip", CSRC / "ssd_chunk_scan_bf16_y32.hip",
           CSRC / "ssd_fused_scan_bf16.hip", CSRC / "ssd_fused_scan_bf16_y32.hip", CSRC / "ssd_fused_scan_f32.hip",
           CSRC / "ssd_fused_scan_segments.hip", CSRC / "ssd_fused_scan_wide.hip", CSRC / "ssd_fused_scan_transposed.hip", CSRC / "ssd_fused_scan_adjoint_rows.hip", CSRC / "ssd_block_proj.hip",
           CSRC / "ssd_block_kernels.hip", CSRC / "ssd_block_step.hip", CSRC / "ssd_block_backward.hip", CSRC / "ssd_backward_kernels.hip", CSRC / "ssd_api.cpp"]
OBJ_DIR = PKG_DIR / "build"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # hipcc forms packed-fp32 instructions from ordinary float code on its own; keep them off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; libssd_hip.so cannot be built")
    return exe


def _run(cmd, verbose):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only target feature and says so; drop that line
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if "packed-fp32-ops" not in l)
    if verbose or proc.returncode != 0:
        print(" ".join(map(str, cmd)))
        if log.strip():
            print(log)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}")


def build_library(verbose: bool = False) -> Path:
    """Compiles every translation unit (in parallel) and links libssd_hip.so."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = hipcc_path()
    OBJ_DIR.mkdir(exist_ok=True)
    objs = [OBJ_DIR / (src.stem + ".o") for src in SOURCES]
    cmds = [[hipcc, *HIPCC_FLAGS, f"-I{REPO_DIR / 'include'}", "-c", str(src), "-o", str(obj)]
            for src, obj in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=len(cmds)) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(LIB_PATH)], verbose)
    return LIB_PATH
