"""Builds libpith_hip.so (the C-ABI library of HIP kernels) for gfx950 with hipcc.

The library is placed in-tree at pithtrain_amd/lib/libpith_hip.so so that it travels with a
source snapshot; nothing is installed into site-packages and nothing is compiled at import time.
Run as `python -m pithtrain_amd.build` (from the pith-train_amd/ directory) or call build().
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(os.path.dirname(PKG_DIR), "csrc")
INCLUDE_DIR = os.path.join(os.path.dirname(os.path.dirname(PKG_DIR)), "include")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpith_hip.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

SOURCES = ["api.hip", "combine.hip", "norm_rope.hip", "mla_assemble.hip", "attn_fwd.hip", "attn_fwd_direct.hip", "attn_bwd_dq.hip", "attn_bwd_dq_d128.hip", "attn_bwd_dq_direct.hip", "attn_bwd_dq_ds.hip", "attn_bwd_dkdv.hip", "attn_bwd_dkdv_d128.hip", "attn_bwd_dkdv_d192.hip"]

# -packed-fp32-ops is switched off on purpose: some packed fp32 forms have produced wrong results
# on the target machines. Code object v5 is understood by both the ROCm 7.0 runtime bundled with
# PyTorch and the system ROCm 7.2 runtime.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-mcode-object-version=5",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libpith_hip.so can only be built with the ROCm toolchain")
    return exe


def _compile(src: str, extra: list) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-I", INCLUDE_DIR, "-I", SRC_DIR, "-c", os.path.join(SRC_DIR, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, extra_flags=()) -> str:
    """Compiles every HIP source and links libpith_hip.so. Returns the library path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    # libamdhip64 is referenced by soname only (no rpath): inside a PyTorch process the loader
    # then resolves it to the HIP runtime PyTorch has already loaded instead of a second copy.
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-mcode-object-version=5", *objs, "-o", LIB_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
