"""Builds the device probes that back the ceilings the design argues from (tests/probes/*.hip) into
tests/probes/bin/ with hipcc for gfx950. Called by __graft_entry__.build(); the GPU test tests/test_probes_gpu.py runs
the binaries. The probes are measurement programs, not part of the library, and link against the HIP runtime only."""

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
BIN_DIR = os.path.join(HERE, "bin")
PROBES = ("mfma_rate_probe", "atomic_rate_probe", "wide_wave_probe")
CSRC = os.path.join(os.path.dirname(os.path.dirname(HERE)), "pith-train_amd", "csrc")  # attn_tiles.h (wide_wave_probe)


def build(verbose: bool = True) -> None:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(BIN_DIR, exist_ok=True)
    for name in PROBES:
        out = os.path.join(BIN_DIR, name)
        cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-mcode-object-version=5",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I", CSRC,
               "-I", os.path.join(os.path.dirname(os.path.dirname(HERE)), "include"),
               os.path.join(HERE, name + ".hip"), "-o", out]  # fmt: skip
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}.hip:\n{proc.stderr}")
        if verbose:
            print(f"built {out}")


if __name__ == "__main__":
    build()
