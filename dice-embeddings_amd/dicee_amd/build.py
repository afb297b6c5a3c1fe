"""Compile the HIP kernels into ``libkge_hip.so`` next to this file (gfx950 only)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
OUT = os.path.join(HERE, "libkge_hip.so")
SOURCES = ["kge_query.hip", "kge_kernels.hip", "kge_csr.hip", "kge_probe.hip"]
# -ffp-contract=off: a score is compared bit for bit across kernels, so `acc * scale` must be rounded
# before it is compared or subtracted; a fused multiply-add would skip that rounding.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-shared", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False):
    cmd = ["hipcc"] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
