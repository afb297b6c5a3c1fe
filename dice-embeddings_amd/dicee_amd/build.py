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


def resources(out=None):
    """Compile the device code of every source once more with ``-Rpass-analysis=kernel-resource-usage`` and return
    (and optionally write to ``out``) a Markdown table of what each kernel takes: VGPRs, AGPRs, spilled VGPRs,
    scratch bytes per lane, LDS bytes per workgroup, SGPRs, waves per SIMD.  ``python -m dicee_amd.build --resources
    [file]``."""
    import re
    rows = []
    base = ["hipcc"] + [f for f in FLAGS if f not in ("-shared", "-fPIC")] + [
        "--cuda-device-only", "-c", "-Rpass-analysis=kernel-resource-usage", "-o", os.devnull]
    for src in SOURCES:
        proc = subprocess.run(base + [os.path.join(CSRC, src)], capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stderr[-2000:]}")
        for block in re.split(r"remark: [^\n]*Function Name: ", proc.stderr)[1:]:
            name = block.split()[0]

            def num(key):
                m = re.search(re.escape(key) + r": (\d+)", block)
                return int(m.group(1)) if m else -1
            rows.append((src, name, num("VGPRs"), num("AGPRs"), num("VGPRs Spill"), num("ScratchSize [bytes/lane]"),
                         num("LDS Size [bytes/block]"), num("SGPRs"), num("Occupancy [waves/SIMD]")))
    names = subprocess.run(["c++filt"], input="\n".join(r[1] for r in rows), capture_output=True, text=True).stdout.split("\n")
    lines = ["| Source | Kernel | VGPRs | AGPRs | VGPRs spilled | Scratch (B/lane) | LDS (B/workgroup) | SGPRs | Waves/SIMD |",
             "|---|---|---:|---:|---:|---:|---:|---:|---:|"]
    for r, nm in zip(rows, names):
        nm = nm.replace("kge::(anonymous namespace)::", "").replace("kge::", "")
        nm = re.sub(r"\((?:[^()]|\([^()]*\))*\)$", "", nm)              # drop the argument list
        nm = re.sub(r"^void ", "", nm)
        lines.append(f"| {r[0]} | `{nm}` | {r[2]} | {r[3]} | {r[4]} | {r[5]} | {r[6]} | {r[7]} | {r[8]} |")
    text = "\n".join(lines) + "\n"
    if out:
        with open(out, "w") as fh:
            fh.write(text)
    return text


if __name__ == "__main__":
    if "--resources" in sys.argv:
        i = sys.argv.index("--resources")
        print(resources(sys.argv[i + 1] if len(sys.argv) > i + 1 else None))
    else:
        print(build(verbose="-q" not in sys.argv))
