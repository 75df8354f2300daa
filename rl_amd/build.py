"""Builds ``librl_amd_hip.so`` (the C-ABI HIP library) for gfx950 with hipcc.

``python -m rl_amd.build`` compiles every ``csrc/*.hip`` into ``rl_amd/lib/``.  hipcc
cross-compiles without a GPU.  Packed-FP32 instruction selection is switched off for all
device code.
"""

from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "librl_amd_hip.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",  # token arithmetic mirrors separate fp32 PyTorch ops: no fused multiply-add
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = True) -> str:
    """Compile every HIP source and link the shared library; returns its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in sources():
        obj = os.path.join(LIB_DIR, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        cmd = [hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, proc in procs:
        out, _ = proc.communicate()
        noise = "packed-fp32-ops"
        text = "\n".join(l for l in out.splitlines() if noise not in l and l.strip())
        if proc.returncode != 0:
            failed = True
            print(f"hipcc failed for {src}:\n{out}", file=sys.stderr)
        elif verbose and text:
            print(text)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    for obj in objs:
        os.remove(obj)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
