"""Builds libmiles_quant.so (the C-ABI HIP library) and libmq_probes.so (self-tests and streaming probes that only
the GPU tests and bench.py load; not part of the product) for gfx950 with hipcc, in-tree.

    python -m miles_amd.build

-ffp-contract=off keeps every fp32 operation separately rounded (a fused multiply-add appears only
where the source writes one); packed-fp32 instruction selection is switched off.
"""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmiles_quant.so")
PROBES_LIB_PATH = os.path.join(LIB_DIR, "libmq_probes.so")

SOURCES = ["mq_core.hip", "mq_fp8_block.hip", "mq_mxfp8.hip", "mq_rescale.hip", "mq_mxfp4.hip", "mq_fake_quant.hip", "mq_int4.hip", "mq_nvfp4.hip", "mq_fp8_tensor.hip", "mq_sync.hip"]
PROBE_SOURCES = ["mq_selftest.hip", "mq_probe.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def _link(target: str, sources: list[str], verbose: bool) -> None:
    cmd = ["hipcc", *FLAGS, "-o", target, *(os.path.join(CSRC, s) for s in sources)]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in proc.stdout.splitlines() if "is not a recognized feature" not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{out}")
    if verbose and out.strip():
        print(out)


def build(verbose: bool = False) -> str:
    """Compiles both libraries; returns the path of the product library."""
    os.makedirs(LIB_DIR, exist_ok=True)
    _link(LIB_PATH, SOURCES, verbose)
    _link(PROBES_LIB_PATH, PROBE_SOURCES, verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
