"""Compiles the HIP library for gfx950 in-tree (hipcc cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(_PKG, "csrc", "fa_paged_attention.hip")
LIBRARY = os.path.join(_PKG, "libfa_paged_attention.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    # packed-fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
]


def build(verbose: bool = False, extra_flags=(), output: str = LIBRARY) -> str:
    """The product library, or with extra_flags and another output a debug build beside it
    (-DFA_TIMELINE: in-kernel timeline; -DFA_COST_PROBE=1|2: the segment kernels without their stores
    of partials), which FA_PAGED_ATTENTION_LIBRARY selects at run time."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, SOURCE, "-o", output]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    return output


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--output", default=LIBRARY)
    args, flags = ap.parse_known_args()  # everything else goes to hipcc (-DFA_TIMELINE ...)
    print(build(verbose=True, extra_flags=flags, output=os.path.abspath(args.output)))
