"""Builds ``libtftq.so`` (HIP kernels + C ABI) in-tree for gfx950 with hipcc."""

from __future__ import annotations

import os
import shutil
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libtftq.so")
SOURCES = ["tftq_kernels.hip", "tftq_plan.cpp"]

# -ffp-contract=off: the arithmetic contract is separate IEEE multiply, divide
# and add; fused multiply-adds are written out where they are wanted.
# packed-fp32-ops off: no v_pk_*_f32 instructions are generated.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; libtftq.so cannot be built")


def build_library(verbose: bool = False) -> str:
    """Compile unconditionally and return the path of the shared library."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", LIB_PATH,
           *[os.path.join(CSRC, s) for s in SOURCES]]
    res = subprocess.run(cmd, cwd=CSRC, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l)  # host pass does not know the feature
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
