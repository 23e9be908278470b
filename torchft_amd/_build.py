"""Builds ``libtftq.so`` (HIP kernels + C ABI) in-tree for gfx950 with hipcc."""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libtftq.so")
SOURCES = ["tftq_quantize.hip", "tftq_reduce.hip", "tftq_dequantize.hip", "tftq_runtime.hip", "tftq_plan.cpp"]
# Streaming kernels without arithmetic that bench.py times beside the product kernels
# (benchmark infrastructure; torchft_amd never loads this library).
CEILING_LIB_PATH = os.path.join(_HERE, "libtftq_ceiling.so")
CEILING_SOURCE = "tftq_ceiling.hip"
# The C++ walk over lists of tensors: a CPython extension module built with the host compiler
# against the Python and libtorch headers.  Host code only; not part of libtftq.so.
PYLIST_SOURCE = "tftq_pylist.cpp"

# -ffp-contract=off: the arithmetic contract is separate IEEE multiply, divide
# and add; fused multiply-adds are written out where they are wanted.
# packed-fp32-ops off: no v_pk_*_f32 instructions are generated.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def source_hash() -> str:
    """Hash of everything libtftq.so is compiled from; the library reports the hash it was
    built with as tftq_build_id()."""
    h = hashlib.sha256()
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC))
             if f.endswith((".hip", ".h", ".cpp")) and f not in (CEILING_SOURCE, PYLIST_SOURCE)]
    files.append(os.path.join(os.path.dirname(_HERE), "include", "tftq.h"))
    for path in files:
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; libtftq.so cannot be built")


# The C++ walk over lists of tensors (tftq_pylist.cpp): a CPython extension module built with
# the host compiler against the Python and libtorch headers.  Host code only.



def pylist_path() -> str:
    import sysconfig
    return os.path.join(_HERE, "_pylist" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def pylist_hash() -> str:
    with open(os.path.join(CSRC, PYLIST_SOURCE), "rb") as fh:
        return hashlib.sha256(fh.read()).hexdigest()[:16]


def pylist_command() -> list[str]:
    import sysconfig

    import torch
    from torch.utils import cpp_extension
    cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("no C++ compiler found; _pylist cannot be built")
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f'-DTFTQ_PYLIST_ID="{pylist_hash()}"']
    cmd += ["-I" + d for d in cpp_extension.include_paths()]
    cmd += ["-I" + sysconfig.get_paths()["include"], "-o", pylist_path(), os.path.join(CSRC, PYLIST_SOURCE),
            "-L" + libdir, "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10", "-Wl,-rpath," + libdir]
    return cmd


def build_pylist() -> str:
    _run(pylist_command())
    return pylist_path()


def load_pylist():
    """The _pylist module, built first if there is no build or if the build is of another
    source; None (with a warning) when it can be neither loaded nor built.  Callers then
    walk their lists in Python: same results, more host time on long lists."""
    import importlib
    import warnings
    for attempt in (0, 1):
        try:
            if attempt == 1 or not os.path.exists(pylist_path()):
                build_pylist()
            mod = importlib.import_module("torchft_amd._pylist")
            if getattr(mod, "BUILD_ID", None) == pylist_hash() or os.environ.get("TFTQ_ALLOW_STALE"):
                return mod
            if attempt == 1:  # a module that is already imported cannot be replaced in this process
                warnings.warn("torchft_amd._pylist was built from another source; rebuild it with "
                              "`python -m torchft_amd._build` (lists are walked in Python until then)")
                return None
        except Exception as exc:  # missing compiler or headers, an ABI that does not load
            if attempt == 1:
                warnings.warn(f"torchft_amd._pylist is not available ({exc}); lists are walked in Python")
                return None
    return None


def _run(cmd: list[str]) -> str:
    res = subprocess.run(cmd, cwd=CSRC, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l)  # host pass does not know the feature
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    return out


def build_library(verbose: bool = False) -> str:
    """Compile unconditionally and return the path of the shared library.  The
    sources are compiled side by side (one hipcc per file), then linked."""
    hipcc = hipcc_path()
    with tempfile.TemporaryDirectory(prefix="tftq_build_") as tmp:
        objs = [os.path.join(tmp, os.path.splitext(s)[0] + ".o") for s in SOURCES]
        build_id = f'-DTFTQ_BUILD_ID="{source_hash()}"'
        cmds = [[hipcc, *HIPCC_FLAGS, build_id, "-c", "-o", o, os.path.join(CSRC, s)] for s, o in zip(SOURCES, objs)]
        cmds.append([hipcc, *HIPCC_FLAGS, "-shared", "-o", CEILING_LIB_PATH, os.path.join(CSRC, CEILING_SOURCE)])
        cmds.append(pylist_command())
        with ThreadPoolExecutor(max_workers=len(cmds)) as pool:
            outs = list(pool.map(_run, cmds))
        outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]))
    out = "\n".join(o for o in outs if o.strip())
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
