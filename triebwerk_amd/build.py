"""Build the gfx950 shared library (and, on request, the CPU oracle).

The library is compiled in-tree to ``triebwerk_amd/lib/libtriebwerk_kv.so`` with
plain ``hipcc``; nothing is JIT-compiled at import time.  hipcc cross-compiles
gfx950 code objects on a machine without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIBDIR = PKG / "lib"
LIB = LIBDIR / "libtriebwerk_kv.so"
ORACLE_DIR = ROOT / "oracle"
ORACLE_LIB = ORACLE_DIR / "libkv_oracle.so"

SOURCES = [
    "kv_append.hip",
    "kv_attention_valu.hip",
    "kv_attention_mfma.hip",
    "kv_attention_pair.hip",
    "kv_decode_fused.hip",
    "kv_prefill_mfma.hip",
    "kv_prefill_f16_mfma.hip",
    "kv_prefill_tq_mfma.hip",
    "kv_producer.hip",
    "kv_rotate.hip",
    "kv_capi.hip",
    "kv_engine.hip",
]

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    # packed fp32 VALU forms are kept out of every code object
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Files whose kernels run faster with another of LLVM's schedulers than with the default one (measured on
# MI355X): the two prompt kernels with the iterative ILP scheduler, 3-8 %.  The decode kernels keep the default:
# with the ILP schedulers the scans get spills inside their loops, and nothing else measured faster.
PER_FILE_FLAGS = {
    "kv_prefill_f16_mfma.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp"],
    "kv_prefill_tq_mfma.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp"],
}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        sys.stderr.write(proc.stderr)
        raise RuntimeError("command failed: " + " ".join(cmd))


def build_library(verbose: bool = False) -> Path:
    """Compile every HIP source for gfx950 and link the shared library."""
    LIBDIR.mkdir(exist_ok=True)
    objdir = LIBDIR / "obj"
    objdir.mkdir(exist_ok=True)
    hipcc = _hipcc()

    def compile_one(src: str) -> str:
        obj = objdir / (Path(src).stem + ".o")
        base = [hipcc, *HIPCC_FLAGS]
        tail = ["-c", str(CSRC / src), "-o", str(obj)]
        extra = PER_FILE_FLAGS.get(src, [])
        cmd = [*base, *extra, *tail]
        if verbose:
            print(" ".join(cmd), flush=True)
        try:
            _run(cmd)
        except RuntimeError:
            if not extra:
                raise
            # a compiler that does not know the scheduler option: the same code with its default scheduler
            print(f"{src}: retrying without {' '.join(extra)}", file=sys.stderr, flush=True)
            _run([*base, *tail])
        return str(obj)

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    _run(cmd)
    return LIB


def pybind_module_path() -> Path:
    import sysconfig
    return LIBDIR / ("jetson_engine" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_pybind(verbose: bool = False) -> Path:
    """Compile the pybind11 module `jetson_engine` (host code, g++) next to the library it links against."""
    import sysconfig

    import pybind11
    out = pybind_module_path()
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
           "-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"],
           str(CSRC / "jetson_engine_py.cpp"), "-o", str(out),
           "-L", str(LIBDIR), "-ltriebwerk_kv", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    _run(cmd)
    return out


def build_oracle(verbose: bool = False) -> Path:
    """Compile the CPU oracle (test infrastructure) with its own Makefile."""
    cmd = ["make", "-C", str(ORACLE_DIR), "-B"]
    if verbose:
        print(" ".join(cmd), flush=True)
    _run(cmd)
    return ORACLE_LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_pybind(verbose=True))
    print(build_oracle(verbose=True))
