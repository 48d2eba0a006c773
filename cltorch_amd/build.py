"""Builds ``libthcl_hip.so`` (the C-ABI library) in-tree with hipcc for gfx950.

Run as ``python -m cltorch_amd.build``.  Nothing here needs a GPU: hipcc
cross-compiles.  The step that is not a plain compile is the embedding of
``csrc/apply_device.h`` as a string (``apply_device_src.inc``) so that the
run-time compiler builds user expressions from the very same kernel text.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libthcl_hip.so")

ARCH = "gfx950"
SOURCES = ["rt.cpp", "state.cpp", "tensor.cpp", "layout.cpp", "expr.cpp", "math.cpp", "host_copy.cpp", "catalogue.cpp", "user_kernel.cpp", "blas.cpp", "unavailable.cpp",
           "apply.hip", "apply_catalogue.hip", "reduce.hip", "scan.hip", "index.hip", "blas12.hip", "gemm.hip"]

COMMON = ["-O3", "-fPIC", "-fvisibility=hidden", "-std=c++17", "-ffp-contract=off", "-Wall", "-Wno-unused-function", "-Wno-unused-const-variable",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC]
# packed fp32 instructions stay out of the generated code
DEVICE = [f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HOST_ONLY = ["-x", "c++", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the library cannot be built")
    return exe


def embed_skeleton() -> None:
    src = os.path.join(CSRC, "apply_device.h")
    dst = os.path.join(CSRC, "apply_device_src.inc")
    text = open(src).read()
    delim = "THCLSKEL"
    assert f"){delim}\"" not in text
    # split into chunks: some compilers cap the length of one string literal
    chunks, step = [], 8000
    for i in range(0, len(text), step):
        chunks.append(f'R"{delim}({text[i:i + step]}){delim}"')
    body = "// generated from apply_device.h by cltorch_amd/build.py -- do not edit\n" + "\n".join(chunks) + "\n"
    if not os.path.exists(dst) or open(dst).read() != body:
        with open(dst, "w") as f:
            f.write(body)


def _compile(name: str) -> str:
    out = os.path.join(OBJ, name + ".o")
    src = os.path.join(CSRC, name)
    cmd = [hipcc()]
    if name.endswith(".hip"):
        cmd += COMMON + DEVICE
    else:
        cmd += HOST_ONLY + COMMON
    cmd += ["-c", src, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"compiling {name} failed:\n{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    return warn


def build(verbose: bool = False, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    embed_skeleton()
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        for name, warn in zip(SOURCES, ex.map(_compile, SOURCES)):
            if verbose and warn:
                print(f"--- {name}\n{warn}", file=sys.stderr)
    objs = [os.path.join(OBJ, s + ".o") for s in SOURCES]
    # the dynamic symbol table is exactly what the two public headers declare
    from cltorch_amd import _lib
    names = sorted(_lib.declared_symbols())
    vmap = os.path.join(OBJ, "exports.map")
    with open(vmap, "w") as f:
        f.write("{\n  global:\n" + "".join(f"    {n};\n" for n in names) + "  local:\n    *;\n};\n")
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", f"-Wl,--version-script={vmap}", "-o", LIB] + objs + ["-lhiprtc", "-pthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"linking failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
