"""Builds ``libjaxpp_amd.so`` (HIP kernels + C ABI) for gfx950 with hipcc.

The library is built in-tree (``jaxpp_amd/lib/``); nothing is installed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libjaxpp_amd.so")
SOURCES = ["abi.hip", "gemm.hip", "attention.hip", "attention_dq.hip", "attention_dkv.hip", "elementwise.hip",
           "moe.hip", "optimizer.hip", "f32_ops.hip", "stage.hip"]
# measurement aids: a library of their own beside the product library
DIAG_LIB = os.path.join(LIBDIR, "libjaxpp_amd_diag.so")
DIAG_SOURCES = ["diagnostics.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         # packed fp32 ops are kept out of generated code on this hardware pool
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# Per-file additions to FLAGS (none at present).
EXTRA_FLAGS = {}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{p.stdout}\n{p.stderr}")
    return p


def build(verbose: bool = True, jobs: int = 6) -> str:
    """Compile every source and link the shared library; returns its path."""
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = _hipcc()
    objs = []

    def compile_one(src):
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        extra = EXTRA_FLAGS.get(src)
        if extra:
            try:
                _run(cmd[:1] + extra + cmd[1:])
            except RuntimeError:
                if verbose:
                    print(f"[jaxpp_amd.build] {src}: {' '.join(extra)} not accepted, "
                          "building without", flush=True)
                _run(cmd)
        else:
            _run(cmd)
        if verbose:
            print(f"[jaxpp_amd.build] compiled {src}", flush=True)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        all_objs = list(ex.map(compile_one, SOURCES + DIAG_SOURCES))
    objs, diag_objs = all_objs[:len(SOURCES)], all_objs[len(SOURCES):]
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    if verbose:
        print(f"[jaxpp_amd.build] linked {LIB}", flush=True)
    # resolves jpp_set_error from the product library next to it
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", DIAG_LIB, *diag_objs,
          "-L" + LIBDIR, "-ljaxpp_amd", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print(f"[jaxpp_amd.build] linked {DIAG_LIB}", flush=True)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
