"""
Ahead-of-time build of ``librtn_native_lstm2.so`` for gfx950 with hipcc.

Takes the place of the reference's run-time compile-and-cache step for native ops
(returnn/util/native_code_compiler.py:216-354, returnn/torch/util/native_op_code_compiler.py:94-131):
there is one fixed target (MI355X), so the library is built once, in-tree, and loaded with ctypes.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from typing import List, Optional

_dir = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_dir, "csrc")
LIB_NAME = "librtn_native_lstm2.so"
LIB_PATH = os.path.join(CSRC_DIR, LIB_NAME)
SOURCES = ["rtn_native_lstm2.hip"]
HEADERS = ["lstm2_kernels.h", "lstm2_bwd_kernels.h", "lstm2_params.h", os.path.join("..", "..", "include", "rtn_native_lstm2.h")]
OFFLOAD_ARCH = "gfx950"
ROCM_LIB_DIR = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")  # rocBLAS (weight-gradient GEMM of the backward op)


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def compile_command(output: Optional[str] = None) -> List[str]:
    """The exact hipcc line.  Packed fp32 VALU instructions are disabled on purpose.  Floating-point
    contraction is off so that every kernel variant and decomposition rounds the gate and cell arithmetic
    identically (results do not depend on the execution mode) and like the CPU reference code."""
    return [
        hipcc_path(),
        "--offload-arch=%s" % OFFLOAD_ARCH,
        "-O3",
        "-ffp-contract=off",
        "-std=c++17",
        "-fPIC",
        "-shared",
        "-Xclang",
        "-target-feature",
        "-Xclang",
        "-packed-fp32-ops",
        "-Wall",
        "-Wno-unused-command-line-argument",
        "-o",
        output or LIB_PATH,
    ] + [os.path.join(CSRC_DIR, s) for s in SOURCES] + ["-L%s" % ROCM_LIB_DIR, "-lrocblas", "-Wl,-rpath,%s" % ROCM_LIB_DIR]


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC_DIR, f) for f in SOURCES + HEADERS] + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def build_library(force: bool = True, verbose: bool = False) -> str:
    """
    Compile the HIP library in-tree.

    :param force: rebuild even if the library is newer than its sources
    :return: path of the built library
    """
    if not force and not needs_build():
        return LIB_PATH
    tmp = LIB_PATH + ".tmp.%i" % os.getpid()
    cmd = compile_command(tmp)
    if verbose:
        print("$", " ".join(cmd), file=sys.stderr)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise RuntimeError("hipcc failed (%i):\n$ %s\n%s" % (proc.returncode, " ".join(cmd), proc.stdout))
    if verbose and proc.stdout.strip():
        print(proc.stdout, file=sys.stderr)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True, verbose=True))
