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
HOST_SOURCE = "rtn_native_lstm2.hip"
TABLES_SOURCE = "lstm2_kernel_tables.hip"  # compiled once per part: the instantiations of the persistent kernels
TABLE_PARTS = 8
SOURCES = [HOST_SOURCE, TABLES_SOURCE]
HEADERS = ["lstm2_kernels.h", "lstm2_bwd_kernels.h", "lstm2_params.h", "lstm2_kernel_tables.h",
           os.path.join("..", "..", "include", "rtn_native_lstm2.h")]  # fmt: skip
OBJ_DIR = os.path.join(CSRC_DIR, "_obj")
OFFLOAD_ARCH = "gfx950"
ROCM_LIB_DIR = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")  # rocBLAS (weight-gradient GEMM of the backward op)


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def _flags() -> List[str]:
    """Packed fp32 VALU instructions are disabled on purpose.  Floating-point contraction is off so that every kernel
    variant and decomposition rounds the gate and cell arithmetic identically (results do not depend on the execution
    mode) and like the CPU reference code."""
    return [
        "--offload-arch=%s" % OFFLOAD_ARCH,
        "-O3",
        "-ffp-contract=off",
        "-std=c++17",
        "-fPIC",
        "-Xclang",
        "-target-feature",
        "-Xclang",
        "-packed-fp32-ops",
        "-Wall",
        "-Wno-unused-command-line-argument",
    ]


def compile_commands(obj_dir: Optional[str] = None) -> List[List[str]]:
    """The exact hipcc lines that make the objects: the host code, and the kernel tables once per part."""
    obj_dir = obj_dir or OBJ_DIR
    cmds = [[hipcc_path()] + _flags() + ["-c", os.path.join(CSRC_DIR, HOST_SOURCE), "-o", os.path.join(obj_dir, "host.o")]]
    for part in range(1, TABLE_PARTS + 1):
        cmds.append(
            [hipcc_path()] + _flags()
            + ["-DRTN_TABLE_PART=%i" % part, "-Wno-unused-function", "-c", os.path.join(CSRC_DIR, TABLES_SOURCE), "-o", os.path.join(obj_dir, "tables_%i.o" % part)]
        )  # fmt: skip
    return cmds


def link_command(output: Optional[str] = None, obj_dir: Optional[str] = None) -> List[str]:
    obj_dir = obj_dir or OBJ_DIR
    objs = [os.path.join(obj_dir, "host.o")] + [os.path.join(obj_dir, "tables_%i.o" % part) for part in range(1, TABLE_PARTS + 1)]
    return [hipcc_path(), "--offload-arch=%s" % OFFLOAD_ARCH, "-shared", "-fPIC", "-o", output or LIB_PATH] + objs + [
        "-L%s" % ROCM_LIB_DIR, "-lrocblas", "-Wl,-rpath,%s" % ROCM_LIB_DIR,
    ]  # fmt: skip


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC_DIR, f) for f in SOURCES + HEADERS] + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def _jobs() -> int:
    try:
        limit = int(os.environ.get("MAX_JOBS", "0"))
    except ValueError:
        limit = 0
    return max(1, min(TABLE_PARTS + 1, limit or (os.cpu_count() or 1)))


def build_library(force: bool = True, verbose: bool = False) -> str:
    """
    Compile the HIP library in-tree: the objects side by side (as many at once as the machine has cores, or MAX_JOBS),
    then one link.

    :param force: rebuild even if the library is newer than its sources
    :return: path of the built library
    """
    if not force and not needs_build():
        return LIB_PATH
    from concurrent.futures import ThreadPoolExecutor

    obj_dir = OBJ_DIR + ".tmp.%i" % os.getpid()
    os.makedirs(obj_dir, exist_ok=True)
    tmp = LIB_PATH + ".tmp.%i" % os.getpid()

    def run(cmd):
        if verbose:
            print("$", " ".join(cmd), file=sys.stderr)
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        return cmd, proc.returncode, proc.stdout

    try:
        with ThreadPoolExecutor(max_workers=_jobs()) as pool:
            results = list(pool.map(run, compile_commands(obj_dir)))
        results.append(run(link_command(tmp, obj_dir)) if all(rc == 0 for _, rc, _ in results) else (["(link skipped)"], 0, ""))
        for cmd, rc, out in results:
            if rc != 0:
                raise RuntimeError("hipcc failed (%i):\n$ %s\n%s" % (rc, " ".join(cmd), out))
            if verbose and out.strip():
                print(out, file=sys.stderr)
        os.replace(tmp, LIB_PATH)
    finally:
        shutil.rmtree(obj_dir, ignore_errors=True)
        if os.path.exists(tmp):
            os.remove(tmp)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(force=True, verbose=True))
