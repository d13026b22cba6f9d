"""
Test infrastructure, never shipped with the library: builds nineteen of the reference's native ops for gfx950 through this
package's op loader -- sixteen of its OTHER ops, and its three LSTM ops with the gradient ops the loader derives for them --
so that the GPU tests can run them against the known answers the reference's own tests hold, against the committed
golden vectors and, where the reference holds no numbers, against the library routines and numpy forms its own tests use.

The op descriptions are read as text where they lie (``/root/reference/returnn/native_op.py``, parsed with :mod:`ast` by
``tests/_reference_op_sources.py``; nothing of the reference is imported or executed), the loader generates the unit and
hipcc compiles it in a temporary directory, and only the shared object is kept: ``tests/_built_ref_ops/<OpName>.so`` plus
``ops.json`` with each op's argument table (names, ranks, element types: what a caller needs to bind it).  No source of
the reference, generated or not, is written into this tree.  ``tests/_built_ref_ops/`` is not under version control.
These objects are neither a reference build nor an oracle: they are the thing under test.

What this checks is the loader (dialect header, generated entry point, Python wrapper), not the LSTM kernels: the ops run
against this package's support header, where the reference would use its own ``native_op.cpp``.

Run: ``python tests/build_ref_ops.py`` (no GPU needed).  Without the reference tree it does nothing.
"""

from __future__ import annotations

import json
import os
import shutil
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
OUT_DIR = os.path.join(HERE, "_built_ref_ops")

# ops whose expected results the reference's tests hold as numbers (tests/test_torch_native_op.py:95-160, :582-631,
# :689-812, :922-1034, :1036-1400)
OPS = ("FastBaumWelchOp", "FastViterbiOp", "EditDistanceOp", "OptimalCompletionEditDistanceOp",
       "OptimalCompletionEditDistancePerSuccessorOp", "NextEditDistanceRowOp", "NextEditDistanceReduceOp",
       "NativeLstm2", "LstmGenericBase", "LstmLowMem",
       # ops the reference's tests check against library routines and numpy instead (tests/test_TFNativeOp.py:1297-1560,
       # :1629-1760); tests/test_gpu_ref_more_ops.py does the same
       "Chunking", "UnChunking", "SubtensorBatchedIndex", "SparseToDense", "MaxAndArgmaxSparse",
       "CrossEntropySoftmaxAndGradientZSparse", "GetCtcFsaFastBwOp", "GetCtcFsaFastBwPackedOp", "FastBaumWelchPackedOp")
# of these also the gradient op that the loader derives from c_bw_code and grad_input_map ("GradOf<name>")
WITH_GRADIENT = ("NativeLstm2", "LstmGenericBase", "LstmLowMem")


def _plain(x):
    """in_info / out_info as JSON: tuples become lists."""
    if isinstance(x, (tuple, list)):
        return [_plain(v) for v in x]
    if isinstance(x, dict):
        return {k: _plain(v) for k, v in x.items()}
    return x


def build(ops=OPS, out_dir: str = OUT_DIR, verbose: bool = True) -> bool:
    """:return: whether anything was built (False: no reference tree here)"""
    for p in (ROOT, os.path.join(ROOT, "tests")):
        if p not in sys.path:
            sys.path.insert(0, p)
    import _reference_op_sources as ref_sources
    from returnn_amd import op_loader

    if not ref_sources.available():
        if verbose:
            print("build_ref_ops: no reference tree at %s, nothing to do" % ref_sources.REFERENCE_NATIVE_OP)
        return False
    classes, _ = ref_sources.read_descriptions()
    os.makedirs(out_dir, exist_ok=True)
    table = {}
    with tempfile.TemporaryDirectory(prefix="rtn_ref_ops_") as tmp:

        def one(name):
            """Compiles the op (and its gradient op): [(entry name, argument table)]."""
            fields = classes[name]
            op = op_loader.compile_op(ref_sources.as_description(name, fields), compiler_opts={"cache_dir": tmp})
            shutil.copyfile(op.compiler.so_filename, os.path.join(out_dir, name + ".so"))
            made = [(name, {"in_info": _plain(fields["in_info"]), "out_info": _plain(fields["out_info"])})]
            if name in WITH_GRADIENT:
                grad = op_loader.grad_description(ref_sources.as_description(name, fields))
                gname, g_in, g_out = op_loader.description_fields(grad)[:3]
                gop = op_loader.compile_op(grad, compiler_opts={"cache_dir": tmp})
                shutil.copyfile(gop.compiler.so_filename, os.path.join(out_dir, gname + ".so"))
                made.append((gname, {"in_info": _plain(g_in), "out_info": _plain(g_out)}))
            return made

        # (one hipcc per op, several at a time: as many as the machine has cores, or MAX_JOBS)
        try:
            limit = int(os.environ.get("MAX_JOBS", "0"))
        except ValueError:
            limit = 0
        with ThreadPoolExecutor(max_workers=max(1, min(len(ops), limit or (os.cpu_count() or 1)))) as pool:
            for made in pool.map(one, ops):
                for entry, info in made:
                    table[entry] = info
                    if verbose:
                        print("build_ref_ops: %s -> %s" % (entry, os.path.join(out_dir, entry + ".so")))
    with open(os.path.join(out_dir, "ops.json"), "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
    return True


if __name__ == "__main__":
    build()
