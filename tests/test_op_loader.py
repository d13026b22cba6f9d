"""
The HIP op loader without a GPU: code generation, the compile cache, the exported C ABI of a compiled op and its host-side
error paths (hipcc cross-compiles for gfx950 here; nothing is launched).  Where the reference tree is present, its own op
sources are read as text and compiled against this package's dialect header.
"""

from __future__ import annotations

import concurrent.futures
import ctypes
import os

import pytest

import _reference_op_sources as ref_sources
import dialect_ops
from returnn_amd import op_loader

_root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class Tiny:
    in_info = ({"name": "x", "ndim": 1, "shape": (None,), "need_contiguous": True},)
    out_info = ({"name": "y", "ndim": 1, "shape": ((0, 0),)},)
    c_extra_support_code = {
        "b_second": "DEF_KERNEL void tiny_twice(long n, const float* x, float* y) { for (long k = threadIdx.x; k < n; k += blockDim.x) y[k] = first_helper(x[k]); }",
        "a_first": "DEV_FUNC float first_helper(float v) { return 2.f * v; }",
    }
    c_fw_code = """
        assert(n_inputs == 1);
        assert(n_outputs == 1);
        if (Ndarray_DIMS(inputs[0])[0] %% 2 == 1) { %(fail)s }
        start_dev_kernel2(tiny_twice, 1, 64, 0, (Ndarray_DIMS(inputs[0])[0], Ndarray_DEV_DATA(inputs[0]), Ndarray_DEV_DATA(*outputs[0])));
        HANDLE_LAST_ERROR();
    """
    code_version = 3


def test_make_code_layout():
    code = op_loader.make_code("Tiny", Tiny.in_info, Tiny.out_info, Tiny.c_fw_code, Tiny.c_extra_support_code)
    assert '#include "rtn_op_dialect.h"' in code
    assert code.index("first_helper(float v)") < code.index("tiny_twice(long n")  # support code in key order
    assert code.index("tiny_twice(long n") < code.index("void Tiny_forward(")
    assert "n_inputs = 1, n_outputs = 1" in code
    assert "% 2 == 1" in code and "%%" not in code  # the forward code is %-formatted once, as in the reference
    assert "the op code gave up" in code  # %(fail)s
    for symbol in ("Tiny_fw(", "Tiny_last_error(", "Tiny_abi_version("):
        assert symbol in code
    with pytest.raises(ValueError):
        op_loader.make_code("not a name", (), (), "")


def test_want_inplace_dummy_out():
    in_info, out_info, n = op_loader.resolve_want_inplace_dummy(dialect_ops.BucketSum.in_info, dialect_ops.BucketSum.out_info)
    assert n == 1 and len(out_info) == 3
    assert in_info[0]["want_inplace"] == 0 and in_info[1]["want_inplace"] == 2
    assert out_info[2]["shape"] == ((1, 0),) and out_info[2]["ndim"] == 1
    assert dialect_ops.BucketSum.in_info[1]["want_inplace"] == "dummy_out"  # the description itself is untouched


def test_grad_description():
    """Derivation of the gradient op from a description with c_bw_code (rules of returnn/native_op.py:112-127, 165-226)."""
    g = op_loader.grad_description(dialect_ops.ElmanScan)
    assert g.__name__ == "GradOfElmanScan"
    assert [v["name"] for v in g.in_info] == ["W", "h0", "i", "start", "step", "Y", "D_Y", "D_hT"]  # X and hT dropped by the map
    assert g.grad_input_map_resolved == (1, 2, 3, 4, 5, 6, 8, 9)
    assert [v["name"] for v in g.out_info] == ["X", "W", "h0"]  # mask, start and step are disconnected
    assert g.out_info[0]["shape"] == ((5, 0), (5, 1), (5, 2))  # bw_out_var: from Y, input 5 of the gradient op
    assert g.out_info[1]["shape"] == ((0, 0), (0, 1)) and g.out_info[2]["shape"] == ((1, 0), (1, 1))
    assert g.c_fw_code is dialect_ops.ElmanScan.c_bw_code
    assert op_loader.grad_description(dialect_ops.RowLogSumExp) is None
    # default map: everything; an input whose gradient needs its shape must then be there
    assert op_loader.convert_grad_input_map(None, 4) == (0, 1, 2, 3)
    no_x = type("NoX", (), dict(vars(dialect_ops.ElmanScan), in_info=tuple({k: v for k, v in d.items() if k != "bw_out_var"} for d in dialect_ops.ElmanScan.in_info)))
    with pytest.raises(ValueError, match="grad_input_map drops that input"):
        op_loader.grad_description(no_x)


def test_compile_cache(tmp_path):
    opts = {"cache_dir": str(tmp_path)}
    op = op_loader.compile_op(Tiny, compiler_opts=opts)
    so = op.compiler.so_filename
    assert so.startswith(str(tmp_path / "Tiny")) and os.path.exists(so)
    for name in ("Tiny.hip", "compile.log", "info.json"):
        assert os.path.exists(os.path.join(os.path.dirname(so), name))
    assert "--offload-arch=gfx950" in open(os.path.join(os.path.dirname(so), "compile.log")).read()
    mtime = os.stat(so).st_mtime_ns
    again = op_loader.compile_op(Tiny, compiler_opts=opts)
    assert again.compiler.so_filename == so and os.stat(so).st_mtime_ns == mtime  # reused, not rebuilt
    changed = type("Tiny", (), dict(vars(Tiny), code_version=4))
    other = op_loader.CompiledOp(*op_loader.description_fields(changed), compiler_opts=opts)
    assert other.compiler.so_filename != so and other.compiler.need_recompile()  # another version, another directory


def test_compile_error_is_reported(tmp_path):
    broken = type("Broken", (), dict(vars(Tiny), c_fw_code="this is not C++;"))
    with pytest.raises(RuntimeError) as exc:
        op_loader.compile_op(broken, compiler_opts={"cache_dir": str(tmp_path)})
    assert "hipcc failed" in str(exc.value) and "Broken.hip" in str(exc.value)
    assert not [f for f in os.listdir(tmp_path / "Broken" / os.listdir(tmp_path / "Broken")[0]) if f.endswith(".so")]


@pytest.fixture(scope="module")
def built_ops():
    """The test ops in the in-tree cache: what the GPU tests load.  Compiled here if this tree has not built them yet."""
    ops = {cls.__name__: op_loader.compile_op(cls) for cls in dialect_ops.ALL_OPS}
    ops["GradOfElmanScan"] = op_loader.compile_op(op_loader.grad_description(dialect_ops.ElmanScan))
    return ops


def test_compiled_ops_export_the_c_abi(built_ops):
    header = open(os.path.join(_root, "include", "rtn_native_op.h")).read()
    assert "#define RTN_NATIVE_OP_ABI_VERSION %i" % op_loader.ABI_VERSION in header
    for name, op in built_ops.items():
        assert op.compiler.so_filename.startswith(op_loader.default_cache_dir())
        lib = ctypes.CDLL(op.compiler.so_filename)
        for suffix in ("_fw", "_last_error", "_abi_version"):
            assert getattr(lib, name + suffix) is not None
        version = getattr(lib, name + "_abi_version")
        version.restype = ctypes.c_int32
        assert version() == op_loader.ABI_VERSION


def test_struct_layout_matches_header():
    """ctypes mirrors of the two C structs: sizes and offsets as a C compiler lays out include/rtn_native_op.h on x86-64."""
    assert ctypes.sizeof(op_loader.RtnNdarray) == 32
    assert op_loader.RtnNdarray.dims.offset == 8 and op_loader.RtnNdarray.ndim.offset == 16
    assert op_loader.RtnNdarray.elem_size.offset == 20 and op_loader.RtnNdarray.on_host.offset == 24
    assert ctypes.sizeof(op_loader.RtnOpHost) == 32
    assert op_loader.RtnOpHost.alloc.offset == 8 and op_loader.RtnOpHost.release.offset == 16 and op_loader.RtnOpHost.user.offset == 24


def test_entry_point_rejects_bad_calls_without_touching_the_gpu(built_ops):
    op = built_ops["RowLogSumExp"]
    lib = op.lib()
    fw = getattr(lib, "RowLogSumExp_fw")
    err = getattr(lib, "RowLogSumExp_last_error")
    assert fw(None, 1, None, 2, None) == 1 and b"host must not be null" in err()
    host = op_loader.RtnOpHost()
    arr = (op_loader.RtnNdarray * 2)()
    assert fw(ctypes.byref(host), 3, arr, 2, arr) == 1 and b"expected 1 inputs and 2 outputs, got 3 and 2" in err()
    # a failed check in the op code itself: ndim of x is 0, not 2 (the check runs before anything is launched)
    assert fw(ctypes.byref(host), 1, arr, 2, arr) == 1
    assert b"NativeOp assertion failed: Ndarray_NDIM(x) == 2, 0 == 2" in err()
    # the %(fail)s statement: a matrix without columns
    dims = (ctypes.c_int64 * 2)(4, 0)
    arr[0].dims, arr[0].ndim, arr[0].elem_size = dims, 2, 4
    out = (op_loader.RtnNdarray * 2)()
    out_dims = (ctypes.c_int64 * 1)(4)
    for k in range(2):
        out[k].dims, out[k].ndim, out[k].elem_size = out_dims, 1, 4
    assert fw(ctypes.byref(host), 1, arr, 2, out) == 1 and b"the op code gave up" in err()


def test_python_wrapper_checks_arguments(built_ops):
    import torch

    op = built_ops["ElmanScan"]
    with pytest.raises(TypeError):
        op(torch.zeros(2, 2, 2))
    with pytest.raises(RuntimeError, match="compiled for HIP"):
        op(torch.zeros(2, 2, 2), torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2), 0, 1)


@pytest.mark.skipif(not ref_sources.available(), reason="the reference tree is not present")
def test_reference_op_sources_compile_for_gfx950(tmp_path):
    """
    Every op description of the reference that has forward code goes through the loader: generated unit + dialect header
    + hipcc.  The sources are read as text where they lie and compiled into a temporary directory.  Not covered:
    TwoDLSTM, MultiEndFastBaumWelchOp and SegmentFastBaumWelchOp, whose code calls the CUDA runtime by name
    (cudaMemcpy ...) instead of the dialect's vocabulary.
    """
    classes, skipped = ref_sources.read_descriptions()
    assert not skipped, skipped
    assert len(classes) >= 20
    n_forward = len(classes)
    expected_failures = {"TwoDLSTM", "MultiEndFastBaumWelchOp", "SegmentFastBaumWelchOp"}
    # SegmentFastBaumWelchOp completes its code in its constructor (returnn/native_op.py:4914-4946); these are the lines a
    # default-constructed instance gets
    segment = classes["SegmentFastBaumWelchOp"]
    segment["c_extra_support_code"]["000_batch_format"] = "#define NEW_BATCH_IDX_FORMAT false\n"
    segment["c_fw_code"] = (
        "const bool segmentwise_normalization = false;\nconst bool dump_targets = false;\nconst unsigned dump_targets_interval = 0;\n"
        + segment["c_fw_code"]
    )

    # the gradient ops: derived from c_bw_code and grad_input_map by the loader's own rule
    grads = {}
    for name, fields in classes.items():
        if fields.get("c_bw_code"):
            g = op_loader.grad_description(ref_sources.as_description(name, fields))
            grads[g.__name__] = {k: getattr(g, k) for k in ("in_info", "out_info", "c_fw_code", "c_extra_support_code", "code_version")}
    assert {"GradOfNativeLstm2", "GradOfLstmGenericBase", "GradOfLstmLowMem"} <= set(grads)
    classes.update(grads)
    expected_failures |= {"GradOfTwoDLSTM"} & set(grads)

    def build(item):
        name, fields = item
        try:
            op = op_loader.compile_op(ref_sources.as_description(name, fields), compiler_opts={"cache_dir": str(tmp_path)})
            lib = ctypes.CDLL(op.compiler.so_filename)
            return name, getattr(lib, name + "_fw") is not None, ""
        except RuntimeError as exc:
            return name, False, str(exc)[-1500:]

    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(build, sorted(classes.items())))
    failed = {name: msg for name, ok, msg in results if not ok}
    assert set(failed) == expected_failures, "\n\n".join("%s:\n%s" % kv for kv in failed.items() if kv[0] not in expected_failures)
    for name in expected_failures:
        assert "cuda" in failed[name], failed[name]
