"""
CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, and its
host logic (argument validation, plan, workspace size) behaves -- no kernel is launched here.
"""

from __future__ import annotations

import ctypes
import os
import re

import pytest

from returnn_amd import build, lib

_root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def cabi():
    if not os.path.exists(build.LIB_PATH):
        build.build_library()
    return lib.load()


def test_header_symbols_are_exported(cabi):
    header = open(os.path.join(_root, "include", "rtn_native_lstm2.h")).read()
    declared = set(re.findall(r"\b(rtn_[a-z0-9_]+)\s*\(", header))
    assert declared == set(lib.SYMBOLS)
    for name in declared:
        assert getattr(cabi, name) is not None


def test_abi_version(cabi):
    assert cabi.rtn_native_lstm2_abi_version() == lib.EXPECTED_ABI


def test_loader_refuses_another_abi_version(monkeypatch):
    """A stale build with other struct layouts must not be called."""
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "EXPECTED_ABI", lib.EXPECTED_ABI + 1)
    with pytest.raises(lib.NativeLibraryMismatch):
        lib.load()


def test_error_codes_match_header():
    header = open(os.path.join(_root, "include", "rtn_native_lstm2.h")).read()
    for name, value in re.findall(r"#define (RTN_[A-Z0-9_]+) (\d+)", header):
        py = {"RTN_DTYPE_F32": "DTYPE_F32", "RTN_DTYPE_BF16": "DTYPE_BF16"}.get(name, name.replace("RTN_MODE_", "MODE_"))
        assert getattr(lib, py) == int(value), name


def test_call_structs_match_the_header(tmp_path):
    """The ctypes mirrors of the header's call structs: same size and the same offset of every member, as a C compiler
    lays the header out."""
    import subprocess

    mirrors = {"rtn_lstm2_call": lib.Lstm2Call, "rtn_lstm2_bwd_call": lib.Lstm2BwdCall}
    lines = ['#include <stddef.h>', '#include <stdio.h>', '#include "rtn_native_lstm2.h"', "int main(void) {"]
    for cname, mirror in mirrors.items():
        lines.append('  printf("%s %%zu\\n", sizeof(%s));' % (cname, cname))
        for field, _ in mirror._fields_:
            lines.append('  printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (cname, field, cname, field))
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(_root, "include"), "-o", str(exe), str(src)], check=True)
    out = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    header = open(os.path.join(_root, "include", "rtn_native_lstm2.h")).read()
    for cname, mirror in mirrors.items():
        assert int(out[cname]) == ctypes.sizeof(mirror), cname
        for field, _ in mirror._fields_:
            assert int(out["%s.%s" % (cname, field)]) == getattr(mirror, field).offset, (cname, field)
        # every member of the C struct has a mirror: count the declarations between the braces
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), header, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        assert len([d for d in body.split(";") if d.strip()]) == len(mirror._fields_), cname


def _call(cabi, T, B, n, start=0, step=1, dtype=0, mode=0, ptr=4096, ws=None, ws_bytes=0):
    p = ctypes.c_void_p(ptr)
    return cabi.rtn_native_lstm2_fwd(p, p, p, p, p, start, step, p, p, p, p, T, B, n, dtype, mode, ws, ws_bytes, None)


def test_range_and_argument_errors(cabi):
    """The reference only prints on these under NDEBUG (returnn/native_op.cpp:60-69, native_op.py:1249-1252); here they are errors."""
    assert _call(cabi, 3, 2, 2, start=3) == lib.RTN_ERR_RANGE
    assert "start" in lib.last_error()
    assert _call(cabi, 3, 2, 2, start=-1) == lib.RTN_ERR_RANGE
    assert _call(cabi, 3, 2, 2, step=0) == lib.RTN_ERR_RANGE
    assert "step" in lib.last_error()
    assert _call(cabi, -1, 2, 2) == lib.RTN_ERR_SHAPE
    assert _call(cabi, 3, -2, 2) == lib.RTN_ERR_SHAPE
    assert _call(cabi, 3, 2, 2, dtype=7) == lib.RTN_ERR_ARG
    assert _call(cabi, 3, 2, 2, mode=9) == lib.RTN_ERR_ARG
    assert _call(cabi, 3, 2, 2, ptr=0) == lib.RTN_ERR_ARG  # null pointers
    assert _call(cabi, 3, 2, 2, ptr=4100) == lib.RTN_ERR_ARG  # misaligned
    assert "aligned" in lib.last_error()
    assert _call(cabi, 3, 2, 2) == lib.RTN_ERR_WORKSPACE  # no workspace
    assert "workspace" in lib.last_error()
    # persistent mode is refused, not silently replaced, for a shape the MFMA kernel cannot take
    assert _call(cabi, 3, 2, 3, mode=lib.MODE_PERSISTENT) == lib.RTN_ERR_UNSUPPORTED


def test_workspace_and_plan(cabi):
    # benchmark configuration cfg3 (returnn_amd/synthetic.py): bf16, T=1000, B=32, n=1024: persistent, all weights on chip
    text = lib.describe_plan(1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert "mode=persistent" in text and "kernel=mfma" in text
    ws = lib.workspace_bytes(1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert ws >= 4 * 1024 * 1024 * 2  # at least the packed W
    # odd n: generic per-step kernels
    text = lib.describe_plan(3, 2, 2, lib.DTYPE_F32, lib.MODE_AUTO)
    assert "kernel=generic" in text and "mode=graph" in text
    assert lib.workspace_bytes(3, 2, 2, lib.DTYPE_F32, lib.MODE_AUTO) >= 2 * 2 * 2 * 4
    assert lib.workspace_bytes(-1, 2, 2, lib.DTYPE_F32, lib.MODE_AUTO) == 0
    # the workspace of AUTO covers its per-step fallback
    for T, B, n, dt in [(10, 64, 512, 0), (10, 32, 1024, 1), (10, 1, 1024, 1), (10, 200, 1024, 1), (5, 7, 96, 0)]:
        assert lib.workspace_bytes(T, B, n, dt, lib.MODE_AUTO) >= lib.workspace_bytes(T, B, n, dt, lib.MODE_STEPWISE)


def test_plan_of_large_batches_padded_widths_and_wide_layers(cabi):
    # a batch too large for one persistent launch: several in turn, each on a share of the batch groups
    text = lib.describe_plan(100, 256, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert "mode=persistent" in text and "kernel=mfma_regw" in text and "launches=2 " in text, text
    assert "launches=1 " in lib.describe_plan(100, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    # a width that is not a multiple of 32 runs zero-padded; the workspace holds the padded copies
    text = lib.describe_plan(100, 32, 1000, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert "kernel=mfma_regw" in text and "padded_width=1024" in text, text
    exact = lib.workspace_bytes(100, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    padded = lib.workspace_bytes(100, 32, 1000, lib.DTYPE_BF16, lib.MODE_AUTO)
    copies = 100 * 32 * 1024 * (4 * 2 + 4 * 2 + 2 + 4)  # X, H, Y, C at the padded width
    assert padded >= exact + copies
    assert cabi.rtn_native_lstm2_bwd_workspace_bytes(100, 32, 1000, lib.DTYPE_BF16) > cabi.rtn_native_lstm2_bwd_workspace_bytes(100, 32, 1024, lib.DTYPE_BF16)
    assert "padded_width" not in lib.describe_plan(100, 32, 20, lib.DTYPE_F32, lib.MODE_AUTO)  # tiny layers stay as they are
    # W does not fit on chip: one launch per step, a few KB of LDS (W goes from memory straight to the matrix cores)
    text = lib.describe_plan(100, 16, 4096, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert "mode=graph" in text and "kernel=mfma_lds" in text and "lds=4096 " in text, text


def test_xcd_local_plans(cabi):
    """Which shapes put every batch group on one XCD (planned for MI355X's 8 XCDs of 32 CUs when no device is visible)."""
    pair = lib.describe_multi_plan(2, 1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)  # the benchmark pair
    assert "kernel=mfma_regw_xcd_half mt=8 nt=1 groups=4 wgs_per_group=32 wgs=256 rows_per_group=8 " in pair, pair
    one = lib.describe_plan(1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert "kernel=mfma_regw_xcd_half" in one and "groups=8 " in one and "rows_per_group=4 " in one, one
    # a single bf16 sequence goes to one XCD too (its hidden state then never leaves that XCD's L2)
    single = lib.describe_plan(4000, 1, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    assert "kernel=mfma_regw_xcd_half mt=8 nt=1 groups=1 wgs_per_group=32 " in single, single
    # float32 at n = 512 keeps W spread over more CUs (fewer MFMAs per wavefront and step)
    assert "kernel=mfma_regw " in lib.describe_plan(500, 64, 512, lib.DTYPE_F32, lib.MODE_AUTO)
    # the environment switch: read once, and again when the library is told to
    os.environ["RTN_LSTM2_LOCAL"] = "0"
    try:
        assert "kernel=mfma_regw_xcd_half" in lib.describe_multi_plan(2, 1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)  # old snapshot
        lib.reload_env()
        assert "kernel=mfma_regw " in lib.describe_multi_plan(2, 1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    finally:
        del os.environ["RTN_LSTM2_LOCAL"]
        lib.reload_env()
    assert "kernel=mfma_regw_xcd_half" in lib.describe_multi_plan(2, 1000, 32, 1024, lib.DTYPE_BF16, lib.MODE_AUTO)
    # a layer whose group does not fit the CUs of one XCD has no such plan
    assert "_xcd" not in lib.describe_plan(100, 32, 2048, lib.DTYPE_BF16, lib.MODE_AUTO)


def test_two_threads_plan_alike(cabi):
    """Planning is deterministic and safe from several host threads at once: the same shapes, planned concurrently and
    while a third thread keeps re-reading the environment, give the same plan texts as planned alone."""
    import threading

    shapes = [(T, B, n, dt) for T in (1, 37, 1000) for B in (1, 5, 32, 200) for n in (32, 96, 512, 1024, 2048)
              for dt in (lib.DTYPE_F32, lib.DTYPE_BF16)]
    alone = [lib.describe_plan(*sh, lib.MODE_AUTO) for sh in shapes]
    results, stop = {}, threading.Event()

    def plan(tag, order):
        results[tag] = {k: lib.describe_plan(*shapes[k], lib.MODE_AUTO) for k in order}

    def reload():
        while not stop.is_set():
            lib.reload_env()

    ts = [threading.Thread(target=plan, args=("a", range(len(shapes)))),
          threading.Thread(target=plan, args=("b", range(len(shapes) - 1, -1, -1))),
          threading.Thread(target=reload)]
    for t in ts:
        t.start()
    ts[0].join(); ts[1].join()  # noqa: E702
    stop.set()
    ts[2].join()
    for k, want in enumerate(alone):
        assert results["a"][k] == want and results["b"][k] == want, (shapes[k], want, results["a"][k], results["b"][k])


def test_plan_invariants_over_shapes(cabi):
    """Every persistent plan covers the batch, keeps its grid on the device (256 CUs, at most two workgroups each) and,
    where it is XCD-local, keeps a group within the 32 CUs of an XCD and sizes its grid in multiples of the 8 XCDs."""
    def fields(text):
        out = {}
        for w in text.split():
            if "=" in w:
                k, v = w.split("=", 1)
                out[k] = int(v) if v.lstrip("-").isdigit() else v
        return out

    seen_local_turns = False
    for dt in (lib.DTYPE_BF16, lib.DTYPE_F32):
        for n in (64, 192, 256, 320, 512, 768, 1024, 1536, 2048):
            for B in (1, 3, 8, 9, 16, 31, 64, 100, 128, 200, 256, 513, 1024):
                for count in (1, 2):
                    text = lib.describe_plan(50, B, n, dt, lib.MODE_AUTO) if count == 1 else lib.describe_multi_plan(2, 50, B, n, dt, lib.MODE_AUTO)
                    f = fields(text)
                    if f.get("mode") != "persistent" or not str(f.get("kernel", "")).startswith("mfma_regw"):
                        continue
                    what = (dt, n, B, count, text)
                    assert f["rows_per_group"] * f["groups"] * f["launches"] >= B, what
                    assert f["rows_per_group"] * f["groups"] * (f["launches"] - 1) < B, what  # no idle turn
                    assert 1 <= f["rows_per_group"] <= 64 and f["rows_per_group"] <= 16 * f["nt"], what
                    assert f["wgs_per_group"] * 4 * f["mt"] == n, what
                    assert f["wgs"] <= 512, what
                    if "_xcd" in f["kernel"]:
                        assert f["wgs_per_group"] <= 32 and f["wgs"] % 8 == 0 and f["wgs"] <= 256, what
                        per_xcd = 32 // f["wgs_per_group"]
                        problems = count if f["launches"] == 1 else 1  # a turn is a launch of one problem
                        assert f["groups"] * problems <= 8 * per_xcd, what
                        seen_local_turns = seen_local_turns or f["launches"] > 1
                    if f["kernel"].endswith("_half"):
                        assert f["rows_per_group"] <= 8 and f["nt"] == 1 and f["mt"] % 2 == 0, what
    assert seen_local_turns


def test_op_description_contract():
    """Names, order, ndim and host-memory flags of returnn/native_op.py:1054-1068."""
    from returnn_amd import native_op

    d = native_op.OpDescription.from_gen_base(native_op.NativeLstm2)
    assert d.name == "NativeLstm2"
    assert [v["name"] for v in d.in_info] == ["X", "W", "y0", "c0", "i", "start", "step"]
    assert [v["ndim"] for v in d.in_info] == [3, 2, 2, 2, 2, 0, 0]
    assert all(v.get("host_memory") and v["dtype"] == "int32" for v in d.in_info[5:])
    assert [v["name"] for v in d.out_info] == ["Y", "C", "H", "d"]
    T, B, n = 7, 3, 5
    shapes = d.infer_shape(None, [(T, B, 4 * n), (n, 4 * n), (B, n), (B, n), (T, B), (), ()])
    assert shapes == [(T, B, n), (T, B, n), (T, B, 4 * n), (B, n)]
    assert len(native_op.NativeLstm2.grad_input_map(*range(15))) == 12


def test_schema_string():
    from returnn_amd import native_op, torch_native_op

    maker = torch_native_op.OpMaker(native_op.OpDescription.from_gen_base(native_op.NativeLstm2))
    assert maker.schema() == (
        "NativeLstm2(Tensor X, Tensor W, Tensor y0, Tensor c0, Tensor i, int start, int step) -> (Tensor, Tensor, Tensor, Tensor)"
    )


def test_make_op_rejects_cpu_tensors(cabi):
    """No CPU implementation is shipped: the op must fail loudly instead of computing somewhere else."""
    import torch

    from returnn_amd import native_op, torch_native_op

    op = torch_native_op.make_op(native_op.NativeLstm2)
    assert op is torch_native_op.make_op(native_op.NativeLstm2)  # cached per name
    T, B, n = 3, 2, 2
    with pytest.raises(RuntimeError, match="HIP"):
        op(torch.zeros(T, B, 4 * n), torch.zeros(n, 4 * n), torch.zeros(B, n), torch.zeros(B, n), torch.ones(T, B), 0, 1)


def test_fake_impl_shapes(cabi):
    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode

    from returnn_amd import native_op, torch_native_op

    op = torch_native_op.make_op(native_op.NativeLstm2)
    T, B, n = 5, 3, 4
    with FakeTensorMode():
        outs = op(torch.zeros(T, B, 4 * n), torch.zeros(n, 4 * n), torch.zeros(B, n), torch.zeros(B, n), torch.ones(T, B), 0, 1)
    assert [tuple(o.shape) for o in outs] == [(T, B, n), (T, B, n), (T, B, 4 * n), (B, n)]
