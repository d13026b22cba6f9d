"""
The native op as a PyTorch operator on HIP tensors.

Drop-in for the reference's ``returnn.torch.util.native_op.make_op`` (returnn/torch/util/native_op.py:450-458)
for the op this package implements: ``make_op(NativeLstm2)`` returns ``torch.ops.NativeLstm2.NativeLstm2`` with
the schema the reference's generator would register (:242-277)::

    NativeLstm2(Tensor X, Tensor W, Tensor y0, Tensor c0, Tensor i, int start, int step)
        -> (Tensor, Tensor, Tensor, Tensor)

Where the reference generates and compiles a C++ translation unit per op, this module registers the schema
with ``torch.library`` from Python and the device implementation calls the prebuilt gfx950 library through
its C ABI with raw device pointers and the current stream.  PyTorch only supplies memory and streams.

Argument handling follows the generated wrapper (:144-193): dtype normalisation, ndim checks,
``.contiguous()`` for ``need_contiguous`` inputs, device guard on the first tensor, outputs allocated on
that device.  Differences, on purpose: bfloat16 inputs stay bfloat16 (X, W, y0, Y, H in bf16; c0, C, d,
mask in float32) instead of being up-cast; outputs are not zero-filled first because the library writes
every element; CPU tensors are rejected (no CPU implementation is shipped).
"""

from __future__ import annotations

import collections
import os
import sys
from threading import RLock
from typing import Any, Dict, Optional

import torch

from . import lib as _lib
from . import native_op
from .native_op import OpDescription

_DTYPE_MAP = {"float32": torch.float32, "int32": torch.int32}


def _schema_type_str(v: Dict[str, Any]) -> str:
    if v.get("host_memory", False):
        assert v["ndim"] == 0
        return {"float32": "float", "int32": "int"}[v.get("dtype", "float32")]
    return "Tensor"


class OpMaker:
    """
    Registers one op with ``torch.library`` and hands out the ``torch.ops`` callable.
    Cached per op name under a process-wide lock, like the reference's OpMaker (:33-36, :430-447).

    The execution mode belongs to the maker and is fixed in the op it makes: ``mode="auto"`` registers the op under the
    reference's name (``torch.ops.NativeLstm2.NativeLstm2``), any other mode under ``<name>_<mode>``
    (``torch.ops.NativeLstm2_stepwise.NativeLstm2_stepwise``), so that ops of different modes can be used side by side,
    from any thread, and the mode shows in the op's name.
    """

    global_lock = RLock()
    op_cache: Dict[str, Any] = {}  # cache_key -> op
    lib_cache: Dict[str, Any] = {}  # cache_key -> torch.library.Library (kept alive)
    log_stream = sys.stdout

    def __init__(
        self,
        description: OpDescription,
        *,
        compiler_opts: Optional[Dict[str, str]] = None,
        with_cuda: Optional[bool] = None,
        mode: Optional[str] = None,
    ):
        """
        :param description:
        :param compiler_opts: accepted for signature compatibility; the library is prebuilt, nothing is compiled here
        :param with_cuda: accepted for signature compatibility; the device path is always HIP
        :param mode: "auto" (default), "persistent", "graph" or "stepwise": execution mode of the library
        """
        del compiler_opts, with_cuda
        self.description = description
        self.name = description.name
        if mode is not None and mode not in _lib.MODES:
            raise ValueError("mode must be one of %r" % sorted(_lib.MODES))
        self.mode = mode or "auto"

    @property
    def op_name(self) -> str:
        return self.name if self.mode == "auto" else "%s_%s" % (self.name, self.mode)

    @property
    def cache_key(self) -> str:
        return self.op_name

    def schema(self) -> str:
        d = self.description
        args = ", ".join("%s %s" % (_schema_type_str(v), v["name"]) for v in d.in_info)
        rets = ", ".join(_schema_type_str(v) for v in d.out_info)
        return "%s(%s) -> (%s)" % (self.op_name, args, rets)

    def _impl_for(self):
        _lib.load()  # fail now, loudly, if the HIP library is not there
        impl = {
            "rtn_native_lstm2_fwd": _native_lstm2_device_impl,
            "rtn_lstm_generic_base_fwd": _lstm_generic_base_device_impl,
            "rtn_lstm_low_mem_fwd": _lstm_low_mem_device_impl,
        }.get(self.description.c_abi_fw)
        if impl is None:
            raise NotImplementedError("no gfx950 implementation for op %r" % self.name)
        mode_code = _lib.MODES[self.mode]

        def _device_impl(*args):
            return impl(*args, mode=mode_code)

        return _device_impl

    def make_op(self):
        with self.global_lock:
            if self.cache_key in self.op_cache:
                return self.op_cache[self.cache_key]
            impl = self._impl_for()
            tlib = torch.library.Library(self.op_name, "DEF")
            tlib.define(self.schema())
            tlib.impl(self.op_name, impl, "CUDA")  # the dispatch key PyTorch-ROCm uses for HIP tensors
            tlib.impl(self.op_name, _cpu_not_supported(self.op_name), "CPU")
            self._register_fake_impl()
            op = getattr(getattr(torch.ops, self.op_name), self.op_name)
            self.lib_cache[self.cache_key] = tlib
            self.op_cache[self.cache_key] = op
            return op

    def _register_fake_impl(self):
        """Shapes from ``out_info`` for fake-tensor tracing (role of :396-428 in the reference)."""
        description = self.description

        def _fake_impl(*args):
            tensors = [a for a in args if isinstance(a, torch.Tensor)]
            device = tensors[0].device
            shapes = description.infer_shape(None, [tuple(a.shape) if isinstance(a, torch.Tensor) else () for a in args])
            act = torch.bfloat16 if tensors[0].dtype == torch.bfloat16 else torch.float32
            dtypes = {"Y": act, "H": act}  # cell states (C, d) are always float32
            return tuple(
                torch.empty(shape, dtype=dtypes.get(o["name"], torch.float32), device=device)
                for o, shape in zip(description.out_info, shapes)
            )

        torch.library.register_fake("%s::%s" % (self.op_name, self.op_name), _fake_impl)


class CompiledOpMaker(OpMaker):
    """
    An op given as source in the native-op dialect (``c_fw_code`` ...): compiled with hipcc by
    :mod:`returnn_amd.op_loader` and registered like the prebuilt ones.  Stands in for the reference's code-generating
    OpMaker (returnn/torch/util/native_op.py:27-447) on ROCm.
    """

    def __init__(self, cls, *, compiler_opts: Optional[Dict[str, Any]] = None, with_cuda: Optional[bool] = None):
        """
        :param cls: description class or object with in_info, out_info, c_fw_code, c_extra_support_code, code_version
        :param compiler_opts: passed to :class:`returnn_amd.op_loader.HipOpCodeCompiler` (``cache_dir``, ``extra_flags``, ...)
        :param with_cuda: accepted for signature compatibility; the device path is always HIP
        """
        from . import op_loader

        del with_cuda
        self.compiled = op_loader.CompiledOp(*op_loader.description_fields(cls), compiler_opts=compiler_opts)
        description = OpDescription(
            in_info=self.compiled.in_info, out_info=self.compiled.out_info, c_abi_fw=self.compiled.name + "_fw", name=self.compiled.name
        )
        super().__init__(description)

    def _impl_for(self):
        compiled = self.compiled
        compiled.lib()  # compile (if needed) and load now; a compiler error surfaces here

        def _compiled_op_impl(*args):
            return compiled(*args)

        return _compiled_op_impl

    def _register_fake_impl(self):
        description = self.description
        dtype_map = {"float32": torch.float32, "int32": torch.int32}

        def _fake_impl(*args):
            device = next(a.device for a in args if isinstance(a, torch.Tensor))
            shapes = description.infer_shape(None, [tuple(a.shape) if isinstance(a, torch.Tensor) else () for a in args])
            return tuple(
                torch.empty(shape, dtype=dtype_map[o.get("dtype", "float32")], device=device) for o, shape in zip(description.out_info, shapes)
            )

        torch.library.register_fake("%s::%s" % (self.op_name, self.op_name), _fake_impl)


def make_op(cls, **kwargs):
    """
    :param type[returnn_amd.native_op.NativeOpGenBase] cls: e.g. :class:`returnn_amd.native_op.NativeLstm2`, or a
        description that carries source in the native-op dialect (``c_fw_code``) instead of naming a prebuilt entry point
    :param kwargs: passed to :class:`OpMaker` / :class:`CompiledOpMaker`
    :return: op, e.g. ``(X, W, y0, c0, i, start, step) -> (Y, C, H, d)``
    """
    if not getattr(cls, "c_abi_fw", None) and getattr(cls, "c_fw_code", None):
        return CompiledOpMaker(cls, **kwargs).make_op()
    maker = OpMaker(OpDescription.from_gen_base(cls), **kwargs)
    return maker.make_op()


def make_op_with_grad(cls, **kwargs):
    """
    A differentiable callable for a description in the native-op dialect that carries ``c_bw_code``: forward = the
    compiled op, backward = its compiled gradient op ``GradOf<name>``, wired through ``torch.autograd.Function``.
    The reference's torch OpMaker stops short of this (returnn/torch/util/native_op.py:444-445); the rule that derives
    the gradient op and maps its results back onto the inputs is the backend-neutral one of returnn/native_op.py:
    189-252.

    :param cls: description with in_info, out_info, c_fw_code, c_bw_code (and grad_input_map, c_extra_support_code)
    :param kwargs: passed to :class:`CompiledOpMaker` for both ops
    :return: function ``(*inputs) -> tuple of outputs`` (dummy outputs of ``want_inplace="dummy_out"`` included)
    """
    from . import op_loader

    grad_cls = op_loader.grad_description(cls)
    if grad_cls is None:
        raise ValueError("%s has no c_bw_code" % getattr(cls, "__name__", cls))
    fw_op = make_op(cls, **kwargs)
    bw_op = make_op(grad_cls, **kwargs)
    in_info = tuple(cls.in_info)
    n_in = len(in_info)
    n_out_declared = len(cls.out_info)
    gi_map = grad_cls.grad_input_map_resolved
    connected = [v.get("gradient", "") != "disconnected" for v in in_info]

    class _Function(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *inputs):
            outs = fw_op(*inputs)
            ctx.inputs = inputs
            ctx.outs = outs[:n_out_declared]
            for v, o in zip(cls.out_info, outs):
                if v.get("gradient", "") == "disconnected":
                    ctx.mark_non_differentiable(o)
            return tuple(outs)

        @staticmethod
        def backward(ctx, *grad_outs):
            grads = [g if g is not None else torch.zeros_like(o) for g, o in zip(grad_outs[:n_out_declared], ctx.outs)]
            pool = list(ctx.inputs) + list(ctx.outs) + grads
            results = list(bw_op(*[pool[k] for k in gi_map]))
            per_input = []
            for k in range(n_in):  # returnn/native_op.py:228-252
                per_input.append(results.pop(0) if connected[k] else None)
            return tuple(g if (g is None or isinstance(ctx.inputs[k], torch.Tensor)) else None for k, g in enumerate(per_input))

    def op(*inputs):
        return _Function.apply(*inputs)

    op.forward_op, op.gradient_op = fw_op, bw_op
    return op


class NativeOpAborted(RuntimeError):
    """A bounded wait inside a persistent kernel expired: the results of that call are invalid."""


class StatusWatch:
    """
    Looks after the status words of the library's workspaces without stalling the stream.

    The persistent kernels bound every wait for another workgroup (2 s of wall clock by default).  A wait that runs
    into its bound sets the first word of the call's workspace slice to 1 and the workgroups that see it put NaN into
    results every caller consumes (final cell state, last visited frame of Y; Dy0 and Dc0 of the gradient).  On top of
    that, every op call here queues a copy of its status words to pinned host memory behind its kernels and records an
    event; the next op call (or :meth:`poll`) looks at the copies whose event has completed and raises
    :class:`NativeOpAborted` for a word that is 1.  Nothing waits for the device.

    ``RTN_LSTM2_CHECK_STATUS=1`` in the environment (or ``status_watch.synchronous = True``) makes every op call wait
    for its own kernels and check at once: the error then names the call that failed, at the price of one stream
    synchronisation per call.  ``RTN_LSTM2_CHECK_STATUS=0`` switches the watch off.  Under stream capture nothing is
    queued (a captured copy would be replayed without anybody looking at it); captured calls rely on the NaN marks.
    """

    SLOTS = 64  # status words per pinned block; a block is reused once its event has completed

    def __init__(self):
        self.lock = RLock()
        self.pending = collections.deque()  # (event, host block, number of words, what)
        self.free_blocks = []
        self.synchronous: Optional[bool] = None  # None: from the environment, read at each call
        self.checked = 0  # completed calls looked at so far (for tests)

    def _setting(self) -> str:
        if self.synchronous is not None:
            return "1" if self.synchronous else "lazy"
        return os.environ.get("RTN_LSTM2_CHECK_STATUS", "lazy")

    def after_call(self, what: str, ws: torch.Tensor, count: int, device) -> None:
        """Queue the look at the status word of each of the ``count`` equal slices of ``ws`` (current device = ``device``)."""
        setting = self._setting()
        if setting == "0" or count > self.SLOTS or torch.cuda.is_current_stream_capturing():
            return
        each = ws.numel() // count
        words = ws.view(torch.int32)[: (count - 1) * (each // 4) + 1 : max(each // 4, 1)]
        with self.lock:
            block = self.free_blocks.pop() if self.free_blocks else torch.zeros((self.SLOTS,), dtype=torch.int32, pin_memory=True)
        block[:count].copy_(words, non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(device))
        with self.lock:
            self.pending.append((event, block, count, what))
        if setting == "1":
            event.synchronize()
            self.poll()

    def poll(self) -> None:
        """Raise for the oldest completed call whose status word says that a wait expired; never blocks."""
        if torch.cuda.is_current_stream_capturing():
            return  # (no queries while a capture is under way)
        failed = None
        with self.lock:
            while self.pending and self.pending[0][0].query():
                _, block, count, what = self.pending.popleft()
                self.checked += 1
                if failed is None and any(int(w) == 1 for w in block[:count].tolist()):
                    failed = what
                self.free_blocks.append(block)
        if failed is not None:
            raise NativeOpAborted(
                "%s: a bounded wait in the persistent kernel expired (device shared, preempted or paused?); the results of "
                "that call are invalid.  RTN_LSTM2_TIMEOUT_TICKS sets the bound in 10 ns ticks." % failed
            )

    def drain(self) -> None:
        """Wait for every queued look and check it (end of a step, end of the program, tests)."""
        with self.lock:
            events = [e for e, _, _, _ in self.pending]
        for e in events:
            e.synchronize()
        self.poll()


status_watch = StatusWatch()


def _cpu_not_supported(name):
    def _impl(*args):
        raise RuntimeError(
            "%s: this build implements the op for HIP (MI355X) tensors only; got CPU tensors. "
            "Move the inputs to the GPU." % name
        )

    return _impl


def _check_ndim(t: torch.Tensor, info: Dict[str, Any]):
    if t.dim() != info["ndim"]:
        raise RuntimeError("%s shape ndim is not %i, got shape %s" % (info["name"], info["ndim"], tuple(t.shape)))


def _row_pitch(t: torch.Tensor, *, itemsize: int) -> int:
    """
    Row pitch in elements if ``t`` ([T,B,width]) can be handed to the library as it is: unit stride along the last axis,
    rows of consecutive (frame, sequence) pairs a constant number of elements apart, 16-byte aligned rows.  0 if not
    (the caller then makes a contiguous copy).  A contiguous tensor gives ``width``.
    """
    if t.dim() != 3:
        return 0
    T, B, width = t.shape
    if T * B * width == 0:
        return width if t.is_contiguous() else 0
    ld = t.stride(1) if B > 1 else (t.stride(0) if T > 1 else width)
    ok = (width == 1 or t.stride(2) == 1) and ld >= width and (B == 1 or t.stride(1) == ld) and (T == 1 or t.stride(0) == B * ld)
    ok = ok and (ld * itemsize) % 16 == 0 and t.data_ptr() % 16 == 0
    return int(ld) if ok else 0


def _normalise_lstm2_args(X, W, y0, c0, i, *, pitched_x: bool = False):
    """Argument handling of the generated wrapper (returnn/torch/util/native_op.py:144-193) plus the op's shape
    asserts (returnn/native_op.py:1215-1223) as hard errors.  Returns the tensors to hand to the library and (T, B, n, bf16)."""
    infos = native_op.NativeLstm2.in_info
    for t, info in zip((X, W, y0, c0, i), infos):
        _check_ndim(t, info)
    device = X.device
    for t, info in zip((W, y0, c0, i), infos[1:]):
        if t.device != device:
            raise RuntimeError("%s is on %s but X is on %s" % (info["name"], t.device, device))
    bf16 = X.dtype == torch.bfloat16
    act = torch.bfloat16 if bf16 else torch.float32
    X, W, y0 = (t if t.dtype == act else t.to(act) for t in (X, W, y0))
    c0, i = (t if t.dtype == torch.float32 else t.to(torch.float32) for t in (c0, i))
    if not (pitched_x and _row_pitch(X, itemsize=X.element_size())):  # (a view with a row pitch goes to the library as it is)
        X = X if X.is_contiguous() else X.contiguous()
    W, y0, c0, i = (t if t.is_contiguous() else t.contiguous() for t in (W, y0, c0, i))
    T, B = i.shape
    n = y0.shape[1]
    expect = {"X": (T, B, 4 * n), "W": (n, 4 * n), "y0": (B, n), "c0": (B, n)}
    for name, t in (("X", X), ("W", W), ("y0", y0), ("c0", c0)):
        if tuple(t.shape) != expect[name]:
            raise RuntimeError(
                "NativeLstm2: %s has shape %s, expected %s (T=%i, B=%i from i; n=%i from y0)"
                % (name, tuple(t.shape), expect[name], T, B, n)
            )
    return (X, W, y0, c0, i), (T, B, n, bf16)


def _alloc_lstm2_outputs(T, B, n, bf16, device):
    act = torch.bfloat16 if bf16 else torch.float32
    Y = torch.empty((T, B, n), dtype=act, device=device)
    C = torch.empty((T, B, n), dtype=torch.float32, device=device)
    H = torch.empty((T, B, 4 * n), dtype=act, device=device)
    d = torch.empty((B, n), dtype=torch.float32, device=device)
    return Y, C, H, d


def _native_lstm2_device_impl(X, W, y0, c0, i, start, step, *, mode=_lib.MODE_AUTO):
    """``NativeLstm2`` on HIP tensors: normalise the arguments, allocate outputs and scratch, enqueue the library call."""
    (X, W, y0, c0, i), (T, B, n, bf16) = _normalise_lstm2_args(X, W, y0, c0, i)
    device = X.device
    lib = _lib.load()
    dtype = _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32
    with torch.cuda.device(device):
        status_watch.poll()
        Y, C, H, d = _alloc_lstm2_outputs(T, B, n, bf16, device)
        ws_bytes = int(lib.rtn_native_lstm2_fwd_workspace_bytes(T, B, n, dtype, mode))
        ws = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=device)
        stream = torch.cuda.current_stream(device).cuda_stream
        rc = lib.rtn_native_lstm2_fwd(
            X.data_ptr(), W.data_ptr(), y0.data_ptr(), c0.data_ptr(), i.data_ptr(), int(start), int(step),
            Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr(), T, B, n, dtype, mode,
            ws.data_ptr(), ws.numel(), stream,
        )  # fmt: skip
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("NativeLstm2", ws, 1, device)
    # The workspace goes back to the caching allocator here; the allocator keeps it out of other
    # streams' hands until the work queued on this stream has passed it (stream-ordered reuse).
    return Y, C, H, d


def _act_and_dtype(first: torch.Tensor):
    bf16 = first.dtype == torch.bfloat16
    act = torch.bfloat16 if bf16 else torch.float32
    dtype = _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32
    return act, dtype


def _lstm_generic_base_device_impl(Z, V_h, c, i, *, mode=_lib.MODE_AUTO):
    """``LstmGenericBase`` forward on HIP tensors (returnn/native_op.py:333-523)."""
    for t, info in zip((Z, V_h, c, i), native_op.LstmGenericBase.in_info):
        _check_ndim(t, info)
    device = Z.device
    act, dtype = _act_and_dtype(Z)
    Z, V_h = (t.to(act).contiguous() for t in (Z, V_h))
    c, i = (t.to(torch.float32).contiguous() for t in (c, i))
    T, B = i.shape
    n = c.shape[1]
    for name, t, shape in (("Z", Z, (T, B, 4 * n)), ("V_h", V_h, (n, 4 * n)), ("c", c, (B, n))):
        if tuple(t.shape) != shape:
            raise RuntimeError("LstmGenericBase: %s has shape %s, expected %s" % (name, tuple(t.shape), shape))
        if t.device != device:
            raise RuntimeError("LstmGenericBase: %s is on %s but Z is on %s" % (name, t.device, device))
    lib = _lib.load()
    with torch.cuda.device(device):
        status_watch.poll()
        Y = torch.empty((T, B, n), dtype=act, device=device)
        H = torch.empty((T, B, 4 * n), dtype=act, device=device)
        d = torch.empty((B, n), dtype=torch.float32, device=device)
        ws = torch.empty((max(int(lib.rtn_lstm_generic_base_fwd_workspace_bytes(T, B, n, dtype, mode)), 256),), dtype=torch.uint8, device=device)
        rc = lib.rtn_lstm_generic_base_fwd(
            Z.data_ptr(), V_h.data_ptr(), c.data_ptr(), i.data_ptr(), Y.data_ptr(), H.data_ptr(), d.data_ptr(), T, B, n, dtype, mode,
            ws.data_ptr(), ws.numel(), torch.cuda.current_stream(device).cuda_stream,
        )  # fmt: skip
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("LstmGenericBase", ws, 1, device)
    return Y, H, d


def _lstm_low_mem_device_impl(X, W, b, y0, c0, i, start, step, *, mode=_lib.MODE_AUTO):
    """``LstmLowMem`` forward on HIP tensors (returnn/native_op.py:577-836)."""
    for t, info in zip((X, W, b, y0, c0, i), native_op.LstmLowMem.in_info):
        _check_ndim(t, info)
    device = X.device
    act, dtype = _act_and_dtype(X)
    X, W, b, y0 = (t.to(act).contiguous() for t in (X, W, b, y0))
    c0, i = (t.to(torch.float32).contiguous() for t in (c0, i))
    T, B = i.shape
    n = y0.shape[1]
    n_in = X.shape[2]
    for name, t, shape in (("X", X, (T, B, n_in)), ("W", W, (n_in + n, 4 * n)), ("b", b, (4 * n,)), ("y0", y0, (B, n)), ("c0", c0, (B, n))):
        if tuple(t.shape) != shape:
            raise RuntimeError("LstmLowMem: %s has shape %s, expected %s" % (name, tuple(t.shape), shape))
        if t.device != device:
            raise RuntimeError("LstmLowMem: %s is on %s but X is on %s" % (name, t.device, device))
    lib = _lib.load()
    with torch.cuda.device(device):
        status_watch.poll()
        Y = torch.empty((T, B, n), dtype=act, device=device)
        C = torch.empty((T, B, n), dtype=torch.float32, device=device)
        d = torch.empty((B, n), dtype=torch.float32, device=device)
        ws = torch.empty((max(int(lib.rtn_lstm_low_mem_fwd_workspace_bytes(T, B, n_in, n, dtype, mode)), 256),), dtype=torch.uint8, device=device)
        rc = lib.rtn_lstm_low_mem_fwd(
            X.data_ptr(), W.data_ptr(), b.data_ptr(), y0.data_ptr(), c0.data_ptr(), i.data_ptr(), int(start), int(step),
            Y.data_ptr(), C.data_ptr(), d.data_ptr(), T, B, n_in, n, dtype, mode, ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream(device).cuda_stream,
        )  # fmt: skip
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("LstmLowMem", ws, 1, device)
    return Y, C, d


def native_lstm2_multi(calls, *, mode: Optional[str] = None, joint_output: bool = False):
    """
    Several independent ``NativeLstm2`` calls of one shape through one entry of the library, e.g. the forward and
    the backward direction of a bidirectional layer.  Same results as calling the op once per element; when the
    device can hold them together they run in a single launch and overlap.

    ``X`` may be a view with a row pitch (e.g. ``P[:, :, 4n:8n]`` of a projection ``P [T,B,8n]`` for both directions): it is
    handed to the library as it is, not copied.

    :param calls: sequence of ``(X, W, y0, c0, i, start, step)``, all with the same T, B, n and element type
    :param mode: as for :class:`OpMaker`; default "auto"
    :param joint_output: the calls write their outputs side by side into ONE array ``[T,B,count*n]`` (what a bidirectional
        layer hands on, returnn/tf/layers/rec.py:1229-1270): every ``Y`` returned is a view of it
    :return: list of ``(Y, C, H, d)``; with ``joint_output`` a pair of that list and the joint array
    """
    calls = list(calls)
    if not calls:
        return []
    lib = _lib.load()
    norm = [_normalise_lstm2_args(*c[:5], pitched_x=True) for c in calls]
    shape = norm[0][1]
    device = norm[0][0][0].device
    for tensors, sh in norm:
        if sh != shape:
            raise RuntimeError("native_lstm2_multi: all calls need the same T, B, n and element type; got %r and %r" % (shape, sh))
        if tensors[0].device != device:
            raise RuntimeError("native_lstm2_multi: all calls must be on one device")
    if not norm[0][0][0].is_cuda:
        raise RuntimeError("NativeLstm2: this build implements the op for HIP (MI355X) tensors only; got CPU tensors.")
    T, B, n, bf16 = shape
    dtype = _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32
    mode_code = _lib.MODES[mode or "auto"]
    count = len(calls)
    arr = (_lib.Lstm2Call * count)()
    outs = []
    with torch.cuda.device(device):
        status_watch.poll()
        act = torch.bfloat16 if bf16 else torch.float32
        joint = torch.empty((T, B, count * n), dtype=act, device=device) if joint_output else None
        if joint is not None and ((n * joint.element_size()) % 16 != 0):
            joint = None  # (columns of the calls would not be 16-byte aligned: separate arrays, joined below)
        for k, ((X, W, y0, c0, i), c) in enumerate(zip((t for t, _ in norm), calls)):
            Y, C, H, d = _alloc_lstm2_outputs(T, B, n, bf16, device)
            if joint is not None:
                Y = joint[:, :, k * n : (k + 1) * n]
            outs.append((Y, C, H, d))
            arr[k] = _lib.Lstm2Call(
                X.data_ptr(), W.data_ptr(), y0.data_ptr(), c0.data_ptr(), i.data_ptr(), int(c[5]), int(c[6]),
                Y.data_ptr(), C.data_ptr(), H.data_ptr(), d.data_ptr(),
                0 if X.is_contiguous() else _row_pitch(X, itemsize=X.element_size()), 0 if joint is None else count * n,
            )  # fmt: skip
        ws_bytes = int(lib.rtn_native_lstm2_fwd_multi_workspace_bytes(count, T, B, n, dtype, mode_code))
        ws = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=device)
        stream = torch.cuda.current_stream(device).cuda_stream
        rc = lib.rtn_native_lstm2_fwd_multi(arr, count, T, B, n, dtype, mode_code, ws.data_ptr(), ws.numel(), stream)
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("NativeLstm2 (%i calls)" % count, ws, count, device)
    del norm  # the normalised inputs stay alive until here; the stream-ordered allocator covers the rest
    if joint_output:
        return outs, (joint if joint is not None else torch.cat([o[0] for o in outs], dim=-1))
    return outs


def _normalise_grad_args(W, y0, c0, i, Y, C, H, DY, Dd):
    if not Y.is_cuda:
        raise RuntimeError("NativeLstm2 gradient: this build implements the op for HIP (MI355X) tensors only; got CPU tensors.")
    bf16 = Y.dtype == torch.bfloat16
    act = torch.bfloat16 if bf16 else torch.float32
    device = Y.device
    W, y0, H = (t.to(act).contiguous() for t in (W, y0, H))
    # (Y and DY may be views with a row pitch, e.g. one direction's half of a [T,B,2n] array: handed over as they are)
    Y, DY = (t if _row_pitch(t, itemsize=t.element_size()) else t.contiguous() for t in (Y.to(act), DY.to(act)))
    c0, i, C, Dd = (t.to(torch.float32).contiguous() for t in (c0, i, C, Dd))
    T, B = i.shape
    n = y0.shape[1]
    expect = {"W": (n, 4 * n), "y0": (B, n), "c0": (B, n), "Y": (T, B, n), "C": (T, B, n), "H": (T, B, 4 * n),
              "DY": (T, B, n), "Dd": (B, n)}  # fmt: skip
    for name, t in (("W", W), ("y0", y0), ("c0", c0), ("Y", Y), ("C", C), ("H", H), ("DY", DY), ("Dd", Dd)):
        if tuple(t.shape) != expect[name]:
            raise RuntimeError("NativeLstm2 gradient: %s has shape %s, expected %s" % (name, tuple(t.shape), expect[name]))
        if t.device != device:
            raise RuntimeError("NativeLstm2 gradient: %s is on %s but Y is on %s" % (name, t.device, device))
    return (W, y0, c0, i, Y, C, H, DY, Dd), (T, B, n, bf16)


def _alloc_grad_outputs(T, B, n, bf16, device):
    act = torch.bfloat16 if bf16 else torch.float32
    DX = torch.empty((T, B, 4 * n), dtype=act, device=device)
    DW = torch.empty((n, 4 * n), dtype=torch.float32, device=device)
    Dy0 = torch.empty((B, n), dtype=act, device=device)
    Dc0 = torch.empty((B, n), dtype=torch.float32, device=device)
    return DX, DW, Dy0, Dc0


def native_lstm2_grad(W, y0, c0, i, start, step, Y, C, H, DY, Dd):
    """
    The gradient op of ``NativeLstm2`` on HIP tensors (returnn/native_op.py:1288-1464; arguments as
    ``grad_input_map`` :1071-1077 without X, which the computation does not read).

    :return: DX [T,B,4n] and Dy0 [B,n] in the element type of Y; DW [n,4n] and Dc0 [B,n] in float32
    """
    return native_lstm2_grad_multi([(W, y0, c0, i, start, step, Y, C, H, DY, Dd)])[0]


def native_lstm2_grad_multi(calls, *, joint_dx: bool = False):
    """
    Several gradient calls of one shape in one library entry (``rtn_native_lstm2_bwd_multi``): the two directions of
    a bidirectional layer share one kernel launch when the device can hold both.

    ``Y`` and ``DY`` may be views with a row pitch (one direction's columns of a ``[T,B,2n]`` array): they are handed to the
    library as they are, not copied.

    :param calls: list of ``(W, y0, c0, i, start, step, Y, C, H, DY, Dd)``
    :param joint_dx: the calls write their ``DX`` side by side into ONE array ``[T,B,count*4n]`` (the error of a projection
        made once for all of them): every ``DX`` returned is a view of it
    :return: list of ``(DX, DW, Dy0, Dc0)``, element k as :func:`native_lstm2_grad` gives for ``calls[k]``; with
        ``joint_dx`` a pair of that list and the joint array
    """
    calls = list(calls)
    if not calls:
        return ([], None) if joint_dx else []
    norm = []
    shape = None
    for W, y0, c0, i, start, step, Y, C, H, DY, Dd in calls:
        tensors, this = _normalise_grad_args(W, y0, c0, i, Y, C, H, DY, Dd)
        if shape is None:
            shape, device = this, tensors[4].device
        elif this != shape or tensors[4].device != device:
            raise RuntimeError("native_lstm2_grad_multi: all calls must have one shape, dtype and device; got %r and %r" % (shape, this))
        norm.append((tensors, int(start), int(step)))
    T, B, n, bf16 = shape
    lib = _lib.load()
    dtype = _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32
    count = len(norm)
    with torch.cuda.device(device):
        status_watch.poll()
        outs = [_alloc_grad_outputs(T, B, n, bf16, device) for _ in range(count)]
        joint = None
        if joint_dx and (4 * n * outs[0][0].element_size()) % 16 == 0:  # (else: separate arrays, joined below)
            joint = torch.empty((T, B, count * 4 * n), dtype=outs[0][0].dtype, device=device)
            outs = [(joint[:, :, k * 4 * n : (k + 1) * 4 * n],) + o[1:] for k, o in enumerate(outs)]
        ws_bytes = int(lib.rtn_native_lstm2_bwd_multi_workspace_bytes(count, T, B, n, dtype))
        ws = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=device)
        arr = (_lib.Lstm2BwdCall * count)()
        for k, ((W, y0, c0, i, Y, C, H, DY, Dd), start, step) in enumerate(norm):
            DX, DW, Dy0, Dc0 = outs[k]
            arr[k] = _lib.Lstm2BwdCall(
                W.data_ptr(), y0.data_ptr(), c0.data_ptr(), i.data_ptr(), start, step, Y.data_ptr(), C.data_ptr(), H.data_ptr(),
                DY.data_ptr(), Dd.data_ptr(), DX.data_ptr(), DW.data_ptr(), Dy0.data_ptr(), Dc0.data_ptr(),
                0 if Y.is_contiguous() else _row_pitch(Y, itemsize=Y.element_size()),
                0 if DY.is_contiguous() else _row_pitch(DY, itemsize=DY.element_size()),
                0 if joint is None else count * 4 * n,
            )  # fmt: skip
        rc = lib.rtn_native_lstm2_bwd_multi(arr, count, T, B, n, dtype, ws.data_ptr(), ws.numel(), torch.cuda.current_stream(device).cuda_stream)
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("NativeLstm2 gradient (%i calls)" % count, ws, count, device)
    del norm  # (the normalised inputs stay alive until here; the stream-ordered allocator covers the rest)
    if joint_dx:
        return outs, (joint if joint is not None else torch.cat([o[0] for o in outs], dim=-1))
    return outs


class NativeLstm2Function(torch.autograd.Function):
    """
    ``NativeLstm2`` with its gradient, for training through autograd: ``Y, C, H, d = NativeLstm2Function.apply(X, W,
    y0, c0, i, start, step)``.  Gradients flow from Y and d to X, W, y0 and c0; C and H are marked non-differentiable
    (the reference's gradient op ignores error signals on them too, returnn/native_op.py:1071-1077); the mask gets none.
    """

    @staticmethod
    def forward(ctx, X, W, y0, c0, i, start, step):
        op = make_op(native_op.NativeLstm2)
        Y, C, H, d = op(X, W, y0, c0, i, int(start), int(step))
        ctx.save_for_backward(W, y0, c0, i, Y, C, H)
        ctx.start, ctx.step = int(start), int(step)
        ctx.in_dtypes = (X.dtype, W.dtype, y0.dtype, c0.dtype)
        ctx.set_materialize_grads(False)  # (no zero tensors for outputs without a gradient: backward takes None)
        ctx.mark_non_differentiable(C, H)
        return Y, C, H, d

    @staticmethod
    def backward(ctx, DY, _DC, _DH, Dd):
        W, y0, c0, i, Y, C, H = ctx.saved_tensors
        if DY is None:
            DY = torch.zeros_like(Y)
        if Dd is None:
            Dd = torch.zeros_like(c0, dtype=torch.float32)
        DX, DW, Dy0, Dc0 = native_lstm2_grad(W, y0, c0, i, ctx.start, ctx.step, Y, C, H, DY, Dd)
        dX, dW, dy0, dc0 = (g.to(t) for g, t in zip((DX, DW, Dy0, Dc0), ctx.in_dtypes))
        return dX, dW, dy0, dc0, None, None, None


def lstm_generic_base_grad(V_h, c, i, Y, H, DY, Dd):
    """
    The gradient op of ``LstmGenericBase`` on HIP tensors (returnn/native_op.py:430-485, :525-574; arguments as its
    ``grad_input_map`` :374-378).

    :return: DZ [T,B,4n] in the element type of Y; DV_h [n,4n] and Dc [B,n] in float32
    """
    if not Y.is_cuda:
        raise RuntimeError("LstmGenericBase gradient: this build implements the op for HIP (MI355X) tensors only; got CPU tensors.")
    bf16 = Y.dtype == torch.bfloat16
    act = torch.bfloat16 if bf16 else torch.float32
    device = Y.device
    V_h, Y, H, DY = (t.to(act).contiguous() for t in (V_h, Y, H, DY))
    c, i, Dd = (t.to(torch.float32).contiguous() for t in (c, i, Dd))
    T, B = i.shape
    n = c.shape[1]
    expect = {"V_h": (n, 4 * n), "c": (B, n), "Y": (T, B, n), "H": (T, B, 4 * n), "DY": (T, B, n), "Dd": (B, n)}
    for name, t in (("V_h", V_h), ("c", c), ("Y", Y), ("H", H), ("DY", DY), ("Dd", Dd)):
        if tuple(t.shape) != expect[name]:
            raise RuntimeError("LstmGenericBase gradient: %s has shape %s, expected %s" % (name, tuple(t.shape), expect[name]))
        if t.device != device:
            raise RuntimeError("LstmGenericBase gradient: %s is on %s but Y is on %s" % (name, t.device, device))
    lib = _lib.load()
    dtype = _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32
    with torch.cuda.device(device):
        status_watch.poll()
        DZ = torch.empty((T, B, 4 * n), dtype=act, device=device)
        DV_h = torch.empty((n, 4 * n), dtype=torch.float32, device=device)
        Dc = torch.empty((B, n), dtype=torch.float32, device=device)
        ws = torch.empty((max(int(lib.rtn_lstm_generic_base_bwd_workspace_bytes(T, B, n, dtype)), 256),), dtype=torch.uint8, device=device)
        rc = lib.rtn_lstm_generic_base_bwd(
            V_h.data_ptr(), c.data_ptr(), i.data_ptr(), Y.data_ptr(), H.data_ptr(), DY.data_ptr(), Dd.data_ptr(), DZ.data_ptr(),
            DV_h.data_ptr(), Dc.data_ptr(), T, B, n, dtype, ws.data_ptr(), ws.numel(), torch.cuda.current_stream(device).cuda_stream,
        )  # fmt: skip
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("LstmGenericBase gradient", ws, 1, device)
    return DZ, DV_h, Dc


class LstmGenericBaseFunction(torch.autograd.Function):
    """``LstmGenericBase`` with its gradient: ``Y, H, d = LstmGenericBaseFunction.apply(Z, V_h, c, i)``; gradients flow from
    Y and d to Z, V_h and c (H is a non-differentiable output, the mask gets none)."""

    @staticmethod
    def forward(ctx, Z, V_h, c, i):
        Y, H, d = make_op(native_op.LstmGenericBase)(Z, V_h, c, i)
        ctx.save_for_backward(V_h, c, i, Y, H)
        ctx.in_dtypes = (Z.dtype, V_h.dtype, c.dtype)
        ctx.set_materialize_grads(False)  # (no zero tensors for outputs without a gradient: backward takes None)
        ctx.mark_non_differentiable(H)
        return Y, H, d

    @staticmethod
    def backward(ctx, DY, _DH, Dd):
        V_h, c, i, Y, H = ctx.saved_tensors
        DY = torch.zeros_like(Y) if DY is None else DY
        Dd = torch.zeros_like(c, dtype=torch.float32) if Dd is None else Dd
        grads = lstm_generic_base_grad(V_h, c, i, Y, H, DY, Dd)
        return (*(g.to(t) for g, t in zip(grads, ctx.in_dtypes)), None)


def lstm_low_mem_grad(X, W, b, y0, c0, i, start, step, Y, C, DY, Dd):
    """
    The gradient op of ``LstmLowMem`` on HIP tensors (returnn/native_op.py:864-1026; arguments as its ``grad_input_map``
    :619-625).  Results as the reference's formulas give them, also on masked frames; strides for which the reference's
    loop would leave the frames of the forward pass are refused (see ``rtn_lstm_low_mem_bwd`` in the C header).

    :return: DX [T,B,n_in] and Dh [B,n] in the element type of Y; DW [n_in+n,4n], Db [4n] and Dc [B,n] in float32
    """
    if not Y.is_cuda:
        raise RuntimeError("LstmLowMem gradient: this build implements the op for HIP (MI355X) tensors only; got CPU tensors.")
    bf16 = Y.dtype == torch.bfloat16
    act = torch.bfloat16 if bf16 else torch.float32
    device = Y.device
    X, W, b, y0, Y, DY = (t.to(act).contiguous() for t in (X, W, b, y0, Y, DY))
    c0, i, C, Dd = (t.to(torch.float32).contiguous() for t in (c0, i, C, Dd))
    T, B = i.shape
    n = y0.shape[1]
    n_in = X.shape[2]
    expect = {"X": (T, B, n_in), "W": (n_in + n, 4 * n), "b": (4 * n,), "y0": (B, n), "c0": (B, n), "Y": (T, B, n), "C": (T, B, n),
              "DY": (T, B, n), "Dd": (B, n)}  # fmt: skip
    for name, t in (("X", X), ("W", W), ("b", b), ("y0", y0), ("c0", c0), ("Y", Y), ("C", C), ("DY", DY), ("Dd", Dd)):
        if tuple(t.shape) != expect[name]:
            raise RuntimeError("LstmLowMem gradient: %s has shape %s, expected %s" % (name, tuple(t.shape), expect[name]))
        if t.device != device:
            raise RuntimeError("LstmLowMem gradient: %s is on %s but Y is on %s" % (name, t.device, device))
    lib = _lib.load()
    dtype = _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32
    with torch.cuda.device(device):
        status_watch.poll()
        DX = torch.empty((T, B, n_in), dtype=act, device=device)
        DW = torch.empty((n_in + n, 4 * n), dtype=torch.float32, device=device)
        Db = torch.empty((4 * n,), dtype=torch.float32, device=device)
        Dh = torch.empty((B, n), dtype=act, device=device)
        Dc = torch.empty((B, n), dtype=torch.float32, device=device)
        ws = torch.empty((max(int(lib.rtn_lstm_low_mem_bwd_workspace_bytes(T, B, n_in, n, dtype)), 256),), dtype=torch.uint8, device=device)
        rc = lib.rtn_lstm_low_mem_bwd(
            X.data_ptr(), W.data_ptr(), b.data_ptr(), y0.data_ptr(), c0.data_ptr(), i.data_ptr(), int(start), int(step), Y.data_ptr(),
            C.data_ptr(), DY.data_ptr(), Dd.data_ptr(), DX.data_ptr(), DW.data_ptr(), Db.data_ptr(), Dh.data_ptr(), Dc.data_ptr(),
            T, B, n_in, n, dtype, ws.data_ptr(), ws.numel(), torch.cuda.current_stream(device).cuda_stream,
        )  # fmt: skip
        _lib.check(rc)
        if T * B * n > 0:  # (an empty problem does not touch its workspace)
            status_watch.after_call("LstmLowMem gradient", ws, 1, device)
    return DX, DW, Db, Dh, Dc


class LstmLowMemFunction(torch.autograd.Function):
    """``LstmLowMem`` with its gradient: ``Y, C, d = LstmLowMemFunction.apply(X, W, b, y0, c0, i, start, step)``; gradients
    flow from Y and d to X, W, b, y0 and c0 (C is a non-differentiable output, as in the reference :596; the mask gets none)."""

    @staticmethod
    def forward(ctx, X, W, b, y0, c0, i, start, step):
        Y, C, d = make_op(native_op.LstmLowMem)(X, W, b, y0, c0, i, int(start), int(step))
        ctx.save_for_backward(X, W, b, y0, c0, i, Y, C)
        ctx.start, ctx.step = int(start), int(step)
        ctx.in_dtypes = (X.dtype, W.dtype, b.dtype, y0.dtype, c0.dtype)
        ctx.set_materialize_grads(False)  # (no zero tensors for outputs without a gradient: backward takes None)
        ctx.mark_non_differentiable(C)
        return Y, C, d

    @staticmethod
    def backward(ctx, DY, _DC, Dd):
        X, W, b, y0, c0, i, Y, C = ctx.saved_tensors
        DY = torch.zeros_like(Y) if DY is None else DY
        Dd = torch.zeros_like(c0, dtype=torch.float32) if Dd is None else Dd
        grads = lstm_low_mem_grad(X, W, b, y0, c0, i, ctx.start, ctx.step, Y, C, DY, Dd)
        return (*(g.to(t) for g, t in zip(grads, ctx.in_dtypes)), None, None, None)


class NativeLstm2PairFunction(torch.autograd.Function):
    """
    The two directions of a bidirectional layer as one differentiable call:
    ``Yf, Cf, Hf, df, Yb, Cb, Hb, db = NativeLstm2PairFunction.apply(Xf, Wf, y0f, c0f, Xb, Wb, y0b, c0b, i)``, the forward
    direction with (start, step) = (0, 1), the backward direction with (0, -1).  Forward and gradient each go through
    the library's multi-call entry (one kernel launch for both directions where the device can hold them); results are
    those of two :class:`NativeLstm2Function` calls.
    """

    @staticmethod
    def forward(ctx, Xf, Wf, y0f, c0f, Xb, Wb, y0b, c0b, i):
        (Yf, Cf, Hf, df), (Yb, Cb, Hb, db) = native_lstm2_multi([(Xf, Wf, y0f, c0f, i, 0, 1), (Xb, Wb, y0b, c0b, i, 0, -1)])
        ctx.save_for_backward(Wf, y0f, c0f, Wb, y0b, c0b, i, Yf, Cf, Hf, Yb, Cb, Hb)
        ctx.in_dtypes = (Xf.dtype, Wf.dtype, y0f.dtype, c0f.dtype, Xb.dtype, Wb.dtype, y0b.dtype, c0b.dtype)
        ctx.set_materialize_grads(False)  # (no zero tensors for outputs without a gradient: backward takes None)
        ctx.mark_non_differentiable(Cf, Hf, Cb, Hb)
        return Yf, Cf, Hf, df, Yb, Cb, Hb, db

    @staticmethod
    def backward(ctx, DYf, _DCf, _DHf, Ddf, DYb, _DCb, _DHb, Ddb):
        Wf, y0f, c0f, Wb, y0b, c0b, i, Yf, Cf, Hf, Yb, Cb, Hb = ctx.saved_tensors
        DYf = torch.zeros_like(Yf) if DYf is None else DYf
        DYb = torch.zeros_like(Yb) if DYb is None else DYb
        Ddf = torch.zeros_like(c0f, dtype=torch.float32) if Ddf is None else Ddf
        Ddb = torch.zeros_like(c0b, dtype=torch.float32) if Ddb is None else Ddb
        gf, gb = native_lstm2_grad_multi(
            [(Wf, y0f, c0f, i, 0, 1, Yf, Cf, Hf, DYf, Ddf), (Wb, y0b, c0b, i, 0, -1, Yb, Cb, Hb, DYb, Ddb)]
        )
        grads = [g.to(t) for g, t in zip(tuple(gf) + tuple(gb), ctx.in_dtypes)]
        return (*grads, None)


class NativeLstm2BidirFunction(torch.autograd.Function):
    """
    A bidirectional layer on ONE projection: ``Y, df, db = NativeLstm2BidirFunction.apply(P, Wf, y0f, c0f, Wb, y0b, c0b, i)``
    with ``P [T,B,8n]`` holding the pre-projected gates of the forward direction in columns ``[0,4n)`` and of the backward
    direction in ``[4n,8n)``, and ``Y [T,B,2n]`` the outputs side by side (what returnn/tf/layers/rec.py:1229-1270 builds
    from two op calls and a concat).  The directions read and write their columns in place (row pitch 8n and 2n); the
    gradient reads the error of ``Y`` the same way and writes the error of ``P`` as one array, so neither pass copies or
    concatenates an activation.  Results are those of two :class:`NativeLstm2Function` calls, (0, 1) and (0, -1).
    """

    @staticmethod
    def forward(ctx, P, Wf, y0f, c0f, Wb, y0b, c0b, i):
        n = y0f.shape[1]
        if P.dim() != 3 or P.shape[2] != 8 * n:
            raise RuntimeError("NativeLstm2 (bidirectional): P has shape %s, expected [T,B,%i]" % (tuple(P.shape), 8 * n))
        outs, Y = native_lstm2_multi(
            [(P[:, :, : 4 * n], Wf, y0f, c0f, i, 0, 1), (P[:, :, 4 * n :], Wb, y0b, c0b, i, 0, -1)], joint_output=True
        )
        (_, Cf, Hf, df), (_, Cb, Hb, db) = outs
        ctx.save_for_backward(Wf, y0f, c0f, Wb, y0b, c0b, i, Y, Cf, Hf, Cb, Hb)
        ctx.in_dtypes = (P.dtype, Wf.dtype, y0f.dtype, c0f.dtype, Wb.dtype, y0b.dtype, c0b.dtype)
        ctx.set_materialize_grads(False)  # (no zero tensors for outputs without a gradient: backward takes None)
        return Y, df, db

    @staticmethod
    def backward(ctx, DY, Ddf, Ddb):
        Wf, y0f, c0f, Wb, y0b, c0b, i, Y, Cf, Hf, Cb, Hb = ctx.saved_tensors
        n = y0f.shape[1]
        DY = torch.zeros_like(Y) if DY is None else DY
        Ddf = torch.zeros_like(c0f, dtype=torch.float32) if Ddf is None else Ddf
        Ddb = torch.zeros_like(c0b, dtype=torch.float32) if Ddb is None else Ddb
        (gf, gb), DP = native_lstm2_grad_multi(
            [
                (Wf, y0f, c0f, i, 0, 1, Y[:, :, :n], Cf, Hf, DY[:, :, :n], Ddf),
                (Wb, y0b, c0b, i, 0, -1, Y[:, :, n:], Cb, Hb, DY[:, :, n:], Ddb),
            ],
            joint_dx=True,
        )
        grads = (DP,) + tuple(gf[1:]) + tuple(gb[1:])
        return (*(g.to(t) for g, t in zip(grads, ctx.in_dtypes)), None)


def lstm_last_output(Y: torch.Tensor, y0: torch.Tensor, i: torch.Tensor, start: int = 0, step: int = 1) -> torch.Tensor:
    """
    Final output per sequence, the caller-side ``_lstm_last_output`` of the reference
    (returnn/tf/native_op.py:913-929), computed by the library on the device.

    :param Y: [T,B,n] output of the op
    :param y0: [B,n]
    :param i: [T,B] mask
    :return: [B,n]
    """
    if not Y.is_cuda:
        raise RuntimeError("lstm_last_output: this build implements the op for HIP (MI355X) tensors only")
    bf16 = Y.dtype == torch.bfloat16
    act = torch.bfloat16 if bf16 else torch.float32
    Y = Y.to(act)
    ldY = _row_pitch(Y, itemsize=Y.element_size())
    if not ldY:
        Y, ldY = Y.contiguous(), Y.shape[2]
    y0 = y0.to(act).contiguous()
    i = i.to(torch.float32).contiguous()
    T, B, n = Y.shape
    if tuple(y0.shape) != (B, n) or tuple(i.shape) != (T, B):
        raise RuntimeError("lstm_last_output: y0 %s / i %s do not match Y %s" % (tuple(y0.shape), tuple(i.shape), tuple(Y.shape)))
    lib = _lib.load()
    with torch.cuda.device(Y.device):
        out = torch.empty((B, n), dtype=act, device=Y.device)
        rc = lib.rtn_native_lstm2_last_output(
            Y.data_ptr(), y0.data_ptr(), i.data_ptr(), int(start), int(step), out.data_ptr(), T, B, n,
            _lib.DTYPE_BF16 if bf16 else _lib.DTYPE_F32, int(ldY), torch.cuda.current_stream(Y.device).cuda_stream,
        )  # fmt: skip
    _lib.check(rc)
    return out
