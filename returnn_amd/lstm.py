"""
LSTM layer forward on top of the NativeLstm2 op: the raw-tensor side of the reference's frontend LSTM.

The reference's ``rf.LSTM`` (returnn/frontend/rec.py:16-77) holds ``ff_weight [4*out,in]``,
``rec_weight [4*out,out]`` and ``bias [4*out]`` in PyTorch's gate order (input, forget, cell-in, output) and
hands them to the backend; ``TorchBackend.lstm`` (returnn/torch/frontend/_backend.py:2718-2850) makes the
input time-major, packs it by the sequence lengths, calls ``torch.lstm`` and returns the padded output
plus the state after each sequence's last frame.  The TF-layers backend shows the mapping onto the native op
(returnn/tf/frontend_layers/_backend.py:1199-1222): gates reordered to cell-in, input, forget, output, weights
transposed to ``[in|out, 4*out]``, the input projection computed outside the op.

:func:`lstm` is that backend function on plain HIP tensors (time-major ``[T,B,in]``, lengths as a tensor
instead of a ``Dim``): one projection GEMM (hipBLASLt through ``torch.addmm``) into the op's ``X`` layout,
then one ``NativeLstm2`` call with the right-padded 0/1 mask; output frames beyond a sequence's length are 0
(what ``pad_packed_sequence`` yields), the new state is ``(h, c)`` after the last valid frame.
``direction=-1`` runs the recurrence from each sequence's last frame to its first without reversing anything
in memory (the caller protocol of returnn/tf/layers/rec.py:1229-1270).

With gradients enabled and an input that requires them, the same functions go through
``NativeLstm2Function`` (the op with its gradient op) and torch's autograd, so the layer trains like ``rf.LSTM``.

:class:`LSTM` and :class:`LstmState` mirror the module and its state (parameters in the frontend's names and layout).
:class:`BLSTM` is one bidirectional layer (:func:`blstm`: ONE projection for both directions, which then go through the
library's multi-call entry -- one launch when the device can hold both -- reading their columns of the projection and
writing their columns of the one output); it keeps its parameters in the op's layout, so that a training step
converts nothing, and speaks the frontend's layout in ``state_dict`` / ``load_state_dict`` / :meth:`BLSTM.frontend_params`.
:class:`BlstmEncoder` stacks such layers.
"""

from __future__ import annotations

import math
from typing import NamedTuple, Optional, Sequence, Tuple, Union

import torch

from . import native_op
from .torch_native_op import NativeLstm2BidirFunction, NativeLstm2Function, lstm_last_output, make_op, native_lstm2_multi

__all__ = [
    "lstm", "blstm", "prepare_weights", "prepare_blstm_weights", "join_weights", "LstmWeights", "BlstmWeights", "LSTM", "BLSTM",
    "LstmState", "BlstmEncoder", "sequence_mask_time_major",
]  # fmt: skip


class LstmState(NamedTuple):
    """``h`` and ``c``, both [B,out] (returnn/frontend/rec.py:86-93)."""

    h: torch.Tensor
    c: torch.Tensor


class LstmWeights(NamedTuple):
    """Weights in the op's layout: gate order cell-in, input, forget, output along the ``4*out`` axis."""

    ff: torch.Tensor  # [in, 4*out] (from prepare_weights: a transposed view of a contiguous [4*out, in] matrix)
    rec: torch.Tensor  # [out, 4*out]
    bias: Optional[torch.Tensor]  # [4*out] or None


class BlstmWeights(NamedTuple):
    """Weights of a bidirectional layer with ONE input projection for both directions: along the ``8*out`` axis the forward
    direction's gates (cell-in, input, forget, output), then the backward direction's."""

    ff: torch.Tensor  # [in, 8*out] (a transposed view of a contiguous [8*out, in] matrix)
    rec_fwd: torch.Tensor  # [out, 4*out]
    rec_bwd: torch.Tensor  # [out, 4*out]
    bias: Optional[torch.Tensor]  # [8*out] or None


def _to_native_gate_order(w: torch.Tensor) -> torch.Tensor:
    """[4*out, ...] in (input, forget, cell-in, output) blocks -> (cell-in, input, forget, output)."""
    i, f, g, o = w.chunk(4, dim=0)
    return torch.cat((g, i, f, o), dim=0)


def prepare_weights(
    ff_weight: torch.Tensor, rec_weight: torch.Tensor, bias: Optional[torch.Tensor], *, dtype: Optional[torch.dtype] = None
) -> LstmWeights:
    """
    Frontend parameters -> op layout (returnn/tf/frontend_layers/_backend.py:1199-1222): reorder the gate blocks
    and transpose.  (:class:`LSTM` and :class:`BLSTM` keep their parameters in the op's layout and need none of this.)

    :param ff_weight: [4*out, in]
    :param rec_weight: [4*out, out]
    :param bias: [4*out] or None
    :param dtype: activation type of the run (float32 or bfloat16); default: as ``ff_weight``
    """
    if ff_weight.dim() != 2 or rec_weight.dim() != 2 or ff_weight.shape[0] != rec_weight.shape[0]:
        raise ValueError("lstm: ff_weight %s / rec_weight %s" % (tuple(ff_weight.shape), tuple(rec_weight.shape)))
    out4, out = rec_weight.shape
    if out4 != 4 * out:
        raise ValueError("lstm: rec_weight must be [4*out,out], got %s" % (tuple(rec_weight.shape),))
    if bias is not None and tuple(bias.shape) != (out4,):
        raise ValueError("lstm: bias must be [4*out], got %s" % (tuple(bias.shape),))
    dtype = dtype or ff_weight.dtype
    # (kept as the [4*out, in] matrix it comes as, transposed as a view only: the projection GEMM and its two gradient
    # GEMMs are faster on that layout than on a transposed copy -- bf16, 32 000 x 2048 x 4096 on MI355X: 0.46 / 0.43 /
    # 0.51 ms against 0.52 / 0.37 / 0.59 -- and the copy and its gradient are saved)
    ff = _to_native_gate_order(ff_weight).to(dtype).contiguous().t()
    rec = _to_native_gate_order(rec_weight).t().to(dtype).contiguous()
    b = None if bias is None else _to_native_gate_order(bias).to(dtype).contiguous()
    return LstmWeights(ff=ff, rec=rec, bias=b)


def _native_gate_blocks(w: torch.Tensor):
    i, f, g, o = w.chunk(4, dim=0)
    return g, i, f, o


def prepare_blstm_weights(
    fwd: Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]],
    bwd: Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]],
    *,
    dtype: Optional[torch.dtype] = None,
) -> BlstmWeights:
    """
    Frontend parameters of the two directions -> one projection matrix ``[in, 8*out]`` and the two recurrent matrices in
    the op's layout.  The eight gate blocks are gathered in a single copy (reorder and join at once).

    :param fwd: ``(ff_weight [4*out,in], rec_weight [4*out,out], bias [4*out] or None)`` of the forward-in-time direction
    :param bwd: the same of the backward-in-time direction
    :param dtype: activation type of the run (float32 or bfloat16); default: as ``ff_weight``
    """
    (ff_f, rec_f, b_f), (ff_b, rec_b, b_b) = fwd, bwd
    if ff_f.shape != ff_b.shape or rec_f.shape != rec_b.shape or (b_f is None) != (b_b is None):
        raise ValueError("blstm: the two directions need parameters of one shape")
    if ff_f.dim() != 2 or rec_f.dim() != 2 or ff_f.shape[0] != rec_f.shape[0] or rec_f.shape[0] != 4 * rec_f.shape[1]:
        raise ValueError("blstm: ff_weight %s / rec_weight %s, expected [4*out,in] / [4*out,out]" % (tuple(ff_f.shape), tuple(rec_f.shape)))
    dtype = dtype or ff_f.dtype
    rec = [_to_native_gate_order(r).t().to(dtype).contiguous() for r in (rec_f, rec_b)]
    ff = torch.cat(_native_gate_blocks(ff_f.to(dtype)) + _native_gate_blocks(ff_b.to(dtype)), dim=0).t()
    bias = None
    if b_f is not None:
        if tuple(b_f.shape) != (rec_f.shape[0],) or tuple(b_b.shape) != (rec_b.shape[0],):
            raise ValueError("blstm: bias must be [4*out]")
        bias = torch.cat(_native_gate_blocks(b_f.to(dtype)) + _native_gate_blocks(b_b.to(dtype)), dim=0)
    return BlstmWeights(ff=ff, rec_fwd=rec[0], rec_bwd=rec[1], bias=bias)


def join_weights(fwd: LstmWeights, bwd: LstmWeights) -> BlstmWeights:
    """Two prepared directions -> one projection (a copy of the two projection matrices; prefer
    :func:`prepare_blstm_weights`, which gets there from the parameters in the same single copy)."""
    if fwd.ff.shape != bwd.ff.shape or fwd.rec.shape != bwd.rec.shape or (fwd.bias is None) != (bwd.bias is None):
        raise ValueError("blstm: weights of the two directions do not match each other")
    ff = torch.cat((fwd.ff.t(), bwd.ff.t()), dim=0).t()
    bias = None if fwd.bias is None else torch.cat((fwd.bias, bwd.bias), dim=0)
    return BlstmWeights(ff=ff, rec_fwd=fwd.rec, rec_bwd=bwd.rec, bias=bias)


def sequence_mask_time_major(lengths: torch.Tensor, *, maxlen: int) -> torch.Tensor:
    """[B] lengths -> [maxlen,B] float32 0/1 mask, right padded (returnn/torch/util/array_.py:196-208)."""
    idx = torch.arange(maxlen, dtype=lengths.dtype, device=lengths.device)
    return (idx[:, None] < lengths[None, :]).to(torch.float32)


def _native_lstm2():
    return make_op(native_op.NativeLstm2)


def lstm(
    source: torch.Tensor,
    *,
    state_h: torch.Tensor,
    state_c: torch.Tensor,
    ff_weight: Optional[torch.Tensor] = None,
    rec_weight: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    weights: Optional[LstmWeights] = None,
    seq_lens: Optional[torch.Tensor] = None,
    direction: int = 1,
) -> Tuple[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """
    :param source: [T,B,in] time-major, or [B,in] for a single step (``single_step_dim`` in the reference);
        float32 or bfloat16, on the GPU
    :param state_h: [B,out] initial output
    :param state_c: [B,out] initial cell
    :param ff_weight: [4*out,in], gate order input, forget, cell-in, output (PyTorch's)
    :param rec_weight: [4*out,out]
    :param bias: [4*out] or None
    :param weights: already prepared weights (:func:`prepare_weights`) instead of the three above
    :param seq_lens: [B] integer lengths (any device), None = all sequences have T frames
    :param direction: +1, or -1 for the backward-in-time layer of a bidirectional pair
    :return: output [T,B,out] (or [B,out]), (h [B,out], c [B,out]) after each sequence's last processed frame;
        output and h in the type of ``source``, c in float32
    """
    if direction not in (1, -1):
        raise ValueError("lstm: direction must be +1 or -1")
    single_step = source.dim() == 2
    if single_step:
        source = source[None]
    if source.dim() != 3:
        raise ValueError("lstm: source must be [T,B,in] or [B,in], got %s" % (tuple(source.shape),))
    if not source.is_cuda:
        raise RuntimeError("lstm: this build implements the LSTM for HIP (MI355X) tensors only; got a CPU tensor")
    act = torch.bfloat16 if source.dtype == torch.bfloat16 else torch.float32
    if weights is None:
        if ff_weight is None or rec_weight is None:
            raise ValueError("lstm: give ff_weight and rec_weight, or weights")
        weights = prepare_weights(ff_weight, rec_weight, bias, dtype=act)
    T, B, in_dim = source.shape
    n = weights.rec.shape[0]
    if weights.ff.shape[0] != in_dim:
        raise ValueError("lstm: source has %i features, ff_weight expects %i" % (in_dim, weights.ff.shape[0]))
    if tuple(state_h.shape) != (B, n) or tuple(state_c.shape) != (B, n):
        raise ValueError("lstm: state_h %s / state_c %s, expected %s" % (tuple(state_h.shape), tuple(state_c.shape), (B, n)))
    device = source.device
    X = _project(source, weights, act)
    if seq_lens is None:
        mask = torch.ones((T, B), dtype=torch.float32, device=device)
    else:
        if tuple(seq_lens.shape) != (B,):
            raise ValueError("lstm: seq_lens must be [B]=[%i], got %s" % (B, tuple(seq_lens.shape)))
        mask = sequence_mask_time_major(seq_lens.to(device), maxlen=T)
    if _wants_grad(X, weights.rec, state_h, state_c):
        _native_lstm2()
        Y, _C, _H, d = NativeLstm2Function.apply(X, weights.rec, state_h, state_c, mask, 0, direction)
        h = _last_output_autograd(Y, state_h, seq_lens, direction)
    else:
        Y, _C, _H, d = _native_lstm2()(X, weights.rec, state_h, state_c, mask, 0, direction)
        h = lstm_last_output(Y, state_h, mask, 0, direction) if T > 0 else state_h.to(act)
    if single_step:
        Y = Y[0]
    return Y, (h, d)


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _last_output_autograd(Y: torch.Tensor, y0: torch.Tensor, seq_lens: Optional[torch.Tensor], direction: int) -> torch.Tensor:
    """
    The final output per sequence with torch indexing, so that gradients flow (the library routine behind
    :func:`lstm_last_output` has no gradient).  Valid for the right-padded masks this module builds from lengths: the
    last processed valid frame is ``len-1`` going forward and frame 0 going backward; empty sequences keep ``y0``.
    """
    T, B, n = Y.shape
    if T == 0:
        return y0.to(Y.dtype)
    lens = torch.full((B,), T, dtype=torch.int64, device=Y.device) if seq_lens is None else seq_lens.to(Y.device).to(torch.int64).clamp(max=T)
    if direction > 0:
        idx = (lens - 1).clamp(min=0)
        last = Y[idx, torch.arange(B, device=Y.device)]
    else:
        last = Y[0]
    return torch.where((lens > 0)[:, None], last, y0.to(Y.dtype))


def _project(source: torch.Tensor, weights: LstmWeights, act: torch.dtype) -> torch.Tensor:
    """``X = source . ff + bias`` in the op's layout [T,B,4*out]."""
    T, B, in_dim = source.shape
    src2 = source.to(act).reshape(T * B, in_dim)
    ff = weights.ff.to(act)
    X = torch.addmm(weights.bias.to(act), src2, ff) if weights.bias is not None else torch.mm(src2, ff)
    return X.view(T, B, ff.shape[1])


def blstm(
    source: torch.Tensor,
    *,
    fwd: Optional[LstmWeights] = None,
    bwd: Optional[LstmWeights] = None,
    weights: Optional[BlstmWeights] = None,
    state_fwd: LstmState,
    state_bwd: LstmState,
    seq_lens: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, LstmState, LstmState]:
    """
    Forward-in-time and backward-in-time layer on the same input: ONE projection ``[T*B, 8*out]`` for both directions,
    then both recurrences through the library's multi-call entry (one launch when the device holds both), each reading
    its columns of the projection and writing its columns of the one output array in place.  Same results as two
    :func:`lstm` calls with ``direction=+1`` and ``-1`` and a concat.

    :param source: [T,B,in]
    :param weights: joint weights (:func:`prepare_blstm_weights`), or ``fwd`` and ``bwd`` prepared one by one (joined here,
        which copies the projection matrices)
    :return: [T,B,2*out] (forward | backward), new forward state, new backward state
    """
    if source.dim() != 3:
        raise ValueError("blstm: source must be [T,B,in], got %s" % (tuple(source.shape),))
    if not source.is_cuda:
        raise RuntimeError("blstm: this build implements the LSTM for HIP (MI355X) tensors only; got a CPU tensor")
    if weights is None:
        if fwd is None or bwd is None:
            raise ValueError("blstm: give weights, or fwd and bwd")
        weights = join_weights(fwd, bwd)
    act = torch.bfloat16 if source.dtype == torch.bfloat16 else torch.float32
    T, B, in_dim = source.shape
    n = weights.rec_fwd.shape[0]
    if weights.rec_bwd.shape[0] != n or tuple(weights.ff.shape) != (in_dim, 8 * n):
        raise ValueError("blstm: weights do not match each other or the input")
    for st in (state_fwd, state_bwd):
        if tuple(st.h.shape) != (B, n) or tuple(st.c.shape) != (B, n):
            raise ValueError("blstm: state %s / %s, expected %s" % (tuple(st.h.shape), tuple(st.c.shape), (B, n)))
    if seq_lens is None:
        mask = torch.ones((T, B), dtype=torch.float32, device=source.device)
    else:
        if tuple(seq_lens.shape) != (B,):
            raise ValueError("blstm: seq_lens must be [B]=[%i], got %s" % (B, tuple(seq_lens.shape)))
        mask = sequence_mask_time_major(seq_lens.to(source.device), maxlen=T)
    _native_lstm2()  # registers the op and fails loudly without the library
    P = _project(source, LstmWeights(ff=weights.ff, rec=weights.rec_fwd, bias=weights.bias), act)  # [T,B,8n]
    if _wants_grad(P, weights.rec_fwd, weights.rec_bwd, state_fwd.h, state_fwd.c, state_bwd.h, state_bwd.c):
        # training: both directions in one differentiable call (forward and gradient each one library entry)
        Y, df, db = NativeLstm2BidirFunction.apply(
            P, weights.rec_fwd, state_fwd.h, state_fwd.c, weights.rec_bwd, state_bwd.h, state_bwd.c, mask
        )
        hf = _last_output_autograd(Y[:, :, :n], state_fwd.h, seq_lens, 1)
        hb = _last_output_autograd(Y[:, :, n:], state_bwd.h, seq_lens, -1)
        return Y, LstmState(h=hf, c=df), LstmState(h=hb, c=db)
    ((Yf, _, _, df), (Yb, _, _, db)), Y = native_lstm2_multi(
        [
            (P[:, :, : 4 * n], weights.rec_fwd, state_fwd.h, state_fwd.c, mask, 0, 1),
            (P[:, :, 4 * n :], weights.rec_bwd, state_bwd.h, state_bwd.c, mask, 0, -1),
        ],
        joint_output=True,
    )
    if T > 0:
        hf = lstm_last_output(Yf, state_fwd.h, mask, 0, 1)
        hb = lstm_last_output(Yb, state_bwd.h, mask, 0, -1)
    else:
        hf, hb = state_fwd.h.to(act), state_bwd.h.to(act)
    return Y, LstmState(h=hf, c=df), LstmState(h=hb, c=db)


class LSTM(torch.nn.Module):
    """
    The module of returnn/frontend/rec.py:16-83 with integer dims.

    Like :class:`BLSTM`, it keeps its parameters in the layout the op takes -- ``ff [4*out, in]`` with the gate blocks in
    the order cell-in, input, forget, output (the projection uses its transposed view), ``rec [out, 4*out]``,
    ``bias [4*out]`` -- so that neither a forward nor a training step reorders or transposes anything.  The frontend's
    layout (``ff_weight [4*out,in]``, ``rec_weight [4*out,out]``, ``bias [4*out]`` in the order input, forget, cell-in,
    output; the mapping of returnn/tf/frontend_layers/_backend.py:1199-1222) is what :meth:`frontend_params`,
    :meth:`load_frontend_params`, ``state_dict()`` and ``load_state_dict()`` speak, under the frontend's parameter names.
    Initialisation as the frontend's: ``ff_weight`` and ``rec_weight`` Glorot-uniform (returnn/frontend/init.py:189-197),
    bias zero.
    """

    _FRONTEND_KEYS = ("ff_weight", "rec_weight", "bias")

    def __init__(self, in_dim: int, out_dim: int, *, with_bias: bool = True, device=None, dtype=None):
        super().__init__()
        self.in_dim = int(in_dim)
        self.out_dim = int(out_dim)
        kw = dict(device=device, dtype=dtype)
        self.ff = torch.nn.Parameter(torch.empty((4 * self.out_dim, self.in_dim), **kw))
        self.rec = torch.nn.Parameter(torch.empty((self.out_dim, 4 * self.out_dim), **kw))
        self.bias = torch.nn.Parameter(torch.zeros((4 * self.out_dim,), **kw)) if with_bias else None
        self.reset_parameters()

    def reset_parameters(self, generator: Optional[torch.Generator] = None):
        with torch.no_grad():
            for p in (self.ff, self.rec):
                limit = math.sqrt(6.0 / (p.shape[0] + p.shape[1]))  # scale 1 / fan_avg, uniform: sqrt(3*scale)
                p.uniform_(-limit, limit, generator=generator)
            if self.bias is not None:
                self.bias.zero_()

    def weights(self, act: torch.dtype) -> LstmWeights:
        """The parameters as :func:`lstm` takes them (views; a cast only when the run's type is not the parameters')."""
        return LstmWeights(ff=self.ff.to(act).t(), rec=self.rec.to(act), bias=None if self.bias is None else self.bias.to(act))

    def frontend_params(self) -> dict:
        """``{"ff_weight" [4*out,in], "rec_weight" [4*out,out], "bias" [4*out] or None}`` in the frontend's gate order
        (copies, detached)."""
        with torch.no_grad():
            return {
                "ff_weight": _from_native_gate_order(self.ff).contiguous(),
                "rec_weight": _from_native_gate_order(self.rec.t()).contiguous(),
                "bias": None if self.bias is None else _from_native_gate_order(self.bias).contiguous(),
            }

    def load_frontend_params(self, params: dict):
        """Takes the parameters in the frontend's layout (arrays or tensors)."""
        n4 = 4 * self.out_dim
        ff_w, rec_w = torch.as_tensor(params["ff_weight"]), torch.as_tensor(params["rec_weight"])
        if tuple(ff_w.shape) != (n4, self.in_dim) or tuple(rec_w.shape) != (n4, self.out_dim):
            raise ValueError("LSTM: ff_weight %s / rec_weight %s, expected %s / %s"
                             % (tuple(ff_w.shape), tuple(rec_w.shape), (n4, self.in_dim), (n4, self.out_dim)))  # fmt: skip
        b = params.get("bias")
        if (b is None) != (self.bias is None):
            raise ValueError("LSTM: the layer was built %s a bias" % ("without" if self.bias is None else "with"))
        with torch.no_grad():
            self.ff.copy_(_to_native_gate_order(ff_w))
            self.rec.copy_(_to_native_gate_order(rec_w).t())
            if b is not None:
                self.bias.copy_(_to_native_gate_order(torch.as_tensor(b)))

    # state_dict / load_state_dict in the frontend's layout, so that checkpoints do not depend on the op's layout
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        for key, value in self.frontend_params().items():
            if value is not None:
                destination[prefix + key] = value

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        keys = [k for k in self._FRONTEND_KEYS if not (k == "bias" and self.bias is None)]
        absent = [k for k in keys if prefix + k not in state_dict]
        if absent:
            if strict:
                missing_keys.extend(prefix + k for k in absent)
            return
        try:
            self.load_frontend_params({k: state_dict.get(prefix + k) for k in self._FRONTEND_KEYS})
        except (ValueError, RuntimeError) as exc:
            error_msgs.append(str(exc))
        if strict:
            unexpected_keys.extend(k for k in state_dict if k.startswith(prefix) and k[len(prefix) :] not in keys)

    def forward(
        self, source: torch.Tensor, *, state: LstmState, seq_lens: Optional[torch.Tensor] = None, direction: int = 1
    ) -> Tuple[torch.Tensor, LstmState]:
        """
        :param source: [T,B,in], or [B,in] for a single step
        :param state: h and c, [B,out]
        :param seq_lens: [B] or None
        :return: output [T,B,out] (or [B,out]), new state
        """
        if state.h is None or state.c is None:
            raise ValueError("%s: state %r needs attributes ``h`` (hidden) and ``c`` (cell)." % (self, state))
        if source.shape[-1] != self.in_dim:
            raise ValueError("%s: input %s does not have in_dim %i" % (self, tuple(source.shape), self.in_dim))
        act = torch.bfloat16 if source.dtype == torch.bfloat16 else torch.float32
        out, (h, c) = lstm(
            source, state_h=state.h, state_c=state.c, weights=self.weights(act), seq_lens=seq_lens, direction=direction
        )
        return out, LstmState(h=h, c=c)

    def default_initial_state(self, *, batch_dims: Sequence[int], device=None) -> LstmState:
        """zeros (returnn/frontend/rec.py:78-83); h in the parameters' type, c in float32"""
        device = device or self.rec.device
        shape = tuple(batch_dims) + (self.out_dim,)
        return LstmState(
            h=torch.zeros(shape, dtype=self.rec.dtype, device=device),
            c=torch.zeros(shape, dtype=torch.float32, device=device),
        )

    def extra_repr(self) -> str:
        return "in_dim=%i, out_dim=%i, with_bias=%s" % (self.in_dim, self.out_dim, self.bias is not None)


def _from_native_gate_order(w: torch.Tensor) -> torch.Tensor:
    """[4*out, ...] in (cell-in, input, forget, output) blocks -> (input, forget, cell-in, output)."""
    g, i, f, o = w.chunk(4, dim=0)
    return torch.cat((i, f, g, o), dim=0)


class BLSTM(torch.nn.Module):
    """
    One bidirectional LSTM layer: a forward-in-time and a backward-in-time recurrence on the same input, outputs side by
    side (``2*out_dim`` features).

    The parameters live in the layout the op takes -- ``ff [8*out, in]`` (rows: the forward direction's gates cell-in,
    input, forget, output, then the backward direction's; the projection uses its transposed view), ``rec_fwd`` /
    ``rec_bwd [out, 4*out]``, ``bias [8*out]`` -- so that neither a forward nor a training step reorders or joins
    anything.  The frontend's layout (returnn/frontend/rec.py:46-77: per direction ``ff_weight [4*out,in]``,
    ``rec_weight [4*out,out]``, ``bias [4*out]`` in the order input, forget, cell-in, output; the mapping of
    returnn/tf/frontend_layers/_backend.py:1199-1222) is what :meth:`frontend_params`, :meth:`load_frontend_params`,
    ``state_dict()`` and ``load_state_dict()`` speak (keys ``fwd.ff_weight``, ``fwd.rec_weight``, ``fwd.bias``, ``bwd. ...``).
    Initialisation as the frontend's: every direction's ``ff_weight`` and ``rec_weight`` Glorot-uniform
    (returnn/frontend/init.py:189-197), biases zero.
    """

    _FRONTEND_KEYS = ("ff_weight", "rec_weight", "bias")

    def __init__(self, in_dim: int, out_dim: int, *, with_bias: bool = True, device=None, dtype=None):
        super().__init__()
        self.in_dim, self.out_dim = int(in_dim), int(out_dim)
        kw = dict(device=device, dtype=dtype)
        n = self.out_dim
        self.ff = torch.nn.Parameter(torch.empty((8 * n, self.in_dim), **kw))
        self.rec_fwd = torch.nn.Parameter(torch.empty((n, 4 * n), **kw))
        self.rec_bwd = torch.nn.Parameter(torch.empty((n, 4 * n), **kw))
        self.bias = torch.nn.Parameter(torch.zeros((8 * n,), **kw)) if with_bias else None
        self.reset_parameters()

    def reset_parameters(self, generator: Optional[torch.Generator] = None):
        n = self.out_dim
        with torch.no_grad():
            self.ff.uniform_(-math.sqrt(6.0 / (4 * n + self.in_dim)), math.sqrt(6.0 / (4 * n + self.in_dim)), generator=generator)
            for p in (self.rec_fwd, self.rec_bwd):
                p.uniform_(-math.sqrt(6.0 / (5 * n)), math.sqrt(6.0 / (5 * n)), generator=generator)
            if self.bias is not None:
                self.bias.zero_()

    def weights(self, act: torch.dtype) -> BlstmWeights:
        """The parameters as :func:`blstm` takes them (views; a cast only when the run's type is not the parameters')."""
        return BlstmWeights(
            ff=self.ff.to(act).t(), rec_fwd=self.rec_fwd.to(act), rec_bwd=self.rec_bwd.to(act),
            bias=None if self.bias is None else self.bias.to(act),
        )  # fmt: skip

    def frontend_params(self) -> dict:
        """``{"fwd": p, "bwd": p}`` with ``p = {"ff_weight" [4*out,in], "rec_weight" [4*out,out], "bias" [4*out] or None}`` in the
        frontend's gate order (copies, detached)."""
        n4 = 4 * self.out_dim
        out = {}
        with torch.no_grad():
            for k, (name, rec) in enumerate((("fwd", self.rec_fwd), ("bwd", self.rec_bwd))):
                out[name] = {
                    "ff_weight": _from_native_gate_order(self.ff[k * n4 : (k + 1) * n4]).contiguous(),
                    "rec_weight": _from_native_gate_order(rec.t()).contiguous(),
                    "bias": None if self.bias is None else _from_native_gate_order(self.bias[k * n4 : (k + 1) * n4]).contiguous(),
                }
        return out

    def load_frontend_params(self, fwd: dict, bwd: dict):
        """Takes the two directions' parameters in the frontend's layout (arrays or tensors)."""
        n4 = 4 * self.out_dim
        with torch.no_grad():
            for k, (p, rec) in enumerate(((fwd, self.rec_fwd), (bwd, self.rec_bwd))):
                ff_w, rec_w = torch.as_tensor(p["ff_weight"]), torch.as_tensor(p["rec_weight"])
                if tuple(ff_w.shape) != (n4, self.in_dim) or tuple(rec_w.shape) != (n4, self.out_dim):
                    raise ValueError("BLSTM: ff_weight %s / rec_weight %s, expected %s / %s"
                                     % (tuple(ff_w.shape), tuple(rec_w.shape), (n4, self.in_dim), (n4, self.out_dim)))  # fmt: skip
                self.ff[k * n4 : (k + 1) * n4].copy_(_to_native_gate_order(ff_w))
                rec.copy_(_to_native_gate_order(rec_w).t())
                b = p.get("bias")
                if (b is None) != (self.bias is None):
                    raise ValueError("BLSTM: the layer was built %s a bias" % ("without" if self.bias is None else "with"))
                if b is not None:
                    self.bias[k * n4 : (k + 1) * n4].copy_(_to_native_gate_order(torch.as_tensor(b)))

    # state_dict / load_state_dict in the frontend's layout, so that checkpoints do not depend on the op's layout
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        for name, p in self.frontend_params().items():
            for key in self._FRONTEND_KEYS:
                if p[key] is not None:
                    destination[prefix + name + "." + key] = p[key]

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        keys = [n + "." + k for n in ("fwd", "bwd") for k in self._FRONTEND_KEYS if not (k == "bias" and self.bias is None)]
        absent = [k for k in keys if prefix + k not in state_dict]
        if absent:
            if strict:
                missing_keys.extend(prefix + k for k in absent)
            return
        try:
            parts = {n: {k: state_dict.get(prefix + n + "." + k) for k in self._FRONTEND_KEYS} for n in ("fwd", "bwd")}
            self.load_frontend_params(parts["fwd"], parts["bwd"])
        except (ValueError, RuntimeError) as exc:
            error_msgs.append(str(exc))
        if strict:
            unexpected_keys.extend(k for k in state_dict if k.startswith(prefix) and k[len(prefix) :] not in keys)

    def default_initial_state(self, *, batch_dims: Sequence[int], device=None, dtype=None) -> LstmState:
        """zeros for one direction (returnn/frontend/rec.py:78-83); h in the parameters' type (or ``dtype``), c in float32"""
        shape = tuple(batch_dims) + (self.out_dim,)
        device = device or self.ff.device
        return LstmState(h=torch.zeros(shape, dtype=dtype or self.ff.dtype, device=device), c=torch.zeros(shape, dtype=torch.float32, device=device))

    def forward(
        self, source: torch.Tensor, *, state_fwd: Optional[LstmState] = None, state_bwd: Optional[LstmState] = None,
        seq_lens: Optional[torch.Tensor] = None,
    ) -> Tuple[torch.Tensor, LstmState, LstmState]:  # fmt: skip
        """
        :param source: [T,B,in]
        :param state_fwd, state_bwd: initial states, default zeros
        :return: [T,B,2*out_dim] (forward | backward), new forward state, new backward state
        """
        if source.dim() != 3 or source.shape[-1] != self.in_dim:
            raise ValueError("%s: input %s is not [T,B,%i]" % (self, tuple(source.shape), self.in_dim))
        act = torch.bfloat16 if source.dtype == torch.bfloat16 else torch.float32
        zero = None
        if state_fwd is None or state_bwd is None:
            zero = self.default_initial_state(batch_dims=(source.shape[1],), device=source.device, dtype=act)
        return blstm(source, weights=self.weights(act), state_fwd=state_fwd or zero, state_bwd=state_bwd or zero, seq_lens=seq_lens)

    def extra_repr(self) -> str:
        return "in_dim=%i, out_dim=%i, with_bias=%s" % (self.in_dim, self.out_dim, self.bias is not None)


class BlstmEncoder(torch.nn.Module):
    """
    Stack of bidirectional LSTM layers (:class:`BLSTM`): per layer a forward-in-time and a backward-in-time recurrence on
    the same input, outputs side by side (``2*out_dim`` features), which feed the next layer.  All layers use the same
    sequence lengths; states start at zero.
    """

    def __init__(self, in_dim: int, out_dim: int, num_layers: int, *, with_bias: bool = True, device=None, dtype=None):
        super().__init__()
        self.in_dim, self.out_dim, self.num_layers = int(in_dim), int(out_dim), int(num_layers)
        self.layers = torch.nn.ModuleList(
            BLSTM(self.in_dim if layer == 0 else 2 * self.out_dim, self.out_dim, with_bias=with_bias, device=device, dtype=dtype)
            for layer in range(self.num_layers)
        )

    def reset_parameters(self, generator: Optional[torch.Generator] = None):
        for m in self.layers:
            m.reset_parameters(generator)

    @classmethod
    def from_params(cls, layers, *, device=None, dtype=None) -> "BlstmEncoder":
        """
        :param layers: per layer ``{"fwd": p, "bwd": p}`` with ``p = {"ff_weight" [4n,in], "rec_weight" [4n,n], "bias" [4n] or None}``
            (arrays or tensors, frontend layout)
        """
        first = layers[0]["fwd"]
        n = first["rec_weight"].shape[1]
        with_bias = first.get("bias") is not None
        enc = cls(first["ff_weight"].shape[1], n, len(layers), with_bias=with_bias, device=device, dtype=dtype)
        for params, layer in zip(layers, enc.layers):
            layer.load_frontend_params(params["fwd"], params["bwd"])
        return enc

    def forward(
        self, source: torch.Tensor, *, seq_lens: Optional[torch.Tensor] = None, collect_states: bool = False
    ) -> Union[torch.Tensor, Tuple[torch.Tensor, list]]:
        """
        :param source: [T,B,in]
        :param seq_lens: [B] or None
        :param collect_states: also return per layer ``(LstmState fwd, LstmState bwd)``
        :return: [T,B,2*out_dim]
        """
        x = source
        states = []
        for layer in self.layers:
            x, sf, sb = layer(x, seq_lens=seq_lens)
            states.append((sf, sb))
        return (x, states) if collect_states else x
