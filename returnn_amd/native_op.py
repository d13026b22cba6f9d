"""
Operator descriptions: the backend-neutral contract of a native op.

Mirrors the role of ``returnn.native_op`` (``NativeOpGenBase`` returnn/native_op.py:300-330,
``OpDescription`` :254-297, shape inference :138-163) for the operators this package
implements (``NativeLstm2`` and, forward only, its siblings ``LstmGenericBase`` and ``LstmLowMem``).  The reference's description classes carry C code strings that a generator compiles at
run time; here a description names the entry point of the prebuilt gfx950 library instead.
"""

from __future__ import annotations

from typing import Any, Dict, List, Optional, Sequence, Tuple


class NativeOpGenBase:
    """Base interface of an op description (class attributes only, as in the reference)."""

    in_info: Optional[Tuple[Dict[str, Any], ...]] = None
    out_info: Optional[Tuple[Dict[str, Any], ...]] = None
    c_abi_fw: Optional[str] = None  # forward entry point in librtn_native_lstm2.so
    c_abi_bw: Optional[str] = None  # gradient entry point, if any
    grad_input_map = None
    cpu_support = False  # HIP only: no CPU implementation is shipped

    @classmethod
    def map_layer_inputs_to_op(cls, *inputs):
        return inputs

    @classmethod
    def map_layer_output_from_op(cls, *outputs):
        return outputs[0]


class OpDescription:
    """Meta-info about an op, consumed by :class:`returnn_amd.torch_native_op.OpMaker`."""

    def __init__(
        self,
        in_info: Sequence[Dict[str, Any]],
        out_info: Sequence[Dict[str, Any]],
        c_abi_fw: str,
        c_abi_bw: Optional[str] = None,
        cpu_support: bool = False,
        grad_input_map=None,
        name: Optional[str] = None,
    ):
        self.in_info = tuple(dict(v) for v in in_info)
        self.out_info = tuple(dict(v) for v in out_info)
        self.c_abi_fw = c_abi_fw
        self.c_abi_bw = c_abi_bw
        self.cpu_support = cpu_support
        self.grad_input_map = grad_input_map
        self.name = name or "UnnamedOp"
        for v in self.in_info + self.out_info:
            assert v["ndim"] == len(v["shape"]), "ndim/shape mismatch in %r" % (v,)

    @classmethod
    def from_gen_base(cls, gen_base) -> "OpDescription":
        """:param type[NativeOpGenBase] gen_base: description class, e.g. :class:`NativeLstm2`"""
        assert gen_base.in_info is not None and gen_base.out_info is not None and gen_base.c_abi_fw
        return cls(
            in_info=gen_base.in_info,
            out_info=gen_base.out_info,
            c_abi_fw=gen_base.c_abi_fw,
            c_abi_bw=gen_base.c_abi_bw,
            cpu_support=gen_base.cpu_support,
            grad_input_map=gen_base.grad_input_map,
            name=gen_base.__name__,
        )

    @property
    def is_grad_defined(self) -> bool:
        return bool(self.c_abi_bw)

    def infer_shape(self, node, input_shapes: Sequence[Sequence[int]]) -> List[Tuple[int, ...]]:
        """Output shapes from input shapes: an out_info dim is an int or an ``(in_idx, dim)`` reference."""
        del node
        if len(input_shapes) != len(self.in_info):
            raise ValueError("%s: expected %i input shapes, got %i" % (self.name, len(self.in_info), len(input_shapes)))
        out_shapes = []
        for info in self.out_info:
            shape = []
            for s in info["shape"]:
                if isinstance(s, tuple):
                    in_idx, dim = s
                    if not (0 <= in_idx < len(input_shapes)) or not (0 <= dim < self.in_info[in_idx]["ndim"]):
                        raise ValueError("%s: bad dim reference %r in %r" % (self.name, s, info))
                    shape.append(input_shapes[in_idx][dim])
                else:
                    shape.append(s)
            if any(s is None for s in shape):
                raise ValueError("%s: cannot infer %r from %r" % (self.name, info, input_shapes))
            out_shapes.append(tuple(shape))
        return out_shapes


class NativeLstm2(NativeOpGenBase):
    """
    LSTM over a whole (time-major) batch with the input projection done outside.
    Contract of ``returnn.native_op.NativeLstm2`` (returnn/native_op.py:1029-1077):

    inputs:
      :param X: (time,batch,dim*4) gate pre-activations from the input; last axis = cell-in, input, forget, output
      :param W: recurrent matrix (dim,dim*4)
      :param y0: initial output (batch,dim)
      :param c0: initial cell state (batch,dim)
      :param i: (time,batch) 0/1 mask
      :param start: host int, first frame, >= 0. For step < 0 counted from the end (starts at T-start-1).
      :param step: host int, +1 forward, -1 backward, \\|step\\|>1 for wider strides
    outputs:
      :param Y: (time,batch,dim), zero on masked frames
      :param C: (time,batch,dim) cell states
      :param H: (time,batch,dim*4) activated cell-in and gates
      :param d: (batch,dim) final cell state
    """

    in_info = (
        {"name": "X", "ndim": 3, "shape": (None, None, None), "need_contiguous": True},
        {"name": "W", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "y0", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "c0", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "i", "ndim": 2, "shape": (None, None), "need_contiguous": True, "gradient": "disconnected"},
        {"name": "start", "ndim": 0, "shape": (), "gradient": "disconnected", "dtype": "int32", "host_memory": True},
        {"name": "step", "ndim": 0, "shape": (), "gradient": "disconnected", "dtype": "int32", "host_memory": True},
    )
    out_info = (
        {"name": "Y", "ndim": 3, "shape": ((0, 0), (0, 1), (1, 0)), "need_contiguous": True},
        {"name": "C", "ndim": 3, "shape": ((0, 0), (0, 1), (1, 0)), "need_contiguous": True},
        {"name": "H", "ndim": 3, "shape": ((0, 0), (0, 1), (1, 1)), "need_contiguous": True},
        {"name": "d", "ndim": 2, "shape": ((0, 1), (1, 0)), "need_contiguous": True},
    )
    c_abi_fw = "rtn_native_lstm2_fwd"
    c_abi_bw = "rtn_native_lstm2_bwd"

    # noinspection PyPep8Naming
    @classmethod
    def grad_input_map(cls, X, W, y0, c0, i, start, step, Y, C, H, d, DY, DC, DH, Dd):
        """What the gradient op consumes (returnn/native_op.py:1071-1077)."""
        del d, DC, DH
        return X, W, y0, c0, i, start, step, Y, C, H, DY, Dd


class LstmGenericBase(NativeOpGenBase):
    """
    Contract of ``returnn.native_op.LstmGenericBase`` (returnn/native_op.py:333-378), forward pass:

    inputs:
      :param Z: (time,batch,dim*4) gate inputs; last axis = cell-in, input, forget, output
      :param V_h: recurrent matrix (dim,dim*4)
      :param c: initial cell state (batch,dim)
      :param i: (time,batch) 0/1 mask
    outputs:
      :param Y: (time,batch,dim)
      :param H: (time,batch,dim*4) cell state, then the activated input, forget and output gates
      :param d: (batch,dim) final cell state

    The reference computes H in place of Z; here H is a new array.  The recurrent input of a frame is the output of
    the frame before (zero where that was masked), there is no initial output.
    """

    in_info = (
        {"name": "Z", "ndim": 3, "shape": (None, None, None), "need_contiguous": True},
        {"name": "V_h", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "c", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "i", "ndim": 2, "shape": (None, None), "need_contiguous": True, "gradient": "disconnected"},
    )
    out_info = (
        {"name": "Y", "ndim": 3, "shape": ((0, 0), (0, 1), (1, 0)), "need_contiguous": True},
        {"name": "H", "ndim": 3, "shape": ((0, 0), (0, 1), (0, 2)), "need_contiguous": True},
        {"name": "d", "ndim": 2, "shape": ((2, 0), (2, 1)), "need_contiguous": True},
    )
    c_abi_fw = "rtn_lstm_generic_base_fwd"
    c_abi_bw = "rtn_lstm_generic_base_bwd"

    # noinspection PyPep8Naming
    @classmethod
    def grad_input_map(cls, Z, V_h, c, i, Y, H, d, DY, DH, Dd):
        """What the gradient op consumes (returnn/native_op.py:374-378)."""
        del Z, d, DH
        return V_h, c, i, Y, H, DY, Dd


class LstmLowMem(NativeOpGenBase):
    """
    Contract of ``returnn.native_op.LstmLowMem`` (returnn/native_op.py:577-615), forward pass:

    inputs:
      :param X: (time,batch,in_dim) raw input
      :param W: input weights stacked on recurrent weights (in_dim+dim,dim*4)
      :param b: bias (dim*4,)
      :param y0: initial output (batch,dim)
      :param c0: initial cell state (batch,dim)
      :param i: (time,batch) 0/1 mask
      :param start, step: host ints as for :class:`NativeLstm2`
    outputs:
      :param Y: (time,batch,dim)
      :param C: (time,batch,dim) cell states
      :param d: (batch,dim) final cell state
    """

    in_info = (
        {"name": "X", "ndim": 3, "shape": (None, None, None), "need_contiguous": True},
        {"name": "W", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "b", "ndim": 1, "shape": (None,), "need_contiguous": True},
        {"name": "y0", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "c0", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "i", "ndim": 2, "shape": (None, None), "need_contiguous": True, "gradient": "disconnected"},
        {"name": "start", "ndim": 0, "shape": (), "gradient": "disconnected", "dtype": "int32", "host_memory": True},
        {"name": "step", "ndim": 0, "shape": (), "gradient": "disconnected", "dtype": "int32", "host_memory": True},
    )
    out_info = (
        {"name": "Y", "ndim": 3, "shape": ((0, 0), (0, 1), (4, 1)), "need_contiguous": True},
        {"name": "C", "ndim": 3, "shape": ((0, 0), (0, 1), (4, 1)), "need_contiguous": True},
        {"name": "d", "ndim": 2, "shape": ((0, 1), (4, 1)), "need_contiguous": True},
    )
    c_abi_fw = "rtn_lstm_low_mem_fwd"
