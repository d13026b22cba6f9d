"""
MI355X-native ``NativeLstm2`` operator of RETURNN: forward pass, gradient op, the sibling LSTM ops, and a loader for
ops given as source in RETURNN's native-op dialect.

* :mod:`returnn_amd.native_op` -- the operator descriptions (the contract of ``returnn.native_op.NativeLstm2``,
  ``LstmGenericBase``, ``LstmLowMem``)
* :mod:`returnn_amd.torch_native_op` -- ``make_op``: an operator as a ``torch.ops`` entry on HIP tensors; the gradient ops
  and ``torch.autograd`` functions (``NativeLstm2Function``, ``NativeLstm2PairFunction``, ``NativeLstm2BidirFunction``, ``LstmGenericBaseFunction``)
* :mod:`returnn_amd.op_loader` -- compiles an op written in the native-op source dialect with hipcc for gfx950
* :mod:`returnn_amd.lstm` -- the LSTM layer on top of the op (counterpart of the frontend's LSTM module and backend function)
* :mod:`returnn_amd.lib` -- ctypes binding of the C ABI in ``include/rtn_native_lstm2.h``
* :mod:`returnn_amd.build` -- hipcc build of the library for gfx950
* :mod:`returnn_amd.synthetic` -- seeded inputs of the benchmark configurations
"""

__version__ = "0.1"
