"""
MI355X-native forward pass of RETURNN's ``NativeLstm2`` operator.

* :mod:`returnn_amd.native_op` -- the operator description (the contract of ``returnn.native_op.NativeLstm2``)
* :mod:`returnn_amd.torch_native_op` -- ``make_op``: the operator as a ``torch.ops`` entry on HIP tensors
* :mod:`returnn_amd.lstm` -- the LSTM layer on top of the op (counterpart of the frontend's LSTM module and backend function)
* :mod:`returnn_amd.lib` -- ctypes binding of the C ABI in ``include/rtn_native_lstm2.h``
* :mod:`returnn_amd.build` -- hipcc build of the library for gfx950
* :mod:`returnn_amd.synthetic` -- seeded inputs of the benchmark configurations
"""

__version__ = "0.1"
