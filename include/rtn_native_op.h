/*
 * C ABI of an op compiled by the HIP op loader (returnn_amd/op_loader.py) from a description in RETURNN's native-op
 * source dialect: `c_fw_code` / `c_extra_support_code` strings as the classes of returnn/native_op.py carry them.
 *
 * The reference compiles such a description into a C++ translation unit that includes returnn/native_op.cpp and
 * registers a torch op whose arguments are torch::Tensor (returnn/torch/util/native_op.py:86-383, compiled by
 * returnn/torch/util/native_op_code_compiler.py with nvcc).  Here the unit is compiled by hipcc for gfx950 against
 * returnn_amd/csrc/rtn_op_dialect.h and exports plain C entry points: arrays are (pointer, dims) pairs, the stream and
 * the allocator for the op's temporaries come from the caller.  This is the shape the reference itself uses where the
 * host framework hands over raw buffers (struct NdarrayJax, returnn/native_op.cpp:683-687).
 *
 * For an op named NAME the shared object exports
 *
 *   int NAME_fw(const rtn_op_host* host, int32_t n_inputs, rtn_ndarray* inputs, int32_t n_outputs, rtn_ndarray* outputs);
 *   const char* NAME_last_error(void);
 *   int32_t NAME_abi_version(void);            (RTN_NATIVE_OP_ABI_VERSION of the loader that built it)
 *
 * NAME_fw runs the op's forward code (role of the generated NAME_cuda function, returnn/torch/util/native_op.py:342-358):
 * `inputs` in the order of the description's in_info, `outputs` in the order of out_info (after dummy outputs for
 * want_inplace="dummy_out" were appended, returnn/native_op.py:61-78).  Outputs are allocated by the caller: zeroed
 * (the reference creates them with torch::zeros, :181-184) or, for an input with want_inplace, the input's own buffer
 * (:131-142).  All arrays are contiguous row-major.  The call only enqueues work on host->stream.  Returns 0, or 1
 * after a failed check in the op code (assert_cmp, CHECK_WITH_MSG, HANDLE_LAST_ERROR, a rocBLAS or allocation
 * failure), with the message in NAME_last_error() (thread-local).
 */
#ifndef RTN_NATIVE_OP_H
#define RTN_NATIVE_OP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RTN_NATIVE_OP_ABI_VERSION 1

/* One array argument.  Stands in for `Ndarray` = torch::Tensor of the reference's torch build
 * (returnn/native_op.cpp:646-658). */
typedef struct rtn_ndarray {
  void* data;          /* device pointer; host pointer when on_host != 0 */
  const int64_t* dims; /* host array of ndim sizes (Ndarray_DIMS) */
  int32_t ndim;        /* Ndarray_NDIM */
  int32_t elem_size;   /* bytes per element (Ndarray_dtype_size): 4 for float32 and int32 */
  int32_t on_host;     /* 1 for the ndim-0 "host_memory" scalars of in_info (read with Ndarray_DEV_DATA_int32_scalar) */
  int32_t reserved;
} rtn_ndarray;

/* What the host framework lends the op for the duration of one call. */
typedef struct rtn_op_host {
  void* stream; /* hipStream_t all work is enqueued on (CUDA_CUR_STREAM, returnn/native_op.cpp:745) */
  /* device_malloc / device_free (returnn/native_op.cpp:954-956 use the framework's caching allocator).  May be null:
   * then hipMallocAsync / hipFreeAsync on `stream`.  A block is released only after the work enqueued so far on
   * `stream` may still use it, so `release` must be stream-ordered (a caching allocator keyed by stream is). */
  void* (*alloc)(size_t bytes, void* user);
  void (*release)(void* ptr, void* user);
  void* user;
} rtn_op_host;

typedef int (*rtn_native_op_fw_fn)(const rtn_op_host* host, int32_t n_inputs, rtn_ndarray* inputs, int32_t n_outputs,
                                   rtn_ndarray* outputs);

#ifdef __cplusplus
}
#endif
#endif /* RTN_NATIVE_OP_H */
