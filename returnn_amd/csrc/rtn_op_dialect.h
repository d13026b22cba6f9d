// The source dialect of RETURNN's native ops, for hipcc / gfx950.
//
// An op description (returnn/native_op.py) carries its forward code and support code as C++ strings written against a
// small vocabulary: `Ndarray` and its accessors, `DEF_KERNEL` / `start_dev_kernel`, `device_malloc`, `affine_raw`,
// `HANDLE_LAST_ERROR` ...  The reference defines that vocabulary in returnn/native_op.cpp, once per host framework and
// once more for CUDA.  This header defines it for one target only: HIP on gfx950, with arrays handed over as plain
// (pointer, dims) records (include/rtn_native_op.h) and the stream and allocator lent by the caller.  The translation
// unit the op loader generates includes this header, then the op's support code, then wraps the op's forward code in
// an extern "C" function.
//
// Differences to the reference's CUDA build that op code can observe:
//  * failed checks (assert, assert_cmp, CHECK_WITH_MSG, HANDLE_ERROR) in host code throw rtn_op::Error, which the
//    generated entry point turns into an error code and message; they do not abort the process;
//  * Ndarray_sgemm works (rocBLAS); the reference's torch build leaves it unimplemented
//    (returnn/native_op.cpp:665-676), which is why its LSTM ops cannot run there;
//  * Ndarray_memset is a fill kernel, so that an op stays recordable into a HIP graph.
#pragma once

#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>

#include <assert.h>
#include <stdint.h>
#include <string.h>

#include <cmath>
#include <fstream>
#include <iostream>
#include <limits>
#include <sstream>
#include <stdexcept>
#include <string>
#include <typeinfo>
#include <utility>
#include <vector>

#include "rtn_native_op.h"

// Which build the op code is in (tests of the kind `#if RETURNN_CUDA` / `#if TENSORFLOW` in op sources,
// e.g. returnn/native_op.py:3699-3706, :3731).  "CUDA" here means "the device build".
#define TENSORFLOW 0
#define TORCH 0
#define JAX 0
#define CUDA 1
#define RETURNN_CUDA 1
#define RETURNN_HIP 1
#define _ns
// Op sources guard device-only statements (__syncthreads in kernels that also run in the CPU emulation) with
// `#ifdef __CUDA_ARCH__` (returnn/native_op.py:3383-3423); on the device pass of hipcc that guard must hold.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__CUDA_ARCH__)
#define __CUDA_ARCH__ 950
#endif

#define ARRAY_LEN(x) (sizeof(x) / sizeof(x[0]))
#define DEF_KERNEL __global__
#define DEV_FUNC __device__
#define HOST_FUNC __host__
#define DEF_SHARED(type, name) extern __shared__ type name[];
#define DIM_GRID 128
#define DIM_BLOCK 512

namespace rtn_op {

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// State of the call in progress on this thread (set by the generated entry point).
struct Call {
  const rtn_op_host* host = nullptr;
  hipStream_t stream = nullptr;
  std::vector<void*> blocks;  // device_malloc'ed and not yet freed: released if the op code throws
};

inline Call*& current_slot() {
  static thread_local Call* c = nullptr;
  return c;
}

inline Call& current() {
  Call* c = current_slot();
  if (!c) throw Error("NativeOp: no call in progress on this thread");
  return *c;
}

inline void message_parts(std::ostringstream&) {}
template <typename T, typename... Rest>
inline void message_parts(std::ostringstream& os, const T& v, const Rest&... rest) {
  os << v;
  message_parts(os, rest...);
}

template <typename... Args>
[[noreturn]] inline void fail(const Args&... args) {
  std::ostringstream os;
  message_parts(os, args...);
  throw Error(os.str());
}

// Host code: throw.  Device code: print and trap, as a device-side assert does.
template <typename A, typename B>
__host__ __device__ inline void fail_cmp(const char* a, const char* cmp, const char* b, const A& va, const B& vb, int line) {
#if defined(__HIP_DEVICE_COMPILE__)
  (void)va;
  (void)vb;
  printf("NativeOp assertion failed: %s %s %s (line %d)\n", a, cmp, b, line);
  abort();
#else
  fail("NativeOp assertion failed: ", a, " ", cmp, " ", b, ", ", va, " ", cmp, " ", vb, " (line ", line, ")");
#endif
}

__host__ __device__ inline void fail_assert(const char* cond, int line) {
#if defined(__HIP_DEVICE_COMPILE__)
  printf("NativeOp assertion failed: %s (line %d)\n", cond, line);
  abort();
#else
  fail("NativeOp assertion failed: ", cond, " (line ", line, ")");
#endif
}

inline void check_hip(hipError_t err, const char* file, int line) {
  if (err != hipSuccess) fail("NativeOp: HIP runtime error: ", hipGetErrorString(err), " in ", file, " at line ", line);
}

inline void* allocate(size_t bytes) {
  Call& c = current();
  void* p = nullptr;
  if (bytes == 0) bytes = 1;
  if (c.host->alloc) {
    p = c.host->alloc(bytes, c.host->user);
  } else {
    check_hip(hipMallocAsync(&p, bytes, c.stream), __FILE__, __LINE__);
  }
  if (!p) fail("NativeOp: cannot allocate ", bytes, " bytes of device memory");
  c.blocks.push_back(p);
  return p;
}

inline void release(void* p) {
  if (!p) return;
  Call& c = current();
  for (size_t k = c.blocks.size(); k-- > 0;) {
    if (c.blocks[k] == p) {
      c.blocks.erase(c.blocks.begin() + (long)k);
      break;
    }
  }
  if (c.host->release) {
    c.host->release(p, c.host->user);
  } else {
    check_hip(hipFreeAsync(p, c.stream), __FILE__, __LINE__);
  }
}

// Entered by the generated entry point around the op code.
struct CallScope {
  Call call;
  Call* outer;
  explicit CallScope(const rtn_op_host* host) {
    call.host = host;
    call.stream = (hipStream_t)host->stream;
    outer = current_slot();
    current_slot() = &call;
  }
  ~CallScope() {
    // only non-empty when the op code threw between device_malloc and device_free
    while (!call.blocks.empty()) {
      void* p = call.blocks.back();
      call.blocks.pop_back();
      if (call.host->release)
        call.host->release(p, call.host->user);
      else
        (void)hipFreeAsync(p, call.stream);
    }
    current_slot() = outer;
  }
  CallScope(const CallScope&) = delete;
  CallScope& operator=(const CallScope&) = delete;
};

inline std::string& last_error() {
  static thread_local std::string s;
  return s;
}

__global__ static void k_fill_words(uint32_t* dst, uint32_t word, size_t n) {
  for (size_t k = blockIdx.x * (size_t)blockDim.x + threadIdx.x; k < n; k += (size_t)gridDim.x * blockDim.x) dst[k] = word;
}

__global__ static void k_fill_bytes(unsigned char* dst, unsigned char byte, size_t n) {
  for (size_t k = blockIdx.x * (size_t)blockDim.x + threadIdx.x; k < n; k += (size_t)gridDim.x * blockDim.x) dst[k] = byte;
}

inline void fill(void* dst, int value, size_t bytes) {
  if (bytes == 0) return;
  hipStream_t stream = current().stream;
  const unsigned char b = (unsigned char)value;
  if (((uintptr_t)dst % 4) == 0 && (bytes % 4) == 0) {
    const size_t n = bytes / 4;
    const unsigned grid = (unsigned)std::min<size_t>((n + 255) / 256, 4096);
    k_fill_words<<<dim3(grid), dim3(256), 0, stream>>>((uint32_t*)dst, 0x01010101u * b, n);
  } else {
    const unsigned grid = (unsigned)std::min<size_t>((bytes + 255) / 256, 4096);
    k_fill_bytes<<<dim3(grid), dim3(256), 0, stream>>>((unsigned char*)dst, b, bytes);
  }
  check_hip(hipGetLastError(), __FILE__, __LINE__);
}

inline int32_t scalar_int32(const rtn_ndarray* x) {
  if (x->ndim != 0) fail("NativeOp: scalar expected, got an array of ", x->ndim, " dimensions");
  if (x->on_host) return *(const int32_t*)x->data;
  int32_t v = 0;  // a device scalar: fetch it, as Tensor::item() does in the reference (returnn/native_op.cpp:650)
  hipStream_t stream = current().stream;
  check_hip(hipMemcpyAsync(&v, x->data, sizeof(v), hipMemcpyDeviceToHost, stream), __FILE__, __LINE__);
  check_hip(hipStreamSynchronize(stream), __FILE__, __LINE__);
  return v;
}

inline int64_t count(const rtn_ndarray* x) {
  int64_t n = 1;
  for (int k = 0; k < x->ndim; ++k) n *= x->dims[k];
  return n;
}

inline int64_t stride(const rtn_ndarray* x, int dim) {
  int64_t s = 1;
  for (int k = dim + 1; k < x->ndim; ++k) s *= x->dims[k];
  return s;
}

// One rocBLAS handle per thread and device, created at the first GEMM of an op in this shared object.
inline rocblas_handle blas() {
  struct PerDevice {
    int device;
    rocblas_handle handle;
  };
  static thread_local std::vector<PerDevice> handles;
  int device = 0;
  check_hip(hipGetDevice(&device), __FILE__, __LINE__);
  for (const PerDevice& h : handles)
    if (h.device == device) return h.handle;
  rocblas_handle handle = nullptr;
  if (rocblas_create_handle(&handle) != rocblas_status_success) fail("NativeOp: rocblas_create_handle failed");
  if (rocblas_set_pointer_mode(handle, rocblas_pointer_mode_host) != rocblas_status_success) fail("NativeOp: rocblas_set_pointer_mode failed");
  handles.push_back({device, handle});
  return handle;
}

inline rocblas_operation blas_op(char t) {
  if (t == 'N' || t == 'n') return rocblas_operation_none;
  if (t == 'T' || t == 't') return rocblas_operation_transpose;
  fail("NativeOp: sgemm transpose flag must be 'N' or 'T', got '", t, "'");
}

// Column-major C[m,n] = alpha op(A)[m,k] op(B)[k,n] + beta C, the BLAS convention the dialect's Ndarray_sgemm has
// (returnn/native_op.cpp:522-525 forwards it to cuBLAS unchanged).
inline void sgemm_colmajor(char transa, char transb, int m, int n, int k, const float* alpha, const float* A, int lda, const float* B,
                           int ldb, const float* beta, float* C, int ldc) {
  if (m == 0 || n == 0) return;
  rocblas_handle h = blas();
  if (rocblas_set_stream(h, current().stream) != rocblas_status_success) fail("NativeOp: rocblas_set_stream failed");
  const rocblas_status st = rocblas_sgemm(h, blas_op(transa), blas_op(transb), m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
  if (st != rocblas_status_success) fail("NativeOp: rocblas_sgemm failed with status ", (int)st, " (m=", m, ", n=", n, ", k=", k, ")");
}

// Row-major C[rows,cols] = alpha op(A) op(B) + beta C; `inner` is the contraction length.  A row-major product is the
// column-major product of the transposes with the operands exchanged.
inline void gemm_rowmajor(const float* A, int lda, bool transpose_a, const float* B, int ldb, bool transpose_b, float* C, int ldc, int rows,
                          int cols, int inner, float alpha, float beta) {
  sgemm_colmajor(transpose_b ? 'T' : 'N', transpose_a ? 'T' : 'N', cols, rows, inner, &alpha, B, ldb, A, lda, &beta, C, ldc);
}

}  // namespace rtn_op

// ------------------------------------------------------------------------------------------------------------------
// The vocabulary (names as in returnn/native_op.cpp; each line cites the definition of the reference's torch/CUDA build
// it stands in for).
// ------------------------------------------------------------------------------------------------------------------

#define Ndarray rtn_ndarray                                                      /* :646 */
typedef const int64_t* Ndarray_DIMS_Type;                                        /* :653 */
typedef int64_t Ndarray_DIM_Type;                                                /* :656 */
#define Ndarray_DEV_DATA(x) ((float*)(x)->data)                                  /* :647 */
#define Ndarray_DEV_DATA_int32(x) ((int32_t*)(x)->data)                          /* :648 */
#define Ndarray_DEV_DATA_uint32(x) ((uint32_t*)(x)->data)                        /* :649 */
#define Ndarray_DEV_DATA_int32_scalar(x) (::rtn_op::scalar_int32(x))             /* :650 */
#define Ndarray_HOST_DIMS(x) ((x)->dims)                                         /* :651 */
#define Ndarray_DIMS(x) ((x)->dims)                                              /* :652 */
#define Ndarray_NDIM(x) ((x)->ndim)                                              /* :654 */
#define Ndarray_dtype_size(x) ((x)->elem_size)                                   /* :655 */
#define Ndarray_SIZE(x) (::rtn_op::count(x))                                     /* :657 */
#define Ndarray_STRIDE(x, dim) (::rtn_op::stride((x), (dim)))                    /* :658 */
#define CHECK_WITH_MSG(cond, ...) do { if (!(cond)) ::rtn_op::fail(__VA_ARGS__); } while (0)   /* :660 */
#define CONTEXT_ARGS                                                             /* :663 */

#define assert_cmp(a, cmp, b) do { if (!((a) cmp (b))) ::rtn_op::fail_cmp(#a, #cmp, #b, (a), (b), __LINE__); } while (0)   /* :58-67 */
#undef assert
#define assert(cond) do { if (!(cond)) ::rtn_op::fail_assert(#cond, __LINE__); } while (0)

#define elem_atomic_add(x, v) atomicAdd(x, v)                                    /* :92 */
#define elem_atomic_min(x, v) atomicMin(x, v)                                    /* :93 */
#define elem_atomic_cas(a, c, v) atomicCAS(a, c, v)                              /* :94 */
__host__ __device__ inline float int_as_float(int x) { return __builtin_bit_cast(float, x); }   /* :96 */
__host__ __device__ inline int float_as_int(float x) { return __builtin_bit_cast(int, x); }     /* :97 */
#define INF_F (__builtin_huge_valf())                                            /* :99 */
#define NAN_F (__builtin_nanf(""))                                               /* :100 */

#define CUDA_CUR_STREAM (::rtn_op::current().stream)                             /* :745 */
#define Ndarray_memcpy(y, x, size) (::rtn_op::check_hip(hipMemcpyAsync((y), (x), (size), hipMemcpyDeviceToDevice, CUDA_CUR_STREAM), __FILE__, __LINE__))   /* :759 */
#define Ndarray_memset(s, c, size) (::rtn_op::fill((s), (c), (size)))            /* :760 */
#define start_dev_kernel(kernel, args) (kernel<<<dim3(DIM_GRID), dim3(DIM_BLOCK), 0, CUDA_CUR_STREAM>>> args);                      /* :766 */
#define start_dev_kernel2(kernel, dim_grid, dim_block, shared_size, args) (kernel<<<(dim_grid), (dim_block), (shared_size), CUDA_CUR_STREAM>>> args);   /* :768 */
#define HANDLE_ERROR(status) (::rtn_op::check_hip((status), __FILE__, __LINE__))  /* :779 */
#define HANDLE_LAST_ERROR() (HANDLE_ERROR(hipGetLastError()))                    /* :780 */

#define Ndarray_sgemm(transpose_A, transpose_B, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc) \
  ::rtn_op::sgemm_colmajor((transpose_A), (transpose_B), (m), (n), (k), (alpha), (A), (lda), (B), (ldb), (beta), (C), (ldc))   /* :522-525 */

#define device_malloc(bytes) (::rtn_op::allocate(bytes))                         /* :955, :983 */
#define device_free(ptr) (::rtn_op::release(ptr))                                /* :956, :984 */

inline int64_t Ndarray_get_n_total_elements(Ndarray* a) { return rtn_op::count(a); }   /* :864-869 */

// The frame `x` of a [time, rows, cols] array; a matrix is returned whole (:873-885).
inline float* data_ptr(Ndarray* a, int x) {
  if (a->ndim == 2) return Ndarray_DEV_DATA(a);
  if (a->ndim != 3) rtn_op::fail("NativeOp: data_ptr needs a 2- or 3-dimensional array, got ", a->ndim, " dimensions");
  return Ndarray_DEV_DATA(a) + (int64_t)x * a->dims[1] * a->dims[2];
}
inline const float* data_ptr(const Ndarray* a, int x) { return data_ptr(const_cast<Ndarray*>(a), x); }

inline void lastTwoDims(const Ndarray* a, int out[2]) {   /* :886-891 */
  if (a->ndim < 2) rtn_op::fail("NativeOp: lastTwoDims needs at least 2 dimensions, got ", a->ndim);
  out[0] = (int)a->dims[a->ndim - 2];
  out[1] = (int)a->dims[a->ndim - 1];
}

inline int lastTwoDimsStride(const Ndarray* a) {   /* :893-897 */
  int d[2];
  lastTwoDims(a, d);
  return d[0] * d[1];
}

inline void Ndarray_set_zero(Ndarray* a) {   /* :922-926 */
  Ndarray_memset(a->data, 0, (size_t)rtn_op::count(a) * (size_t)a->elem_size);
}

// C += A B on raw row-major matrices (:1032-1068): A is [a0,a1], B is [b0,b1], C is [c0,c1] as stored; a transposed
// operand is read as its transpose; the leading dimension of A (B) is a1 (b1) times its factor.
inline void affine_raw(float* A, int a0, int a1, float* B, int b0, int b1, float* C, int c0, int c1, bool transpose_A = false,
                       bool transpose_B = false, float beta = 1.0f, float alpha = 1.0f, int ldA_factor = 1, int ldB_factor = 1) {
  const int lda = a1 * ldA_factor, ldb = b1 * ldB_factor;
  const int rows = transpose_A ? a1 : a0, inner = transpose_A ? a0 : a1;
  const int inner_b = transpose_B ? b1 : b0, cols = transpose_B ? b0 : b1;
  assert_cmp(rows, ==, c0);
  assert_cmp(cols, ==, c1);
  assert_cmp(inner, ==, inner_b);
  rtn_op::gemm_rowmajor(A, lda, transpose_A, B, ldb, transpose_B, C, c1, rows, cols, inner, alpha, beta);
}

// C[x_C] = A[x_A] B[x_B] + beta C[x_C] on the last two dimensions; the index picks a frame of a 3-dimensional array
// and is ignored for a matrix (:990-1027).
inline void affine_y_x(int x_A, Ndarray* A, int x_B, Ndarray* B, int x_C, Ndarray* C, bool transpose_A = false, bool transpose_B = false,
                       float beta = 1.0f) {
  int da[2], db[2], dc[2];
  lastTwoDims(A, da);
  lastTwoDims(B, db);
  lastTwoDims(C, dc);
  affine_raw(data_ptr(A, x_A), da[0], da[1], data_ptr(B, x_B), db[0], db[1], data_ptr(C, x_C), dc[0], dc[1], transpose_A, transpose_B, beta);
}

// C = op(A) op(B) + beta C over all frames at once: the leading dimensions of A and B are folded into rows, B starts
// `offset` frames later and A ends `offset` frames earlier (:1073-1100; e.g. sum_t Y[t-1]^T DZ[t]).
inline void affine_global(Ndarray* A, Ndarray* B, Ndarray* C, bool transpose_A = false, bool transpose_B = false, int offset = 0,
                          float beta = 1.0f) {
  int da[2], db[2];
  lastTwoDims(A, da);
  lastTwoDims(B, db);
  const int a_rows = (int)(rtn_op::count(A) / da[1]) - offset * da[0];
  const int b_rows = (int)(rtn_op::count(B) / db[1]) - offset * db[0];
  const float* b_data = Ndarray_DEV_DATA(B) + (int64_t)offset * db[0] * db[1];
  const int rows = transpose_A ? da[1] : a_rows, inner = transpose_A ? a_rows : da[1];
  const int cols = transpose_B ? b_rows : db[1], inner_b = transpose_B ? db[1] : b_rows;
  assert_cmp(inner, ==, inner_b);
  rtn_op::gemm_rowmajor(Ndarray_DEV_DATA(A), da[1], transpose_A, b_data, db[1], transpose_B, Ndarray_DEV_DATA(C), cols, rows, cols, inner, 1.0f,
                        beta);
}
