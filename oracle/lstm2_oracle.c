/*
 * CPU oracle for the NativeLstm2 forward op.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP path is compared against and the CPU
 * baseline that the benchmark times next to it.  It is never part of the
 * shipped library: nothing under returnn_amd/ may link, load or call it.
 *
 * It restates, in plain C, the algorithm of the reference operator:
 *   - host driver      returnn/native_op.py:1184-1285  (c_fw_code)
 *   - pointwise kernel returnn/native_op.py:1081-1121  (lstm_kernel)
 *   - recurrent GEMM   returnn/native_op.cpp:1032-1067 (_affine_raw: C += A*B,
 *                      row major, alpha = beta = 1)
 *   - time slicing     returnn/native_op.cpp:872-880   (data_ptr)
 *   - zero-initialised outputs before the op body
 *                      returnn/torch/util/native_op.py:170-184
 *   - sequential execution of the kernel's grid-stride loop on the CPU
 *                      returnn/native_op.cpp:782-858   (_KernelLoop)
 *   - caller-side final output (not part of the op)
 *                      returnn/tf/native_op.py:913-929 (_lstm_last_output)
 *
 * Parity status of every function here: PINNED.  tests/test_oracle.py checks
 * them against the reference's own deterministic fixture and comparison rules
 * (tests/test_TFNativeOp.py:824,851-854,866-889) through an independently
 * written textbook LSTM, against torch.lstm (full-length and packed ragged
 * sequences), against closed forms (T=B=n=1; zero X and W; mask == 0), the
 * start/step slice-equivalence and time-reversal invariants, and against an
 * fp64 brute force on tiny shapes.
 *
 * Gate layout in the last axis of X, H and W (returnn/native_op.py:1096-1109):
 *   [0:n) cell-in (tanh), [n:2n) input gate, [2n:3n) forget gate,
 *   [3n:4n) output gate.
 *
 * Two precisions are generated from one body: float (the reference's
 * arithmetic: expf/tanhf, fp32 accumulation) and double (a higher-precision
 * variant used to judge rounding error; same control flow).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define LSTM2_OK 0
#define LSTM2_ERR_SHAPE 1
#define LSTM2_ERR_RANGE 2
#define LSTM2_ERR_ALLOC 3

/* C[b, :] += A[b, :] * Bm  for A:[a0,a1], Bm:[a1,b1], C:[a0,b1], row major.
 * Follows the operand meaning of _affine_raw (returnn/native_op.cpp:1032-1067)
 * with transpose flags false and alpha = beta = 1.  The column range is split
 * over `threads` OpenMP threads (the reference's CPU GEMM back-end is a
 * multi-threaded contraction, returnn/native_op.cpp:557-620); with threads <= 1
 * it is a plain sequential loop.  Every C element is updated over ascending k,
 * whatever the thread count, so results do not depend on `threads`. */
#define DEFINE_AFFINE(NAME, REAL)                                                     \
  static void NAME(const REAL* A, int a0, int a1, const REAL* Bm, int b1, REAL* C,    \
                   int threads) {                                                     \
    const int blk = 128;                                                              \
    const int nblk = (b1 + blk - 1) / blk;                                            \
    (void)threads;                                                                    \
    _Pragma("omp parallel for schedule(static) num_threads(threads) if (threads > 1)") \
    for (int jb = 0; jb < nblk; ++jb) {                                               \
      const int j0 = jb * blk;                                                        \
      const int j1 = (j0 + blk < b1) ? j0 + blk : b1;                                 \
      for (int k = 0; k < a1; ++k) {                                                  \
        const REAL* w = Bm + (size_t)k * b1;                                          \
        for (int r = 0; r < a0; ++r) {                                                \
          REAL* c = C + (size_t)r * b1;                                               \
          const REAL av = A[(size_t)r * a1 + k];                                      \
          for (int j = j0; j < j1; ++j) c[j] += av * w[j];                            \
        }                                                                             \
      }                                                                               \
    }                                                                                 \
  }

DEFINE_AFFINE(affine_f32, float)
DEFINE_AFFINE(affine_f64, double)

/* One time step of the pointwise part, all (batch, cell) pairs in ascending
 * idx order on one thread, as _KernelLoop runs it (returnn/native_op.cpp:834-858).
 * Arithmetic order follows returnn/native_op.py:1097-1116 term by term. */
#define DEFINE_POINTWISE(NAME, REAL, EXPF, TANHF)                                     \
  static void NAME(int n_batch, int n_cells, const REAL* mask, REAL* h,               \
                   const REAL* prev_y, const REAL* prev_c, REAL* y, REAL* c,          \
                   REAL* y_prev_out) {                                                \
    const REAL one = (REAL)1;                                                         \
    for (int idx = 0; idx < n_cells * n_batch; ++idx) {                               \
      const int batch_idx = idx / n_cells;                                            \
      const int cell_idx = idx % n_cells;                                             \
      const size_t off = (size_t)batch_idx * 4 * n_cells + cell_idx;                  \
      const REAL prev_c_b = prev_c[idx];                                              \
      const REAL mask_b = mask[batch_idx];                                            \
      const REAL cell_in = TANHF(h[off]);                                             \
      const REAL inp = one / (one + EXPF(-h[off + n_cells]));                         \
      const REAL fgt = one / (one + EXPF(-h[off + 2 * (size_t)n_cells]));             \
      const REAL out = one / (one + EXPF(-h[off + 3 * (size_t)n_cells]));             \
      h[off] = cell_in;                                                               \
      h[off + n_cells] = inp;                                                         \
      h[off + 2 * (size_t)n_cells] = fgt;                                             \
      h[off + 3 * (size_t)n_cells] = out;                                             \
      const REAL c_b = (prev_c_b * fgt + cell_in * inp) * mask_b                      \
                       + prev_c_b * (one - mask_b);                                   \
      c[idx] = c_b;                                                                   \
      const REAL y_b = TANHF(c_b) * out * mask_b;                                     \
      y[idx] = y_b;                                                                   \
      y_prev_out[idx] = y_b + prev_y[idx] * (one - mask_b);                           \
    }                                                                                 \
  }

DEFINE_POINTWISE(pointwise_f32, float, expf, tanhf)
DEFINE_POINTWISE(pointwise_f64, double, exp, tanh)

/* The op.  Outputs are fully written (zero-initialised first, as the
 * reference's wrapper does).  y_last (optional, may be NULL) receives the
 * content of the y_prev carry after the last visited step, which equals the
 * caller-side _lstm_last_output value; for T == 0 it receives y0.
 * Unlike the reference under -DNDEBUG (returnn/native_op.cpp:60-69 prints
 * only), range violations are returned as errors. */
#define DEFINE_FWD(NAME, REAL, AFFINE, POINTWISE)                                     \
  int NAME(const REAL* X, const REAL* W, const REAL* y0, const REAL* c0,              \
           const REAL* i, int32_t start, int32_t step, REAL* Y, REAL* C, REAL* H,     \
           REAL* d, REAL* y_last, int64_t T, int32_t n_batch, int32_t n_cells,        \
           int32_t threads) {                                                         \
    if (T < 0 || n_batch < 0 || n_cells < 0) return LSTM2_ERR_SHAPE;                  \
    const size_t bn = (size_t)n_batch * n_cells;                                      \
    memset(Y, 0, (size_t)T * bn * sizeof(REAL));                                      \
    memset(C, 0, (size_t)T * bn * sizeof(REAL));                                      \
    memset(H, 0, (size_t)T * bn * 4 * sizeof(REAL));                                  \
    memset(d, 0, bn * sizeof(REAL));                                                  \
    if (T == 0) {                                                                     \
      memcpy(d, c0, bn * sizeof(REAL));                                               \
      if (y_last) memcpy(y_last, y0, bn * sizeof(REAL));                              \
      return LSTM2_OK;                                                                \
    }                                                                                 \
    if (start < 0 || start >= T || step == 0) return LSTM2_ERR_RANGE;                 \
    REAL* y_prev = (REAL*)malloc((bn ? bn : 1) * sizeof(REAL));                       \
    if (!y_prev) return LSTM2_ERR_ALLOC;                                              \
    memcpy(H, X, (size_t)T * bn * 4 * sizeof(REAL));                                  \
    int64_t end = T - 1;                                                              \
    int64_t first = start;                                                            \
    if (step < 0) {                                                                   \
      end = 0;                                                                        \
      first = T - start - 1;                                                          \
    }                                                                                 \
    int64_t t = first;                                                                \
    for (; (step > 0) ? (t <= end) : (t >= end); t += step) {                         \
      REAL* Ht = H + (size_t)t * bn * 4;                                              \
      const REAL* y_in = (t != first) ? y_prev : y0;                                  \
      const REAL* c_in = (t != first) ? C + (size_t)(t - step) * bn : c0;             \
      AFFINE(y_in, n_batch, n_cells, W, n_cells * 4, Ht, threads);                    \
      POINTWISE(n_batch, n_cells, i + (size_t)t * n_batch, Ht, y_in, c_in,            \
                Y + (size_t)t * bn, C + (size_t)t * bn, y_prev);                      \
    }                                                                                 \
    memcpy(d, C + (size_t)(t - step) * bn, bn * sizeof(REAL));                        \
    if (y_last) memcpy(y_last, y_prev, bn * sizeof(REAL));                            \
    free(y_prev);                                                                     \
    return LSTM2_OK;                                                                  \
  }

DEFINE_FWD(lstm2_oracle_fwd_f32, float, affine_f32, pointwise_f32)
DEFINE_FWD(lstm2_oracle_fwd_f64, double, affine_f64, pointwise_f64)

/* Caller-side final output, returnn/tf/native_op.py:913-929: per sequence the
 * row of Y at the last visited frame (in processing order) whose mask is
 * non-zero, or y0 if no visited frame of that sequence is valid.  "Visited"
 * = frames first, first+step, ... inside [0, T).  The mask is cast to int as
 * the reference does (tf.cast(mask, tf.int32)). */
#define DEFINE_LAST_OUTPUT(NAME, REAL)                                                \
  int NAME(const REAL* Y, const REAL* y0, const REAL* i, int32_t start, int32_t step, \
           REAL* out, int64_t T, int32_t n_batch, int32_t n_cells) {                  \
    if (T < 0 || n_batch < 0 || n_cells < 0) return LSTM2_ERR_SHAPE;                  \
    const size_t bn = (size_t)n_batch * n_cells;                                      \
    memcpy(out, y0, bn * sizeof(REAL));                                               \
    if (T == 0) return LSTM2_OK;                                                      \
    if (start < 0 || start >= T || step == 0) return LSTM2_ERR_RANGE;                 \
    int64_t first = (step < 0) ? T - start - 1 : start;                               \
    for (int b = 0; b < n_batch; ++b) {                                               \
      int64_t last = -1;                                                              \
      for (int64_t t = first; t >= 0 && t < T; t += step)                             \
        if ((int)i[(size_t)t * n_batch + b] != 0) last = t;                           \
      if (last >= 0)                                                                  \
        memcpy(out + (size_t)b * n_cells, Y + (size_t)last * bn + (size_t)b * n_cells, \
               (size_t)n_cells * sizeof(REAL));                                       \
    }                                                                                 \
    return LSTM2_OK;                                                                  \
  }

DEFINE_LAST_OUTPUT(lstm2_oracle_last_output_f32, float)
DEFINE_LAST_OUTPUT(lstm2_oracle_last_output_f64, double)

/* One pointwise step on its own (returnn/native_op.py:1081-1121), for a driver that does the
 * recurrent GEMM with a BLAS, as the reference's CPU path does (returnn/native_op.cpp:535-620). */
void lstm2_oracle_pointwise_f32(int32_t n_batch, int32_t n_cells, const float* mask, float* h,
                                const float* prev_y, const float* prev_c, float* y, float* c,
                                float* y_prev_out) {
  pointwise_f32(n_batch, n_cells, mask, h, prev_y, prev_c, y, c, y_prev_out);
}

int lstm2_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
