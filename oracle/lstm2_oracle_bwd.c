/*
 * CPU oracle for the NativeLstm2 backward op.  TEST INFRASTRUCTURE ONLY (see lstm2_oracle.c).
 *
 * Restates, in plain C:
 *   - host driver      returnn/native_op.py:1288-1464  (c_bw_code): DW := 0, Dy0 := 0 (working copy of the error that
 *                      flows into the output of the frame before), Dc0 := Dd (working copy of the cell error), dx0 := 0;
 *                      frames visited in reverse processing order; per frame the pointwise kernel, then
 *                      Dy0 += DX[t] * W^T; afterwards DW = sum_t Y[t_prev]^T * DX[t] over consecutive visited frames
 *                      and DW += y0^T * dx0
 *   - pointwise kernel returnn/native_op.py:1123-1180  (lstm_bwd_kernel)
 *   - GEMMs            returnn/native_op.cpp:1032-1067 (_affine_raw with its transpose flags; ascending-k sums)
 *   - inputs of the gradient op: returnn/native_op.py:1071-1077 (grad_input_map: X W y0 c0 i start step Y C H DY Dd)
 *
 * Parity status: PINNED by tests/test_oracle_bwd.py -- gradients of torch.nn.LSTM (autograd, float64, full-length and
 * packed ragged batches, both directions, with initial states and a loss on Y and on the final cell), central finite
 * differences of the (pinned) forward oracle in float64 for every input incl. start/step variants, and closed forms.
 *
 * Frames that are not visited get DX = 0.  T == 0: DX empty, DW = 0, Dy0 = 0, Dc0 = Dd.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LSTM2_OK 0
#define LSTM2_ERR_RANGE 2
#define LSTM2_ERR_ALLOC 3

/* lstm_bwd_kernel (returnn/native_op.py:1123-1180) for one frame, executed sequentially like the reference's CPU
 * emulation of a kernel launch (returnn/native_op.cpp:782-858). */
#define DEFINE_BWD_POINTWISE(NAME, REAL, TANHF)                                                                    \
  static void NAME(int32_t B, int32_t n, const REAL* m, const REAL* h, const REAL* prev_c, const REAL* d_y,        \
                   REAL* d_h, REAL* d_c, REAL* d_x, REAL* dx0) {                                                   \
    const int64_t bn = (int64_t)B * n, n4 = (int64_t)n * 4;                                                        \
    for (int64_t idx = 0; idx < bn; ++idx) {                                                                       \
      const int64_t b = idx / n, cell = idx % n;                                                                   \
      const int64_t io = b * n4 + cell;                                                                            \
      const REAL mask_b = m[b];                                                                                    \
      const REAL d_y_b = (d_y[idx] + d_h[idx]) * mask_b;                                                           \
      const REAL d_c_b = d_c[idx] * mask_b;                                                                        \
      const REAL prev_c_b = prev_c[idx];                                                                           \
      const REAL cellIn = h[io], inpGate = h[io + n], fgtGate = h[io + 2 * n], outGate = h[io + 3 * n];            \
      const REAL c_b = prev_c_b * fgtGate + cellIn * inpGate;                                                      \
      const REAL gc = TANHF(c_b);                                                                                  \
      const REAL d_outGate_in = ((REAL)1 - outGate) * outGate * gc * d_y_b;                                        \
      const REAL d_c2 = d_c_b + outGate * d_y_b * ((REAL)1 - gc * gc);                                             \
      const REAL d_cellIn_in = ((REAL)1 - cellIn * cellIn) * inpGate * d_c2;                                       \
      const REAL d_inpGate_in = ((REAL)1 - inpGate) * inpGate * cellIn * d_c2;                                     \
      const REAL d_fgtGate_in = ((REAL)1 - fgtGate) * fgtGate * prev_c_b * d_c2;                                   \
      d_c[idx] = fgtGate * d_c2 + d_c[idx] * ((REAL)1 - mask_b);                                                   \
      d_x[io] = d_cellIn_in;                                                                                       \
      d_x[io + n] = d_inpGate_in;                                                                                  \
      d_x[io + 2 * n] = d_fgtGate_in;                                                                              \
      d_x[io + 3 * n] = d_outGate_in;                                                                              \
      for (int g = 0; g < 4; ++g) dx0[io + g * n] = d_x[io + g * n] + dx0[io + g * n] * ((REAL)1 - mask_b);        \
      d_h[idx] *= ((REAL)1 - mask_b);                                                                              \
    }                                                                                                              \
  }

DEFINE_BWD_POINTWISE(bwd_pointwise_f32, float, tanhf)
DEFINE_BWD_POINTWISE(bwd_pointwise_f64, double, tanh)

#define DEFINE_BWD(NAME, REAL, POINTWISE)                                                                            \
  int NAME(const REAL* X, const REAL* W, const REAL* y0, const REAL* c0, const REAL* mask, int32_t start,          \
           int32_t step, const REAL* Y, const REAL* C, const REAL* H, const REAL* DY, const REAL* Dd, REAL* DX,    \
           REAL* DW, REAL* Dy0, REAL* Dc0, int64_t T, int32_t B, int32_t n) {                                      \
    (void)X;                                                                                                       \
    const int64_t bn = (int64_t)B * n, bn4 = bn * 4, n4 = (int64_t)n * 4;                                          \
    memset(DW, 0, sizeof(REAL) * (size_t)n * (size_t)n4);                                                          \
    memset(Dy0, 0, sizeof(REAL) * (size_t)bn);                                                                     \
    memcpy(Dc0, Dd, sizeof(REAL) * (size_t)bn);                                                                    \
    if (T == 0) return LSTM2_OK;                                                                                   \
    if (start < 0 || start >= T || step == 0) return LSTM2_ERR_RANGE;                                              \
    REAL* dx0 = (REAL*)calloc((size_t)bn4, sizeof(REAL));                                                          \
    if (!dx0) return LSTM2_ERR_ALLOC;                                                                              \
    memset(DX, 0, sizeof(REAL) * (size_t)T * (size_t)bn4);                                                         \
    const int64_t abs_step = step > 0 ? step : -(int64_t)step;                                                     \
    const int64_t num_steps = (T - start + abs_step - 1) / abs_step;                                               \
    int64_t first = start;                                                                                         \
    if (step < 0) first = T - start - 1;                                                                           \
    const int64_t end = first + (num_steps - 1) * step; /* inclusive */                                            \
    for (int64_t t = end; (step > 0) ? (t >= first) : (t <= first); t -= step) {                                   \
      const int right = (step > 0) ? (t - step >= first) : (t - step <= first);                                    \
      const REAL* h = H + t * bn4;                                                                                 \
      const REAL* prev_c = right ? C + (t - step) * bn : c0;                                                       \
      const REAL* d_y = DY + t * bn;                                                                               \
      REAL* d_x = DX + t * bn4;                                                                                    \
      const REAL* m = mask + t * B;                                                                                \
      POINTWISE(B, n, m, h, prev_c, d_y, Dy0, Dc0, d_x, dx0);                                                      \
      /* Dy0 += DX[t] * W^T */                                                                                     \
      for (int64_t b = 0; b < B; ++b)                                                                              \
        for (int64_t k = 0; k < n; ++k) {                                                                          \
          REAL acc = Dy0[b * n + k];                                                                               \
          const REAL* dxr = d_x + b * n4;                                                                          \
          const REAL* wr = W + k * n4;                                                                             \
          for (int64_t j = 0; j < n4; ++j) acc += dxr[j] * wr[j];                                                  \
          Dy0[b * n + k] = acc;                                                                                    \
        }                                                                                                          \
    }                                                                                                              \
    /* DW += Y[t - step]^T * DX[t] for every visited frame but the first one */                                    \
    for (int64_t t = end; (step > 0) ? (t - step >= first) : (t - step <= first); t -= step) {                     \
      const REAL* y = Y + (t - step) * bn;                                                                         \
      const REAL* d_x = DX + t * bn4;                                                                              \
      for (int64_t b = 0; b < B; ++b)                                                                              \
        for (int64_t k = 0; k < n; ++k) {                                                                          \
          const REAL yv = y[b * n + k];                                                                            \
          REAL* dwr = DW + k * n4;                                                                                 \
          const REAL* dxr = d_x + b * n4;                                                                          \
          for (int64_t j = 0; j < n4; ++j) dwr[j] += yv * dxr[j];                                                  \
        }                                                                                                          \
    }                                                                                                              \
    /* DW += y0^T * dx0 */                                                                                         \
    for (int64_t b = 0; b < B; ++b)                                                                                \
      for (int64_t k = 0; k < n; ++k) {                                                                            \
        const REAL yv = y0[b * n + k];                                                                             \
        REAL* dwr = DW + k * n4;                                                                                   \
        const REAL* dxr = dx0 + b * n4;                                                                            \
        for (int64_t j = 0; j < n4; ++j) dwr[j] += yv * dxr[j];                                                    \
      }                                                                                                            \
    free(dx0);                                                                                                     \
    return LSTM2_OK;                                                                                               \
  }

DEFINE_BWD(lstm2_oracle_bwd_f32, float, bwd_pointwise_f32)
DEFINE_BWD(lstm2_oracle_bwd_f64, double, bwd_pointwise_f64)

/* The pointwise kernel alone (for the BLAS-based variant the benchmark times as CPU baseline). */
void lstm2_oracle_bwd_pointwise_f32(int32_t B, int32_t n, const float* m, const float* h, const float* prev_c,
                                    const float* d_y, float* d_h, float* d_c, float* d_x, float* dx0) {
  bwd_pointwise_f32(B, n, m, h, prev_c, d_y, d_h, d_c, d_x, dx0);
}
