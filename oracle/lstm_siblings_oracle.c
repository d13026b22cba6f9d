/*
 * CPU oracle for the forward pass of NativeLstm2's sibling ops.  TEST INFRASTRUCTURE ONLY (see lstm2_oracle.c).
 *
 * LstmGenericBase: returnn/native_op.py:486-523 (c_fw_code: H := Z; for every frame x: H[x] += Y[x-1] * V_h for x > 0,
 *   then the kernel with the old state taken from H[x-1]'s first block, or from c for x == 0; d from the last frame)
 *   and :381-429 (lstm_kernel: gates, state := state * i + old_state * (1 - i), output = outGate * tanh(state) * i,
 *   the state and the three activated gates written back into H).
 * LstmLowMem: returnn/native_op.py:771-836 (c_fw_code: per visited frame intern = [X[t], Y[t-step] or y0] * W + b,
 *   then the kernel; d = C of the last visited frame) and :624-655 (lstm_kernel).
 *
 * LstmGenericBase gradient: returnn/native_op.py:525-574 (c_bw_code: frames in descending order; the error of the
 *   output is DY[x] plus DZ[x+1] * V_h^T; the kernel; then DV_h = sum_x Y[x]^T DZ[x+1] and Dc = the error that reaches
 *   the initial cell state) and :430-485 (lstm_bwd_kernel: works on the stored cell state and gates, recovers
 *   tanh(cell-in) as (state - forget * old_state) / max(input, 1e-16), all gate errors multiplied by the mask).
 *
 * Parity status: PINNED by tests/test_oracle_siblings.py -- the reference's own closed-form vector for LstmLowMem
 * (tests/test_TFNativeOp.py:264-297), its all-zero run of the LstmGenericBase cell (:234-250: zero input, zero state
 * => zero output), an independently written float64 loop with masks in the middle of sequences, torch.nn.LSTM on
 * full-length batches, and agreement with the (pinned) NativeLstm2 oracle where the semantics coincide; the gradient
 * by central finite differences of the pinned forward oracle (all three inputs, masks with holes) and by autograd
 * through an independent torch restatement of the forward pass.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DEFINE_GENERIC_BASE(NAME, REAL, EXPF, TANHF)                                                               \
  int NAME(const REAL* Z, const REAL* V_h, const REAL* c, const REAL* mask, REAL* Y, REAL* H, REAL* d, int64_t T,   \
           int32_t B, int32_t n) {                                                                                 \
    if (T <= 0) return 1;                                                                                          \
    const int64_t bn = (int64_t)B * n, n4 = (int64_t)n * 4, bn4 = bn * 4;                                          \
    memcpy(H, Z, sizeof(REAL) * (size_t)T * (size_t)bn4);                                                          \
    for (int64_t x = 0; x < T; ++x) {                                                                              \
      REAL* data = H + x * bn4;                                                                                    \
      if (x > 0) {                                                                                                 \
        const REAL* yp = Y + (x - 1) * bn;                                                                         \
        for (int64_t b = 0; b < B; ++b)                                                                            \
          for (int64_t k = 0; k < n; ++k) {                                                                        \
            const REAL yv = yp[b * n + k];                                                                         \
            const REAL* vr = V_h + k * n4;                                                                         \
            REAL* hr = data + b * n4;                                                                              \
            for (int64_t j = 0; j < n4; ++j) hr[j] += yv * vr[j];                                                  \
          }                                                                                                        \
      }                                                                                                            \
      for (int64_t idx = 0; idx < bn; ++idx) {                                                                     \
        const int64_t b = idx / n;                                                                                 \
        const int64_t start = b * n4 + idx % n;                                                                    \
        const REAL i_batch = mask[x * B + b];                                                                      \
        const REAL inpGate = (REAL)1 / ((REAL)1 + EXPF(-data[start + n]));                                         \
        const REAL fgtGate = (REAL)1 / ((REAL)1 + EXPF(-data[start + 2 * n]));                                     \
        const REAL outGate = (REAL)1 / ((REAL)1 + EXPF(-data[start + 3 * n]));                                     \
        REAL state = inpGate * TANHF(data[start]);                                                                 \
        const REAL old_state = x > 0 ? (H + (x - 1) * bn4)[start] : c[idx];                                        \
        state += fgtGate * old_state;                                                                              \
        state = state * i_batch + old_state * ((REAL)1 - i_batch);                                                 \
        Y[x * bn + idx] = outGate * TANHF(state) * i_batch;                                                        \
        data[start] = state;                                                                                       \
        data[start + n] = inpGate;                                                                                 \
        data[start + 2 * n] = fgtGate;                                                                             \
        data[start + 3 * n] = outGate;                                                                             \
        if (x == T - 1) d[idx] = state;                                                                            \
      }                                                                                                            \
    }                                                                                                              \
    return 0;                                                                                                      \
  }

DEFINE_GENERIC_BASE(lstm_generic_base_oracle_fwd_f32, float, expf, tanhf)
DEFINE_GENERIC_BASE(lstm_generic_base_oracle_fwd_f64, double, exp, tanh)

#define DEFINE_LOW_MEM(NAME, REAL, EXPF, TANHF)                                                                    \
  int NAME(const REAL* X, const REAL* W, const REAL* bias, const REAL* y0, const REAL* c0, const REAL* mask,        \
           int32_t start, int32_t step, REAL* Y, REAL* C, REAL* d, int64_t T, int32_t B, int32_t n_in, int32_t n) { \
    const int64_t bn = (int64_t)B * n, n4 = (int64_t)n * 4;                                                        \
    memset(Y, 0, sizeof(REAL) * (size_t)T * (size_t)bn);                                                           \
    memset(C, 0, sizeof(REAL) * (size_t)T * (size_t)bn);                                                           \
    if (T == 0) {                                                                                                  \
      memcpy(d, c0, sizeof(REAL) * (size_t)bn);                                                                    \
      return 0;                                                                                                    \
    }                                                                                                              \
    if (start < 0 || start >= T || step == 0) return 2;                                                            \
    if (step < 0 && T - start - 1 < start) return 4; /* no frame visited: the reference reads d from an unwritten C */ \
    REAL* intern = (REAL*)malloc(sizeof(REAL) * (size_t)B * (size_t)n4);                                           \
    if (!intern) return 3;                                                                                         \
    int64_t first = start, end = T - 1;                                                                            \
    if (step < 0) {                                                                                                \
      end = start;                                                                                                 \
      first = T - start - 1;                                                                                       \
    }                                                                                                              \
    int64_t t = first;                                                                                             \
    for (; (step > 0) ? (t <= end) : (t >= end); t += step) {                                                      \
      const REAL* yprev = (t != first) ? Y + (t - step) * bn : y0;                                                 \
      const REAL* cprev = (t != first) ? C + (t - step) * bn : c0;                                                 \
      for (int64_t b = 0; b < B; ++b) {                                                                            \
        REAL* ir = intern + b * n4;                                                                                \
        for (int64_t j = 0; j < n4; ++j) ir[j] = 0;                                                                \
        for (int64_t k = 0; k < n_in; ++k) {                                                                       \
          const REAL xv = X[(t * B + b) * n_in + k];                                                               \
          const REAL* wr = W + k * n4;                                                                             \
          for (int64_t j = 0; j < n4; ++j) ir[j] += xv * wr[j];                                                    \
        }                                                                                                          \
        for (int64_t k = 0; k < n; ++k) {                                                                          \
          const REAL yv = yprev[b * n + k];                                                                        \
          const REAL* wr = W + (n_in + k) * n4;                                                                    \
          for (int64_t j = 0; j < n4; ++j) ir[j] += yv * wr[j];                                                    \
        }                                                                                                          \
        for (int64_t j = 0; j < n4; ++j) ir[j] += bias[j];                                                         \
      }                                                                                                            \
      for (int64_t idx = 0; idx < bn; ++idx) {                                                                     \
        const int64_t b = idx / n, cell = idx % n;                                                                 \
        const int64_t io = b * n4 + cell;                                                                          \
        const REAL prev_c_b = cprev[idx];                                                                          \
        const REAL mask_b = mask[t * B + b];                                                                       \
        const REAL cellIn = TANHF(intern[io]);                                                                     \
        const REAL inpGate = (REAL)1 / ((REAL)1 + EXPF(-intern[io + n]));                                          \
        const REAL fgtGate = (REAL)1 / ((REAL)1 + EXPF(-intern[io + 2 * n]));                                      \
        const REAL outGate = (REAL)1 / ((REAL)1 + EXPF(-intern[io + 3 * n]));                                      \
        const REAL c_b = (prev_c_b * fgtGate + cellIn * inpGate) * mask_b + prev_c_b * ((REAL)1 - mask_b);         \
        C[t * bn + idx] = c_b;                                                                                     \
        Y[t * bn + idx] = TANHF(c_b) * outGate * mask_b;                                                           \
      }                                                                                                            \
    }                                                                                                              \
    memcpy(d, C + (t - step) * bn, sizeof(REAL) * (size_t)bn);                                                     \
    free(intern);                                                                                                  \
    return 0;                                                                                                      \
  }

DEFINE_LOW_MEM(lstm_low_mem_oracle_fwd_f32, float, expf, tanhf)
DEFINE_LOW_MEM(lstm_low_mem_oracle_fwd_f64, double, exp, tanh)

/* DZ [T,B,4n], DV_h [n,4n], Dc [B,n] from V_h, c, mask, Y, H (the forward pass's results), DY, Dd. */
#define DEFINE_GENERIC_BASE_BWD(NAME, REAL, TANHF)                                                                 \
  int NAME(const REAL* V_h, const REAL* c, const REAL* mask, const REAL* Y, const REAL* H, const REAL* DY,          \
           const REAL* Dd, REAL* DZ, REAL* DV_h, REAL* Dc, int64_t T, int32_t B, int32_t n) {                       \
    if (T <= 0) return 1;                                                                                          \
    const int64_t bn = (int64_t)B * n, n4 = (int64_t)n * 4, bn4 = bn * 4;                                          \
    REAL* eps = (REAL*)malloc(sizeof(REAL) * (size_t)T * (size_t)bn); /* the reference works in place on DY */      \
    if (!eps) return 3;                                                                                            \
    memcpy(eps, DY, sizeof(REAL) * (size_t)T * (size_t)bn);                                                        \
    memcpy(DZ, H, sizeof(REAL) * (size_t)T * (size_t)bn4); /* ... and in place on H */                              \
    for (int64_t x = T - 1; x >= 0; --x) {                                                                         \
      REAL* delta = DZ + x * bn4;                                                                                  \
      REAL* epsilon = eps + x * bn;                                                                                \
      if (x < T - 1) { /* epsilon += DZ[x+1] * V_h^T */                                                             \
        const REAL* dn = DZ + (x + 1) * bn4;                                                                       \
        for (int64_t b = 0; b < B; ++b)                                                                            \
          for (int64_t k = 0; k < n; ++k) {                                                                        \
            REAL acc = 0;                                                                                          \
            const REAL* vr = V_h + k * n4;                                                                         \
            const REAL* dr = dn + b * n4;                                                                          \
            for (int64_t j = 0; j < n4; ++j) acc += dr[j] * vr[j];                                                 \
            epsilon[b * n + k] += acc;                                                                             \
          }                                                                                                        \
      }                                                                                                            \
      const REAL* next_epsilon = (x == T - 1) ? Dd : eps + (x + 1) * bn;                                           \
      for (int64_t idx = 0; idx < bn; ++idx) {                                                                     \
        const int64_t b = idx / n;                                                                                 \
        const int64_t start = b * n4 + idx % n;                                                                    \
        const REAL i_batch = mask[x * B + b];                                                                      \
        const REAL inpGate = delta[start + n], fgtGate = delta[start + 2 * n], outGate = delta[start + 3 * n];     \
        const REAL oldState = x > 0 ? (DZ + (x - 1) * bn4)[start] : c[idx]; /* H[x-1] is still untouched */         \
        const REAL state = delta[start];                                                                           \
        const REAL e = epsilon[idx];                                                                               \
        const REAL gc = TANHF(state);                                                                              \
        const REAL floor_ = (REAL)1e-16;                                                                           \
        const REAL gzc = (state - fgtGate * oldState) / (inpGate > floor_ ? inpGate : floor_);                     \
        delta[start + 3 * n] = outGate * ((REAL)1 - outGate) * gc * e * i_batch;                                   \
        REAL epsilon_c = ((REAL)1 - gc * gc) * outGate * e;                                                        \
        epsilon_c += next_epsilon[idx];                                                                            \
        epsilon[idx] = epsilon_c * fgtGate * i_batch + next_epsilon[idx] * ((REAL)1 - i_batch);                    \
        delta[start] = inpGate * ((REAL)1 - gzc * gzc) * epsilon_c * i_batch;                                      \
        delta[start + 2 * n] = fgtGate * ((REAL)1 - fgtGate) * oldState * epsilon_c * i_batch;                     \
        delta[start + n] = inpGate * ((REAL)1 - inpGate) * gzc * epsilon_c * i_batch;                              \
      }                                                                                                            \
    }                                                                                                              \
    /* DV_h = Y[0..T-2]^T * DZ[1..T-1] */                                                                          \
    memset(DV_h, 0, sizeof(REAL) * (size_t)n * (size_t)n4);                                                        \
    for (int64_t x = 0; x + 1 < T; ++x)                                                                            \
      for (int64_t b = 0; b < B; ++b)                                                                              \
        for (int64_t k = 0; k < n; ++k) {                                                                          \
          const REAL yv = Y[(x * B + b) * n + k];                                                                  \
          const REAL* dr = DZ + (x + 1) * bn4 + b * n4;                                                            \
          REAL* out = DV_h + k * n4;                                                                               \
          for (int64_t j = 0; j < n4; ++j) out[j] += yv * dr[j];                                                   \
        }                                                                                                          \
    memcpy(Dc, eps, sizeof(REAL) * (size_t)bn);                                                                    \
    free(eps);                                                                                                     \
    return 0;                                                                                                      \
  }

DEFINE_GENERIC_BASE_BWD(lstm_generic_base_oracle_bwd_f32, float, tanhf)
DEFINE_GENERIC_BASE_BWD(lstm_generic_base_oracle_bwd_f64, double, tanh)
