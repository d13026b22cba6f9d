// gfx950 kernels of the NativeLstm2 gradient op: one pointwise launch and one recurrent-GEMM launch per visited
// frame, in reverse processing order (returnn/native_op.py:1288-1464, lstm_bwd_kernel :1123-1180).
#pragma once

#include "lstm2_kernels.h"

namespace rtn {

struct Lstm2BwdParams {
  // inputs (device)
  const void* W;      // [n,4n] AT
  const float* c0;    // [B,n]
  const float* mask;  // [T,B]
  const float* C;     // [T,B,n]
  const void* H;      // [T,B,4n] AT, activated gates of the forward pass
  const void* DY;     // [T,B,n] AT
  // outputs / working arrays (device)
  void* DX;    // [T,B,4n] AT
  float* dyw;  // [B,n]  error flowing into the output of the frame before (working copy of Dy0, float32)
  float* Dc0;  // [B,n]  cell error, worked on in place
  void* dx0;   // [B,4n] AT: DX of each sequence's first processed valid frame
  long long T;
  int B, n;
};

// Pointwise part of one frame t: gate derivatives from the stored activations, cell error carried on.
// prev_t < 0: the frame before is the initial state (prev_c = c0).
template <typename AT>
__global__ void k_bwd_pointwise(Lstm2BwdParams p, long long t, long long prev_t) {
  using E = Elem<AT>;
  const long long bn = (long long)p.B * p.n;
  const long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  if (idx >= bn) return;
  const int n = p.n;
  const long long b = idx / n, cell = idx % n;
  const long long io = b * 4 * n + cell;
  const long long fo = t * bn * 4 + io;  // inside H / DX
  const float m = p.mask[t * p.B + b];
  const float dyw = p.dyw[idx];
  const float d_y_b = (E::load(p.DY, t * bn + idx) + dyw) * m;
  const float dc = p.Dc0[idx];
  const float d_c_b = dc * m;
  const float prev_c = prev_t >= 0 ? p.C[prev_t * bn + idx] : p.c0[idx];
  const float cellIn = E::load(p.H, fo), inpGate = E::load(p.H, fo + n), fgtGate = E::load(p.H, fo + 2 * n),
              outGate = E::load(p.H, fo + 3 * n);
  const float c_b = prev_c * fgtGate + cellIn * inpGate;
  const float gc = Act<AT>::tanh(c_b);
  const float d_out = (1.f - outGate) * outGate * gc * d_y_b;
  const float d_c2 = d_c_b + outGate * d_y_b * (1.f - gc * gc);
  const float d_cin = (1.f - cellIn * cellIn) * inpGate * d_c2;
  const float d_inp = (1.f - inpGate) * inpGate * cellIn * d_c2;
  const float d_fgt = (1.f - fgtGate) * fgtGate * prev_c * d_c2;
  p.Dc0[idx] = fgtGate * d_c2 + dc * (1.f - m);
  const float dx[4] = {E::round(d_cin), E::round(d_inp), E::round(d_fgt), E::round(d_out)};
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    E::store(p.DX, fo + g * n, dx[g]);
    const float old = E::load(p.dx0, io + g * n);
    E::store(p.dx0, io + g * n, dx[g] + old * (1.f - m));
  }
  p.dyw[idx] = dyw * (1.f - m);
}

// dyw[b,k] += sum_j DX[t][b,j] * W[k,j]  (j over the 4n gate columns) on MFMA.  Both operands are contiguous along j
// in memory, which is exactly an MFMA fragment (16 bytes per lane): A = 16 rows of W, B = 16 rows of DX[t].
// One workgroup per 16 values of k and 16*NT batch rows; j dealt round-robin to the 4 wavefronts, partial tiles
// summed through LDS in wave order.  Needs n % 16 == 0.
template <typename AT, int NT>
__global__ __launch_bounds__(kWgThreads) void k_bwd_gemm_dy(Lstm2BwdParams p, long long t) {
  using E = Elem<AT>;
  constexpr int KE = E::KE, KM = E::KM;
  __shared__ f32x4 red[kWaves][NT][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = p.n, n4 = 4 * n;
  const int ktiles = n / 16;
  const int k0 = ((int)blockIdx.x % ktiles) * 16;
  const int b0 = ((int)blockIdx.x / ktiles) * 16 * NT;
  const int S = n4 / KM;
  const AT* Wr = (const AT*)p.W + (size_t)(k0 + (lane & 15)) * n4 + KE * (lane >> 4);
  const AT* Dx = (const AT*)p.DX + (size_t)t * p.B * n4 + KE * (lane >> 4);
  int brow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) brow[nt] = min(b0 + 16 * nt + (lane & 15), p.B - 1);  // rows past B: any row, dropped below
  f32x4 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int s = wave; s < S; s += kWaves) {
    const i32x4 a = *(const i32x4*)(Wr + (size_t)KM * s);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const i32x4 bfrag = *(const i32x4*)(Dx + (size_t)brow[nt] * n4 + (size_t)KM * s);
      acc[nt] = E::mma(a, bfrag, acc[nt]);
    }
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) red[wave][nt][lane] = acc[nt];
  __syncthreads();
  for (int nt = wave; nt < NT; nt += kWaves) {
    f32x4 sum = red[0][nt][lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += red[w][nt][lane];
    const int b = b0 + 16 * nt + (lane & 15);
    if (b < p.B) {
      float* out = p.dyw + (size_t)b * n + k0 + 4 * (lane >> 4);
#pragma unroll
      for (int r = 0; r < 4; ++r) out[r] += sum[r];
    }
  }
}

// The same product for any n: one thread per (b, k), ascending j.
template <typename AT>
__global__ void k_bwd_gemm_dy_generic(Lstm2BwdParams p, long long t) {
  using E = Elem<AT>;
  const long long bn = (long long)p.B * p.n;
  const long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  if (idx >= bn) return;
  const int n = p.n, n4 = 4 * n;
  const long long b = idx / n, k = idx % n;
  float acc = p.dyw[idx];
  const size_t xo = ((size_t)t * p.B + b) * n4, wo = (size_t)k * n4;
  for (int j = 0; j < n4; ++j) acc += E::load(p.DX, xo + j) * E::load(p.W, wo + j);
  p.dyw[idx] = acc;
}

// float32 -> AT copy (the final Dy0).
template <typename AT>
__global__ void k_convert_from_f32(const float* src, void* dst, long long count) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x)
    Elem<AT>::store(dst, i, src[i]);
}

}  // namespace rtn
