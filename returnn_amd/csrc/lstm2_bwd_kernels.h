// gfx950 kernels of the NativeLstm2 gradient op: one launch per visited frame, in reverse processing order
// (returnn/native_op.py:1288-1464, lstm_bwd_kernel :1123-1180).
#pragma once

#include <type_traits>

#include "lstm2_kernels.h"

namespace rtn {

struct Lstm2BwdParams {
  // inputs (device)
  const void* W;      // [n,4n] AT
  const float* c0;    // [B,n]
  const float* mask;  // [T,B]
  const float* C;     // [T,B,n]
  const void* H;      // [T,B,4n] AT, activated gates of the forward pass
  const void* DY;     // [T,B,n] AT, rows ldDY elements apart
  // outputs / working arrays (device)
  void* DX;    // [T,B,4n] AT, rows ldDX elements apart
  float* dyw;  // [B,n]  error flowing into the output of the frame before (working copy of Dy0, float32)
  float* Dc0;  // [B,n]  cell error, worked on in place
  void* dx0;   // [B,4n] AT: DX of each sequence's first processed valid frame
  long long T;
  int B, n;
  int op_flags;  // OpFlags: kOpNoCarry, kOpH0IsCell select the gradient of LstmGenericBase (returnn/native_op.py:430-485)
  int pad_;
  long long ldDY, ldDX;  // row pitch of DY and DX in elements (n and 4n when contiguous); H, C and the mask are contiguous
  const void* Wpk;  // per-frame launches: W in MFMA A-operand order, [n/16][4n/KM][64] fragments of 16 bytes (else null)
};

// W[n,4n] -> fragments in the order the per-frame kernel reads them: tile kt (16 rows of W), macro step s (KM columns),
// lane l holds row 16*kt + l%16, columns KM*s + KE*(l/16) .. +KE.  A wavefront's load of one fragment set is then 1 KB of
// consecutive memory instead of sixteen 64-byte pieces of sixteen rows, which is what lets a launch that uses W once
// read it at memory speed.
template <typename AT>
__global__ void k_bwd_pack_w(const void* __restrict__ W, void* __restrict__ Wpk, int n) {
  constexpr int KE = Elem<AT>::KE, KM = Elem<AT>::KM;
  const int n4 = 4 * n, S = n4 / KM;
  const long long total = (long long)(n / 16) * S * 64;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
    const int l = (int)(i & 63);
    const long long ts = i >> 6;
    const int s = (int)(ts % S);
    const long long kt = ts / S;
    ((i32x4*)Wpk)[i] = *(const i32x4*)((const AT*)W + (size_t)(16 * kt + (l & 15)) * n4 + (size_t)KM * s + KE * (l >> 4));
  }
}

// Gate derivatives of one (sequence, cell) pair in one frame (returnn/native_op.py:1148-1172).
//   h0: first block of H -- tanh(cell-in), or with kOpH0IsCell the cell state, from which tanh(cell-in) is recovered as
//   the reference's gradient kernel does: (state - forget * old_state) / max(input, 1e-16)  (:462-463)
//   err_y, err_c: error of the output and of the cell state, already multiplied by the mask
template <typename AT>
__device__ __forceinline__ float bwd_cell(int op_flags, float h0, float a_in, float a_fg, float a_out, float c_before, float err_y,
                                          float err_c, float (&dx)[4]) {
  using E = Elem<AT>;
  float a_cell, tanh_c;  // tanh(cell-in) and tanh of the frame's cell state
  if (op_flags & kOpH0IsCell) {
    tanh_c = Act<AT>::tanh(h0);
    a_cell = (h0 - a_fg * c_before) / fmaxf(a_in, 1e-16f);
  } else {
    a_cell = h0;
    tanh_c = Act<AT>::tanh(c_before * a_fg + a_cell * a_in);
  }
  const float err_cell = err_c + a_out * err_y * (1.f - tanh_c * tanh_c);  // total error on the frame's cell state
  dx[0] = E::round((1.f - a_cell * a_cell) * a_in * err_cell);
  dx[1] = E::round((1.f - a_in) * a_in * a_cell * err_cell);
  dx[2] = E::round((1.f - a_fg) * a_fg * c_before * err_cell);
  dx[3] = E::round((1.f - a_out) * a_out * tanh_c * err_y);
  return err_cell;
}

// Cell state of the frame before: the forward pass's C, or with kOpH0IsCell the first block of H of that frame.
template <typename AT>
__device__ __forceinline__ float bwd_prev_cell(const Lstm2BwdParams& p, long long prev_t, long long idx, long long io) {
  if (prev_t < 0) return p.c0[idx];
  if (p.op_flags & kOpH0IsCell) return Elem<AT>::load(p.H, prev_t * (long long)p.B * p.n * 4 + io);
  return p.C[prev_t * (long long)p.B * p.n + idx];
}

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
  const long long fo = t * bn * 4 + io;  // inside H
  const long long xo = (t * p.B + b) * p.ldDX + cell;  // inside DX
  const float m = p.mask[t * p.B + b];
  const float dyw = p.dyw[idx];
  const bool raw_dh = (p.op_flags & kOpRawDh) != 0;
  const float dy = E::load(p.DY, (t * p.B + b) * p.ldDY + cell);
  const float err_y = raw_dh ? dy * m + dyw : (dy + dyw) * m;
  const float dc = p.Dc0[idx];
  const float err_c = dc * m;
  const float prev_c = bwd_prev_cell<AT>(p, prev_t, idx, io);
  const float a_fg = E::load(p.H, fo + 2 * n);
  float dx[4];
  const float err_cell = bwd_cell<AT>(p.op_flags, E::load(p.H, fo), E::load(p.H, fo + n), a_fg, E::load(p.H, fo + 3 * n), prev_c, err_y, err_c, dx);
  p.Dc0[idx] = a_fg * err_cell + dc * (1.f - m);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    E::store(p.DX, xo + g * n, dx[g]);
    const float old = E::load(p.dx0, io + g * n);
    E::store(p.dx0, io + g * n, raw_dh ? dx[g] : dx[g] + old * (1.f - m));
  }
  p.dyw[idx] = (p.op_flags & kOpNoCarry) ? 0.f : dyw * (1.f - m);
}

// One launch per visited frame on MFMA shapes (n % 16 == 0): the recurrent GEMM of the frame processed before
// (t_gemm >= 0: dyw[b,k] += sum_j DX[t_gemm][b,j] * W[k,j], j over the 4n gate columns) followed, for the same (b, k)
// pairs, by the pointwise part of frame t (t >= 0; prev_t < 0: the frame before is the initial state).  The last
// launch of a call has t < 0: only the GEMM.
// Both GEMM operands are contiguous along j in memory, which is exactly an MFMA fragment (16 bytes per lane): A = 16
// rows of W, B = 16 rows of DX[t_gemm].  One workgroup per 16 values of k and 16*NT batch rows; j dealt round-robin
// to the 4 wavefronts, partial tiles summed through LDS in wave order.  Every (b, k) pair belongs to exactly one
// workgroup; dyw, Dc0 and dx0 of the pair live in memory between launches.
template <typename AT, int NT>
__global__ __launch_bounds__(kWgThreads) void k_bwd_step(Lstm2BwdParams p, long long t_gemm, long long t, long long prev_t) {
  using E = Elem<AT>;
  constexpr int KE = E::KE, KM = E::KM;
  __shared__ f32x4 red[kWaves][NT][64];
  __shared__ float tile[NT][16][17];  // [nt][b][k] sums of the GEMM, padded against bank conflicts
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = p.n, n4 = 4 * n;
  const int ktiles = n / 16;
  const int k0 = ((int)blockIdx.x % ktiles) * 16;
  const int b0 = ((int)blockIdx.x / ktiles) * 16 * NT;
  // The operands of the pointwise part of the thread's (b, k) pairs do not depend on the GEMM: they are fetched first,
  // so that their latency passes behind it.
  const int pbl = tid >> 4, pkl = tid & 15;
  float q_dyw[NT], q_m[NT], q_dy[NT], q_dc[NT], q_pc[NT], q_h[NT][4], q_dx0[NT][4];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int b = b0 + 16 * nt + pbl, k = k0 + pkl;
    q_dyw[nt] = q_m[nt] = q_dy[nt] = q_dc[nt] = q_pc[nt] = 0.f;
#pragma unroll
    for (int g = 0; g < 4; ++g) q_h[nt][g] = q_dx0[nt][g] = 0.f;
    if (b >= p.B) continue;
    const long long idx = (long long)b * n + k;
    q_dyw[nt] = p.dyw[idx];
    if (t >= 0) {
      const long long bn = (long long)p.B * n;
      const long long io = (long long)b * n4 + k;
      const long long fo = t * bn * 4 + io;
      q_m[nt] = p.mask[t * p.B + b];
      q_dy[nt] = E::load(p.DY, (t * p.B + b) * p.ldDY + k);
      q_dc[nt] = p.Dc0[idx];
      q_pc[nt] = bwd_prev_cell<AT>(p, prev_t, idx, io);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        q_h[nt][g] = E::load(p.H, fo + g * n);
        q_dx0[nt][g] = E::load(p.dx0, io + g * n);
      }
    }
  }
  if (t_gemm >= 0) {
    const int S = n4 / KM;
    const AT* Wr = (const AT*)p.W + (size_t)(k0 + (lane & 15)) * n4 + KE * (lane >> 4);
    const i32x4* Wk = p.Wpk ? (const i32x4*)p.Wpk + (size_t)(k0 / 16) * S * 64 + lane : nullptr;  // packed: fragment s at Wk[64 * s]
    const AT* Dx = (const AT*)p.DX + (size_t)t_gemm * p.B * p.ldDX + KE * (lane >> 4);
    int brow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) brow[nt] = min(b0 + 16 * nt + (lane & 15), p.B - 1);  // rows past B: any row, dropped below
    f32x4 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    // U macro steps at a time: all their loads are issued before the first MFMA, so the memory latency is paid once
    // per chunk and not once per macro step.
    constexpr int U = 8;
    for (int s0 = wave; s0 < S; s0 += kWaves * U) {
      i32x4 a[U], bfrag[U][NT];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int s = min(s0 + kWaves * u, S - 1);  // past the end: a valid address, the product is dropped
        a[u] = Wk ? Wk[(size_t)64 * s] : *(const i32x4*)(Wr + (size_t)KM * s);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) bfrag[u][nt] = *(const i32x4*)(Dx + (size_t)brow[nt] * p.ldDX + (size_t)KM * s);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (s0 + kWaves * u < S) {
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) acc[nt] = E::mma(a[u], bfrag[u][nt], acc[nt]);
        }
      }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) red[wave][nt][lane] = acc[nt];
    __syncthreads();
    for (int nt = wave; nt < NT; nt += kWaves) {
      f32x4 sum = red[0][nt][lane];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) sum += red[w][nt][lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) tile[nt][lane & 15][4 * (lane >> 4) + r] = sum[r];
    }
    __syncthreads();
  }
  // the (b, k) pairs of the tile, one or NT per thread
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int bl = pbl, kl = pkl;
    const int b = b0 + 16 * nt + bl, k = k0 + kl;
    if (b >= p.B) continue;
    const long long idx = (long long)b * n + k;
    float dyw = q_dyw[nt];
    if (t_gemm >= 0) dyw += tile[nt][bl][kl];
    if (t >= 0) {
      const long long io = (long long)b * n4 + k;
      const long long xo = (t * p.B + b) * p.ldDX + k;
      const float m = q_m[nt];
      const bool raw_dh = (p.op_flags & kOpRawDh) != 0;
      const float err_y = raw_dh ? q_dy[nt] * m + dyw : (q_dy[nt] + dyw) * m;
      const float dc = q_dc[nt];
      const float err_c = dc * m;
      const float a_fg = q_h[nt][2];
      float dx[4];
      const float err_cell = bwd_cell<AT>(p.op_flags, q_h[nt][0], q_h[nt][1], a_fg, q_h[nt][3], q_pc[nt], err_y, err_c, dx);
      p.Dc0[idx] = a_fg * err_cell + dc * (1.f - m);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        E::store(p.DX, xo + g * n, dx[g]);
        E::store(p.dx0, io + g * n, raw_dh ? dx[g] : dx[g] + q_dx0[nt][g] * (1.f - m));
      }
      dyw = (p.op_flags & kOpNoCarry) ? 0.f : dyw * (1.f - m);
    }
    p.dyw[idx] = dyw;
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
  const size_t xo = ((size_t)t * p.B + b) * p.ldDX, wo = (size_t)k * n4;
  for (int j = 0; j < n4; ++j) acc += E::load(p.DX, xo + j) * E::load(p.W, wo + j);
  p.dyw[idx] = acc;
}

// float32 -> AT copy (the final Dy0).
template <typename AT>
__global__ void k_convert_from_f32(const float* src, void* dst, long long count) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x)
    Elem<AT>::store(dst, i, src[i]);
}


// ---------------------------------------------------------------------------------------------------------------
// Persistent gradient kernel: all frames in one cooperative launch, W on chip for the whole call.
//
//  * decomposition: `groups` batch groups of up to 16 rows; inside a group, workgroup r owns 16*MT values of k: the
//    rows k of W (A operand of  d_h[b,k] = sum_j DX[b,j] W[k,j],  16*MT x 4n values, in registers for the whole call:
//    wavefront w holds the macro steps [w*ksb, (w+1)*ksb) of j, ksb <= KSB) and, in the pointwise part, the cells k of its rows.
//    What a workgroup has to read per frame (rows x 4n values) is what its step time grows with -- a CU gets
//    device-scope loads at only about 36 GB/s -- so the groups are made small (8 rows) when the device has the CUs.
//  * exchange: a ring of kExRing frames per group in the workspace, in MFMA B-operand order ([4n/KM macro steps][4 lane
//    groups][Bp rows][16 bytes], Bp = 8 or 16): a wavefront's load of a fragment is contiguous memory, whole cache lines
//    (reading DX itself, row-major, made every lane's 16 bytes a request of its own and bound the frame time by the
//    requests a CU can have in flight).  The host fills the ring with all-ones words (a NaN pattern no result can have:
//    NaNs are canonicalised); a workgroup stages the gate derivatives of its cells in LDS in that order and writes them
//    with 16-byte stores: to the ring slot of the frame, to DX (row-major, the op's output, a plain stream), and all-ones
//    again to the slot that was read two frames ago (every workgroup of the group is past it: they all delivered the
//    frame processed before, which they could only do after reading that slot).  Readers load their share of the
//    frame's slot as B fragments and read again until no element is all-ones.  With the group on one XCD (checked at
//    the start, see group_on_one_xcd) the ring's stores are plain and the data goes from writer to readers through that
//    XCD's L2; else stores and loads are device-scope.
//  * per frame: wait for DX of the frame processed before, MFMA, sum of the 4 partial tiles through LDS, the
//    pointwise part of this frame (inputs H, DY, C, mask fetched one frame ahead), DX out, first read of the
//    next wait after an adaptive delay.  The cell error, the output error carried on and dx0 stay in registers.
//  * all waits are bounded as in the forward kernel (status[0] = 1, everybody leaves).
struct Lstm2BwdPersistent {
  Lstm2BwdParams p;
  const float* Dd;    // [B,n]
  void* Dy0;          // [B,n] AT, out
  unsigned* status;   // [0] != 0: a bounded wait expired
  long long t_end;    // first frame processed (the last one the forward pass visited)
  int step;           // the forward pass's signed stride; frames are processed t_end, t_end - step, ...
  int nframes;        // number of visited frames
  int groups, Bg;     // batch groups of this launch and rows per group (<= 16)
  int group_offset;   // index of the launch's first group (a large batch runs as several launches in turn)
  int ksb;            // macro steps of the contraction per wavefront (<= the kernel's KSB; the rest of its slots stay empty)
  int poll_delay, delay_inc, delay_dec_mask;
  unsigned long long timeout_ticks;
  unsigned* sync;     // [2 * groups of the whole problem] words of the XCD check (cleared before the launch)
  void* ex;           // [groups of the whole problem][kExRing][4n * Bp] AT: the exchange ring (all-ones before the launch)
  int Bp, bp_shift;   // rows of a ring frame: 8 or 16 (= 1 << bp_shift), >= Bg
};
constexpr int kExRing = 4;

// Optional instrumentation (-DRTN_LSTM2_TRACE): thread 0 of every workgroup accumulates shader-clock ticks per phase
// of the persistent gradient kernel into a device array that rtn_debug_bwd_trace() copies out.
#ifdef RTN_LSTM2_TRACE
__device__ unsigned long long g_bwd_trace[1024 * 8];
#define RTN_BTRACE_DECL unsigned long long bt_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}; unsigned long long bt_last = clock64();
#define RTN_BTRACE_MARK(k) { const unsigned long long bt_now = clock64(); bt_acc[k] += bt_now - bt_last; bt_last = bt_now; }
#define RTN_BTRACE_ADD(k, v) { bt_acc[k] += (v); }
#define RTN_BTRACE_FLUSH() if (threadIdx.x == 0 && blockIdx.x < 1024) { for (int k = 0; k < 8; ++k) g_bwd_trace[(size_t)blockIdx.x * 8 + k] = bt_acc[k]; }
#else
#define RTN_BTRACE_DECL
#define RTN_BTRACE_MARK(k)
#define RTN_BTRACE_ADD(k, v)
#define RTN_BTRACE_FLUSH()
#endif

// Several gradient problems of one shape in one launch (the two directions of a bidirectional layer):
// workgroup id / wgs_each picks the problem, the remainder is the workgroup's id inside it.
constexpr int kMaxBwdMulti = 2;
struct Lstm2BwdMulti {
  int count;     // problems, 1..kMaxBwdMulti
  int wgs_each;  // workgroups per problem = groups * n / (16 * MT)
  int local;     // 1: every batch group sits on one XCD (workgroup id = slot * xcds + xcd; the groups of the launch, all
                 // problems counted through, are dealt round-robin to the XCDs)
  int xcds;      // XCDs the workgroup ids are dealt to (local plans)
  Lstm2BwdPersistent q[kMaxBwdMulti];
};

// WV wavefronts per workgroup (4, 8 or 16) share the contraction range: a CU moves more bytes per microsecond at device
// scope the more wavefronts have loads in flight, and with 8 or more each wavefront's share of W and of the frame's DX
// fits the ordinary registers.  The 256 (row, k) pairs of a tile belong to the threads with the same tid % 256; thread
// set tid / 256 takes the tiles set, set + WV/4, ...
//
// KSL > 0: a wavefront's share of W is KSB fragments in registers plus KSL fragments in LDS (dynamic shared memory,
// WV * KSL * 1024 bytes), for layers whose slice of W does not fit the registers next to a frame's DX.
//
// HALF (ring frames of 8 rows): a fragment of 8 rows fills only half of the 16 lanes per lane group, and what limits the
// loads of a frame is the number of load instructions (each returns 1 KB to the registers, used or not).  So one load
// takes two macro steps at once: the lanes of rows 0-7 read macro step 2a, the lanes of "rows" 8-15 read the same rows of
// macro step 2a+1 -- 1 KB of consecutive memory.  As a B operand that register is right in columns 0-7 for the A
// fragment of step 2a and right in columns 8-15 for the A fragment of step 2a+1: two MFMAs on the same register into two
// accumulators, the first valid in columns 0-7, the second in columns 8-15, which are added when the partial tiles of
// the wavefronts are.  Same number of MFMAs, half the load instructions, no data movement.
template <typename AT, int KSB, int MT, int WV, int KSL = 0, bool HALF = false>
__global__ __launch_bounds__(64 * WV) void k_lstm2_bwd_regw(const Lstm2BwdMulti multi) {
  static_assert(!HALF || KSL == 0, "the paired loads are not written for the chunked variants");
  constexpr int KST = KSB + KSL;           // fragment slots of a wavefront
  constexpr int TS = WV / 4;               // thread sets of 256
  // tiles whose pairs a thread keeps.  A set of 256 threads covers 16 rows x 16 values of k; with at most 8 rows the
  // threads of the upper 8 row slots take every other tile instead of idling (SPLIT), which halves the pairs, the loads
  // and the pointwise work per thread.
  constexpr bool SPLIT = HALF && ((MT + TS - 1) / TS) % 2 == 0;
  constexpr int PT = SPLIT ? (MT + TS - 1) / TS / 2 : (MT + TS - 1) / TS;
  int which, bid;
  if (multi.local) {
    const int kb = multi.q[0].p.n / (16 * MT), groups_now = multi.q[0].groups;
    const int xcd = (int)blockIdx.x % multi.xcds, slot = (int)blockIdx.x / multi.xcds;
    const int gg = (slot / kb) * multi.xcds + xcd;  // group of the launch, all problems counted through
    which = gg / groups_now;
    bid = (gg - which * groups_now) * kb + slot % kb;
  } else {
    which = (int)blockIdx.x / multi.wgs_each;
    bid = (int)blockIdx.x - which * multi.wgs_each;
  }
  if (which >= multi.count) return;
  const Lstm2BwdPersistent q = multi.q[which];
  using E = Elem<AT>;
  using SN = Sentinel<AT>;
  using LM = LaneMax<AT>;
  constexpr int KE = E::KE, KM = E::KM, ES = (int)sizeof(AT);
  const Lstm2BwdParams& p = q.p;
  // partial tiles of the wavefronts; a lane group's 16 entries are followed by 4 unused ones, so that the four groups of
  // k that a wavefront's threads read together start 16 banks apart (without the gap they met in the same banks)
  constexpr int kRedGroup = 20;
  // (two copies where they are small, frames alternate: no barrier then between the sums of one frame and the partial
  // tiles of the next)
  constexpr int kRedCopies = (WV * MT * 4 * kRedGroup * 16 <= 24 * 1024) ? 2 : 1;
  __shared__ f32x4 red2[kRedCopies][WV][MT][4 * kRedGroup];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // 0..WV-1
  const int n = p.n, n4 = 4 * n;
  const int kblocks = n / (16 * MT);  // workgroups per group; each owns MT tiles of 16 values of k
  const int g = q.group_offset + bid / kblocks, k0 = (bid % kblocks) * 16 * MT;
  const int b_base = g * q.Bg;
  const int rows = min(q.Bg, p.B - b_base);
  const long long bn = (long long)p.B * n;
  const unsigned frame_bytes = (unsigned)((size_t)p.B * n4 * ES);
  const unsigned dx_frame_bytes = (unsigned)((size_t)p.B * p.ldDX * ES);
  const long long dy_frame = (long long)p.B * p.ldDY;  // elements from one frame of DY to the next
  // the exchange ring of this group: kExRing frames of [4n/KM][4][Bp][16 bytes]
  const int Bp = q.Bp;
  const unsigned ex_frame = (unsigned)((size_t)n4 * Bp * ES), frag_stride = (unsigned)(64 * Bp);
  unsigned char* const ex_base = (unsigned char*)q.ex + (size_t)g * kExRing * ex_frame;
  constexpr int KGW = 16 * MT / KE;  // 16-byte pieces per row and gate that this workgroup produces
  __shared__ i32x4 stage[4 * KGW * 16];  // [gate][piece][row]: the workgroup's derivatives of a frame in ring order

  // An XCD-local plan rests on all workgroups of a group being on one XCD: checked here.
  __shared__ int s_local;
  if (tid == 0) s_local = multi.local ? (int)group_on_one_xcd(q.sync + 2 * (size_t)g, (unsigned)kblocks, q.status, q.timeout_ticks) : 0;
  __syncthreads();
  const bool local = s_local != 0;

  // A fragments: this wavefront's macro steps [wave*ksb, (wave+1)*ksb) of the 16*MT rows of W, as far as the 4n/KM macro
  // steps reach.  Slots beyond them hold zeros in W and read nothing (or, in the chunked variants, a fragment that is
  // multiplied by that zero), so that any width whose share per wavefront is at most KSB + KSL runs on this kernel.
  const int ksb = q.ksb;
  const int ks_here = max(0, min(ksb, n4 / KM - ksb * wave));  // uniform over the wavefront
  const int ks_last = max(ks_here, 1) - 1;
  const int wave_at = (KSL > 0 && ks_here == 0) ? 0 : wave;  // chunked variants: a wavefront without a share reads the first one's
  i32x4 wreg[MT][KSB];
  extern __shared__ __align__(16) unsigned char bwd_smem[];
  i32x4* wl = (i32x4*)bwd_smem + (size_t)wave * (KSL > 0 ? KSL : 1) * 64 + lane;  // [WV][KSL][64]: slot s of this lane at wl[s * 64]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const AT* Wr = (const AT*)p.W + (size_t)(k0 + 16 * mt + (lane & 15)) * n4 + (size_t)KM * ksb * wave + KE * (lane >> 4);
#pragma unroll
    for (int ks = 0; ks < KSB; ++ks) wreg[mt][ks] = (ks < ks_here) ? *(const i32x4*)(Wr + (size_t)KM * ks) : i32x4{0, 0, 0, 0};
    if constexpr (KSL > 0) {
      static_assert(KSL == 0 || MT == 1, "the LDS part of W is laid out for one tile per workgroup");
#pragma unroll
      for (int ks = KSB; ks < KST; ++ks) wl[(ks - KSB) * 64] = (ks < ks_here) ? *(const i32x4*)(Wr + (size_t)KM * ks) : i32x4{0, 0, 0, 0};
    }
  }
  // byte offset of this lane's first B fragment inside a ring frame; the others follow at frag_stride bytes each.  The
  // lanes of rows the group lacks carry an out-of-range offset: their loads return 0.
  const int lane_row = HALF ? (lane & 7) : (lane & 15), lane_hi = HALF ? ((lane >> 3) & 1) : 0;  // HALF: lanes 8-15 of a lane group take the next macro step
  const unsigned foff0 = (lane_row < rows) ? (unsigned)(ksb * wave_at + lane_hi) * frag_stride + (unsigned)(((lane >> 4) * Bp + lane_row) * 16) : 0x80000000u;

  // The (row, k) pairs of this thread: one in each of its tiles.
  const int set = (TS == 1) ? 0 : __builtin_amdgcn_readfirstlane(tid >> 8);  // uniform over a wavefront
  const int kl = tid & 15;
  const int bl = SPLIT ? ((tid & 127) >> 4) : ((tid & 255) >> 4);  // row slot
  const int upper = SPLIT ? ((tid & 255) >> 7) : 0;                // SPLIT: which of a pair of tiles
  auto tile_of = [&](int j) { return SPLIT ? set + TS * (2 * j + upper) : set + TS * j; };
  const int b = b_base + ((bl < rows) ? bl : 0);
  const long long dy_row = (long long)b * (p.ldDY - n);  // element idx = b*n + k of a contiguous array sits at dy_row + idx in DY
  bool act[PT];  // the pair exists: the tile does, and the group has the row
  long long idx[PT], io[PT];
  float dyw[PT], dc[PT], dx0[PT][4];
#pragma unroll
  for (int j = 0; j < PT; ++j) {
    const int mt = tile_of(j);
    act[j] = (mt < MT) && (bl < rows);
    const int k = k0 + 16 * ((mt < MT) ? mt : 0) + kl;
    idx[j] = (long long)b * n + k;
    io[j] = (long long)b * n4 + k;
    dyw[j] = 0.f;
    dc[j] = act[j] ? q.Dd[idx[j]] : 0.f;
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) dx0[j][gq] = 0.f;
  }
  // where a pair's element of the summed tile is: tile element D[kl][bl] sits in lane (kl/4)*16 + bl, component kl%4
  const int red_lane = (kl >> 2) * kRedGroup + (HALF ? (bl & 7) : bl), red_comp = kl & 3;

  // Inputs of a frame, fetched one frame ahead.  No branches around the loads and no arithmetic on what they bring: a
  // register that receives its value on two paths, or feeds an instruction, makes the compiler wait for every load in
  // flight at that point -- here that would be a memory latency in front of the ring's loads, every frame.  The cell
  // state of the frame before is c0, C or (kOpH0IsCell) the first block of H: both sources are read, the one that does
  // not apply through a descriptor of no bytes (no memory access, 0 comes back), and added where they are used.
  float in_gate[PT][4], in_dy[PT], in_m;
  unsigned in_pc[PT], in_ph[PT];
  // the frame after, on its way: as the loads bring it (a conversion next to the loads would be scheduled among the
  // MFMAs and wait there for memory)
  typedef typename std::conditional<ES == 2, unsigned short, unsigned>::type RawT;
  unsigned nx_gate[PT][4], nx_dy[PT], nx_pc[PT], nx_ph[PT];
  float nx_m;
  auto widen = [](unsigned raw) {
    if constexpr (ES == 2)
      return __builtin_bit_cast(float, raw << 16);
    else
      return __builtin_bit_cast(float, raw);
  };
  auto fetch = [&](long long t, long long prev_t) {
    const bool from_h = (p.op_flags & kOpH0IsCell) != 0 && prev_t >= 0;
    const float* csrc = prev_t < 0 ? p.c0 : p.C + prev_t * bn;
    __amdgpu_buffer_rsrc_t rs_c = __builtin_amdgcn_make_buffer_rsrc((void*)csrc, 0, from_h ? 0u : (unsigned)(bn * 4), kBufFlags);
    __amdgpu_buffer_rsrc_t rs_ph = __builtin_amdgcn_make_buffer_rsrc((unsigned char*)p.H + (size_t)(prev_t < 0 ? 0 : prev_t) * frame_bytes, 0,
                                                                     from_h ? frame_bytes : 0u, kBufFlags);
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const long long fo = t * bn * 4 + io[j];
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) nx_gate[j][gq] = ((const RawT*)p.H)[fo + (long long)gq * n];
      nx_dy[j] = ((const RawT*)p.DY)[dy_frame * t + dy_row + idx[j]];
      nx_pc[j] = __builtin_amdgcn_raw_buffer_load_b32(rs_c, (unsigned)(idx[j] * 4), 0, 0);
      if constexpr (ES == 2)
        nx_ph[j] = __builtin_amdgcn_raw_buffer_load_b16(rs_ph, (unsigned)(io[j] * ES), 0, 0);
      else
        nx_ph[j] = __builtin_amdgcn_raw_buffer_load_b32(rs_ph, (unsigned)(io[j] * ES), 0, 0);
    }
    nx_m = p.mask[t * p.B + b];
  };
  auto take_next = [&]() {  // what fetch() asked for becomes the current frame's inputs
#pragma unroll
    for (int j = 0; j < PT; ++j) {
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) in_gate[j][gq] = widen(nx_gate[j][gq]);
      in_dy[j] = widen(nx_dy[j]);
      in_pc[j] = nx_pc[j];
      in_ph[j] = nx_ph[j];
    }
    in_m = nx_m;
  };
  auto prev_cell = [&](int j) {
    float vh;
    if constexpr (ES == 2)
      vh = (float)__builtin_bit_cast(AT, (unsigned short)in_ph[j]);
    else
      vh = __builtin_bit_cast(float, in_ph[j]);
    return __builtin_bit_cast(float, in_pc[j]) + vh;
  };
  const int F = q.nframes;
  // EARLY: a frame's inputs are asked for two frames ahead, in front of the MFMAs (see gemm); otherwise one frame ahead,
  // at the end of a frame.  (Measured: the kernels that keep one pair per thread gain 4 % from EARLY, the others lose.)
  constexpr bool EARLY = SPLIT;
  auto frame = [&](int f) { return q.t_end - (long long)f * q.step; };

  // The B fragments of a frame (the group's rows of DX, this wavefront's share of the contraction range) are taken in
  // chunks of CH: up to 32 fragments in one go; a wider share (KSL > 0) in chunks of 16 (8 with 8 wavefronts, which have
  // half the registers each) through two sets of registers: the next chunk is in flight while the matrix cores work on
  // this one.
  constexpr int CH = KSL == 0 ? KST : (WV >= 8 ? 8 : 16);
  constexpr int NCH = KST / CH;
  constexpr int NB = HALF ? CH / 2 : CH;  // registers of B fragments per chunk
  static_assert(!HALF || CH % 2 == 0, "paired loads need an even number of macro steps");
  i32x4 bf[NCH > 1 ? 2 : 1][NB];
  auto issue_chunk = [&](int f, int c, int slot) {  // f: ordinal of the frame whose derivatives are wanted
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(ex_base + (size_t)(f & (kExRing - 1)) * ex_frame, 0, ex_frame, kBufFlags);
    asm volatile("" ::: "memory");  // other workgroups write this memory: really load again
    if constexpr (NCH == 1) {
      // an unused slot carries an out-of-range offset: 0 comes back and no memory is touched (the offsets stay in
      // registers over the frames, which measured faster than instruction immediates)
      if constexpr (HALF) {
#pragma unroll
        for (int a = 0; a < NB; ++a)  // (an odd share: the upper lanes of its last pair read a macro step that meets zeros in W)
          bf[slot][a] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (2 * a < ks_here) ? foff0 : 0x80000000u, (2 * a) * (int)frag_stride, kAuxDevice));
      } else {
#pragma unroll
        for (int ks = 0; ks < CH; ++ks)
          bf[slot][ks] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (ks < ks_here) ? foff0 + (unsigned)ks * frag_stride : 0x80000000u, 0, kAuxDevice));
      }
    } else {
      // 64 offsets would not fit the registers: an unused slot reads the wavefront's last used fragment again (complete
      // when the used ones are, and multiplied by zero); worked out again for every chunk
      int last = ks_last;
      asm volatile("" : "+s"(last));
#pragma unroll
      for (int ks = 0; ks < CH; ++ks)
        bf[slot][ks] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, foff0, min(c * CH + ks, last) * (int)frag_stride, kAuxDevice));
    }
  };
  auto issue = [&](int f) { issue_chunk(f, 0, 0); };
  // (A group that was planned for one XCD and found itself on several takes the adaptive delay of a spread plan.)
  const bool spread_after_all = multi.local && !local;
  int delay = spread_after_all ? 20 : q.poll_delay;
  const int delay_inc = spread_after_all ? 2 : q.delay_inc;
  bool aborted = false;
  // d_h of the thread's pairs from DX of frame t (whose first read has been issued): wait, MFMA, sum over the
  // wavefronts; added to dyw.
  RTN_BTRACE_DECL
  auto gemm = [&](int t) {  // t: ordinal of the frame whose derivatives go through the product
    RTN_BTRACE_MARK(4)  // pointwise tail, fetch, delay, first read
    auto& red = red2[kRedCopies == 2 ? (t & 1) : 0];
    // independent partial sums keep the MFMA pipeline full (one chain would wait for every result)
    constexpr int NACC = HALF ? 2 : ((MT >= 4 || KSB < 2) ? 1 : (MT == 2 || KSB < 4 ? 2 : 4));
    f32x4 part[MT][NACC];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int slot = c & 1;
      unsigned long long t0 = 0;
      unsigned spins = 0;
      for (;;) {
        // (four independent running maxima: one chain of dependent packed operations needs a wait state after every
        // one of them, and there are up to 128 of them here)
        unsigned mw[4] = {0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < NB; ++ks)
#pragma unroll
          for (int w = 0; w < 4; ++w) mw[w] = LM::fold(mw[w], (unsigned)bf[slot][ks][w]);
        const unsigned m = LM::fold(LM::fold(mw[0], mw[1]), LM::fold(mw[2], mw[3]));
        if (!__any(LM::has_sentinel(m))) break;
        if ((spins++ & 15u) == 0) {
          if (__hip_atomic_load(q.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { aborted = true; break; }
          const unsigned long long now = wall_clock64();
          if (spins == 1) {
            t0 = now;
          } else if (now - t0 > q.timeout_ticks) {
            __hip_atomic_store(q.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            aborted = true;
            break;
          }
        }
        issue_chunk(t, c, slot);
      }
      if (c == 0) {
        RTN_BTRACE_MARK(0)  // wait for the frame's DX
        RTN_BTRACE_ADD(6, spins)
        // (as in the forward kernel: an adaptive delay across XCDs, one number for all within an XCD)
        if (spins)
          delay = min(delay + delay_inc, 64);
        else if (delay_inc && delay > 0)
          delay -= ((t & q.delay_dec_mask) == q.delay_dec_mask) ? 1 : 0;
        // W lives in accumulation registers where it is at most half of that file: the B fragments fill up to half of
        // the ordinary registers, and a matrix instruction reads an A operand from either file (without this the compiler
        // parks part of W there anyway and copies four registers back in front of every MFMA, which halves the MFMA rate).
        if constexpr (MT * KSB <= 32) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int ks = 0; ks < KSB; ++ks) asm volatile("" : "+a"(wreg[mt][ks]));
        }
      }
      if (c + 1 < NCH) issue_chunk(t, c + 1, slot ^ 1);
      if (c == 0) {
        // The inputs of the frame after next's pointwise part (frame t + 2: frame t + 1's are in registers already), asked
        // for here, behind the wait for the ring and in front of the MFMAs: a wavefront's loads count as returned in
        // the order they were issued, so loads from memory issued in front of the ring's loads (as they were, at the
        // end of a frame) made the wait for the ring a wait for memory.
        if constexpr (EARLY) {
          const int fn = min(t + 2, F - 1);  // (past the end: the last frame's again, unused)
          fetch(frame(fn), fn + 1 < F ? frame(fn + 1) : -1);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int a = 0; a < NACC; ++a) part[mt][a] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      if constexpr (HALF) {
#pragma unroll
        for (int a = 0; a < NB; ++a)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            part[mt][0] = E::mma(wreg[mt][2 * a], bf[slot][a], part[mt][0]);      // valid in columns 0-7
            part[mt][1] = E::mma(wreg[mt][2 * a + 1], bf[slot][a], part[mt][1]);  // valid in columns 8-15
          }
      } else {
#pragma unroll
        for (int ks = 0; ks < CH; ++ks)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const int s_ = c * CH + ks;
            const i32x4 a = (s_ < KSB) ? wreg[mt][s_ < KSB ? s_ : 0] : wl[(s_ - KSB) * 64];
            part[mt][ks % NACC] = E::mma(a, bf[slot][ks], part[mt][ks % NACC]);
          }
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x4 acc = part[mt][0];
      if constexpr (HALF) {
        // each column keeps the accumulator that is valid there (component by component: a select of whole vectors is
        // compiled into an indexed read of a stack array)
        const bool upper = (lane & 8) != 0;
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = upper ? part[mt][1][r] : part[mt][0][r];
      } else {
#pragma unroll
        for (int a = 1; a < NACC; ++a) acc += part[mt][a];
      }
      red[wave][mt][(lane >> 4) * kRedGroup + (lane & 15)] = acc;
    }
    RTN_BTRACE_MARK(1)  // MFMA, partial tiles to LDS
    __syncthreads();
    RTN_BTRACE_MARK(2)  // barrier
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const int mt = (tile_of(j) < MT) ? tile_of(j) : 0;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < WV; ++w) {
        sum += ((const float*)&red[w][mt][red_lane])[red_comp];
        if constexpr (HALF) sum += ((const float*)&red[w][mt][red_lane + 8])[red_comp];
      }
      dyw[j] += sum;
    }
    // (With two copies this copy of `red` is written again two frames from now, behind that frame's staging barrier and
    // the next frame's barrier above; `stage` is written again behind the barrier above.)
    if constexpr (kRedCopies == 1) __syncthreads();  // red is free for the next frame
    RTN_BTRACE_MARK(3)  // sum over the wavefronts
  };

  const bool raw_dh = (p.op_flags & kOpRawDh) != 0;
  const int bp_shift = q.bp_shift, pieces = (4 * KGW) << bp_shift;
  const i32x4 ones = i32x4{-1, -1, -1, -1};
  fetch(frame(0), F > 1 ? frame(1) : -1);
  if constexpr (EARLY) {
    take_next();
    const int f1 = min(1, F - 1);
    fetch(frame(f1), f1 + 1 < F ? frame(f1 + 1) : -1);
  }
  for (int f = 0; f < F; ++f) {
    const long long t = frame(f);
    if (f > 0) gemm(f - 1);
    if constexpr (!EARLY) take_next();  // (asked for at the end of the frame before, or before the loop)
    // pointwise part of frame t (returnn/native_op.py:1123-1180)
    const float m = in_m;
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const float err_y = raw_dh ? in_dy[j] * m + dyw[j] : (in_dy[j] + dyw[j]) * m;
      const float err_c = dc[j] * m;
      const float a_fg = in_gate[j][2];
      float dx[4];
      const float err_cell = bwd_cell<AT>(p.op_flags, in_gate[j][0], in_gate[j][1], a_fg, in_gate[j][3], prev_cell(j), err_y, err_c, dx);
      dc[j] = a_fg * err_cell + dc[j] * (1.f - m);
      const int mt = tile_of(j);
      if (mt < MT && bl < Bp) {
        const int col = 16 * mt + kl;
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const int at = (((gq * KGW + col / KE) << bp_shift) + bl) * KE + col % KE;  // element index inside `stage`
          if constexpr (ES == 2)
            ((unsigned short*)stage)[at] = (unsigned short)SN::bits(dx[gq]);
          else
            ((unsigned*)stage)[at] = SN::bits(dx[gq]);
        }
      }
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) dx0[j][gq] = raw_dh ? dx[gq] : dx[gq] + dx0[j][gq] * (1.f - m);
      dyw[j] = (p.op_flags & kOpNoCarry) ? 0.f : dyw[j] * (1.f - m);
    }
    __syncthreads();  // the frame's derivatives of this workgroup are staged
    {
      __amdgpu_buffer_rsrc_t rs_out = __builtin_amdgcn_make_buffer_rsrc(ex_base + (size_t)(f & (kExRing - 1)) * ex_frame, 0, ex_frame, kBufFlags);
      __amdgpu_buffer_rsrc_t rs_arm = __builtin_amdgcn_make_buffer_rsrc(ex_base + (size_t)((f + 2) & (kExRing - 1)) * ex_frame, 0, ex_frame, kBufFlags);
      __amdgpu_buffer_rsrc_t rs_dx = __builtin_amdgcn_make_buffer_rsrc((unsigned char*)p.DX + (size_t)t * dx_frame_bytes, 0, dx_frame_bytes, kBufFlags);
      for (int c = tid; c < pieces; c += 64 * WV) {
        const int row = c & (Bp - 1), cg = c >> bp_shift;  // cg = gate * KGW + piece
        const int gate = cg / KGW, piece = cg - gate * KGW;
        if (row < rows) {
          const u32x4 v = __builtin_bit_cast(u32x4, stage[c]);
          const unsigned eo = (unsigned)(((((gate * n + k0) / KE + piece) << bp_shift) + row) * 16);
          const unsigned dxo = (unsigned)(((size_t)(b_base + row) * p.ldDX + (size_t)gate * n + k0 + piece * KE) * ES);
          if (local) {
            __builtin_amdgcn_raw_buffer_store_b128(v, rs_out, eo, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, ones), rs_arm, eo, 0, 0);
          } else {
            __builtin_amdgcn_raw_buffer_store_b128(v, rs_out, eo, 0, kAuxDevice);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, ones), rs_arm, eo, 0, kAuxDevice);
          }
          __builtin_amdgcn_raw_buffer_store_b128(v, rs_dx, dxo, 0, 0);  // the op's output: a plain stream
        }
      }
    }
    RTN_BTRACE_MARK(5)  // pointwise part, staging, stores
    // while the derivatives travel: the inputs of the next frame, then the first read of this frame's ring slot
    if constexpr (EARLY) {
      take_next();  // (asked for in front of the MFMAs of this frame's product, or before the loop)
    } else {
      const int fn = min(f + 1, F - 1);  // (past the end: the last frame's again, unused)
      fetch(frame(fn), fn + 1 < F ? frame(fn + 1) : -1);
    }
    if (!aborted)
      for (int d = 0; d < delay; ++d) __builtin_amdgcn_s_sleep(1);
    issue(f);
  }
  gemm(F - 1);
  RTN_BTRACE_ADD(7, (unsigned long long)delay)
  RTN_BTRACE_FLUSH()
  // After a wait that ran into its bound the gradients are wrong without looking it: the workgroups that see the mark
  // hand out NaN, so that a caller who never asks for the status still finds a non-finite gradient.
  const bool expired = wait_expired(q.status);
  const float nan = __builtin_nanf("");
#pragma unroll
  for (int j = 0; j < PT; ++j) {
    if (act[j]) {
      E::store(q.Dy0, idx[j], expired ? nan : dyw[j]);
      p.Dc0[idx[j]] = expired ? nan : dc[j];
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) E::store(p.dx0, io[j] + (long long)gq * n, expired ? nan : dx0[j][gq]);
    }
  }
}

// Frames the forward pass did not visit: DX = 0.  Rows of row_words 32-bit words, pitch_words apart, rows_per_frame
// rows to a frame; nothing between the rows is touched.
template <typename AT>
__global__ void k_bwd_zero_unvisited(void* DX, long long T, long long rows_per_frame, long long row_words, long long pitch_words,
                                     long long first, long long step, long long nframes) {
  const long long lo = step > 0 ? first : first + (nframes - 1) * step;
  const long long astep = step > 0 ? step : -step;
  unsigned* w = (unsigned*)DX;
  const long long frame_words = rows_per_frame * row_words;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < T * frame_words; i += (long long)gridDim.x * blockDim.x) {
    const long long t = i / frame_words;
    const bool visited = t >= lo && t <= lo + (nframes - 1) * astep && ((t - lo) % astep) == 0;
    if (!visited) {
      const long long r = i / row_words, c = i - r * row_words;
      w[r * pitch_words + c] = 0u;
    }
  }
}

// LstmLowMem gradient: the gates of every frame again from their pre-activations (returnn/native_op.py:683-687):
// data[r, :] (rows of 4n) := [tanh, sigmoid, sigmoid, sigmoid](data[r, :] + bias), in place.
template <typename AT>
__global__ void k_low_mem_gates(void* data, const void* bias, long long rows, int n) {
  using E = Elem<AT>;
  const long long total = rows * 4 * n;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
    const int col = (int)(i % (4 * n));
    const float z = E::load(data, i) + E::load(bias, col);
    E::store(data, i, col < n ? Act<AT>::tanh(z) : Act<AT>::sigmoid(z));
  }
}

// Column sums of data[rows, width] in two deterministic stages: partial[r, c] = sum of rows r, r + R, ... (R = gridDim.y),
// then out[c] = sum over r in ascending order.
template <typename AT>
__global__ void k_column_partial_sums(const void* data, float* partial, long long rows, int width) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float acc = 0.f;
  for (long long r = blockIdx.y; r < rows; r += gridDim.y) acc += Elem<AT>::load(data, r * width + c);
  partial[(long long)blockIdx.y * width + c] = acc;
}
static __global__ void k_column_final_sums(const float* partial, float* out, int parts, int width) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float acc = 0.f;
  for (int r = 0; r < parts; ++r) acc += partial[(long long)r * width + c];
  out[c] = acc;
}

}  // namespace rtn
