// gfx950 (CDNA4) kernels of the NativeLstm2 forward op.
//
// Semantics follow the reference operator: host loop returnn/native_op.py:1184-1285,
// pointwise step returnn/native_op.py:1081-1121, recurrent term H[t] += y_prev . W
// (returnn/native_op.cpp:1032-1067).  The structure does not: the recurrent GEMM, the gate
// non-linearities, the cell update and the mask are one fused step, the cell state and
// the last valid output of every (sequence, cell) live in registers of the thread that
// owns that pair, and in the persistent kernel of the default plan every workgroup keeps
// its slice of the recurrent weights in registers (as MFMA A-operand fragments) for all
// time steps.  The older kernel (k_lstm2_mfma), kept for layers too wide for that and for
// per-step launches, holds its slice in LDS for the steps of one launch, or takes the
// fragments straight from memory where LDS cannot hold them.
#pragma once

#include <hip/hip_runtime.h>

#include "lstm2_params.h"

namespace rtn {

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;

constexpr int kWgThreads = 256;  // 4 wavefronts of 64
constexpr int kWaves = 4;
constexpr int kFragBytes = 16;   // one MFMA operand fragment per lane
constexpr int kTileBytes = 64 * kFragBytes;
constexpr unsigned kBufFlags = 0x00020000;  // raw buffer descriptor word 3 (32-bit data format)
constexpr int kAuxDevice = 16;  // cache policy: device scope (sc1) for raw buffer loads/stores

// Per element type: how many elements fill one 16-byte fragment (KE) and how many k
// indices one macro step of the MFMA loop consumes (KM = 4 lane groups * KE).
template <typename AT>
struct Elem;

template <>
struct Elem<float> {
  static constexpr int KE = 4;
  static constexpr int KM = 16;
  static __device__ __forceinline__ float load(const void* p, size_t i) { return ((const float*)p)[i]; }
  static __device__ __forceinline__ void store(void* p, size_t i, float v) { ((float*)p)[i] = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
  // D[16x16] += A[16x16] * B[16x16] as four 16x16x4 MFMAs, one per fragment element.
  static __device__ __forceinline__ f32x4 mma(i32x4 a, i32x4 b, f32x4 c) {
    f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[0], bf[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[1], bf[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[2], bf[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[3], bf[3], c, 0, 0, 0);
    return c;
  }
  static __device__ __forceinline__ void store_coherent(__amdgpu_buffer_rsrc_t rs, unsigned off, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rs, off, 0, kAuxDevice);
  }
};

template <>
struct Elem<__bf16> {
  static constexpr int KE = 8;
  static constexpr int KM = 32;
  static __device__ __forceinline__ float load(const void* p, size_t i) { return (float)((const __bf16*)p)[i]; }
  static __device__ __forceinline__ void store(void* p, size_t i, float v) { ((__bf16*)p)[i] = (__bf16)v; }
  static __device__ __forceinline__ float round(float v) { return (float)(__bf16)v; }
  static __device__ __forceinline__ f32x4 mma(i32x4 a, i32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  }
  static __device__ __forceinline__ void store_coherent(__amdgpu_buffer_rsrc_t rs, unsigned off, float v) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, (__bf16)v), rs, off, 0, kAuxDevice);
  }
};

// sigmoid exactly as the reference writes it (returnn/native_op.py:1102-1104)
__device__ __forceinline__ float sigmoid_ref(float x) { return 1.f / (1.f + expf(-x)); }

// Gate non-linearities.  float32 runs use the accurate library functions in the reference's own
// formulation (1e-5 relative is the bar there).  bfloat16 runs round every result to 8 bits of
// mantissa anyway, so they use the hardware exp2 and reciprocal (about 1 ulp of float32 each):
// sigmoid(x) = 1 / (1 + 2^(-x log2 e)), tanh(x) = 2 sigmoid(2x) - 1.
template <typename AT>
struct Act;

template <>
struct Act<float> {
  static __device__ __forceinline__ float sigmoid(float x) { return sigmoid_ref(x); }
  static __device__ __forceinline__ float tanh(float x) { return tanhf(x); }
};

template <>
struct Act<__bf16> {
  static __device__ __forceinline__ float sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
  }
  static __device__ __forceinline__ float tanh(float x) {
    // (2 r - 1 as one fused multiply-add: 2 r is exact, so this is bit for bit r + r - 1)
    return __builtin_fmaf(2.f, __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-2.8853900817779268f * x)), -1.f);
  }
};

// True once a bounded wait of the launch has expired (status word 1; 2 marks a measurement run, which is not an error).
__device__ __forceinline__ bool wait_expired(const unsigned* status) {
  return __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1u;
}
// A 32-bit word full of quiet NaNs of the activation type.
template <typename AT>
inline constexpr unsigned kNanWords = 0x7FC00000u;
template <>
inline constexpr unsigned kNanWords<__bf16> = 0x7FC07FC0u;

// Frame visited at step s.
__device__ __forceinline__ long long frame_of(const Lstm2Params& p, int s) {
  return (long long)p.first + (long long)s * p.step;
}

// ---------------------------------------------------------------------------------------------
// Small helper kernels
// ---------------------------------------------------------------------------------------------

// T == 0: d := c0 (returnn/native_op.py:1236-1237)
static __global__ void k_copy_f32(const float* __restrict__ src, float* __restrict__ dst, long long count) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < count;
       i += (long long)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// Frames the loop does not visit keep Y = C = 0 and H = X (zero-initialised outputs plus the
// H := X copy of the reference, returnn/native_op.py:1247).  Only launched when start > 0 or |step| > 1.
template <typename AT>
__global__ void k_fill_unvisited(Lstm2Params p) {
  const long long bn = (long long)p.B * p.n;
  const int n4 = 4 * p.n;
  const long long per_frame = bn * 4;
  const long long total = p.T * per_frame;
  for (long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const long long t = idx / per_frame;
    const long long delta = t - p.first;
    bool visited;
    if (p.step > 0)
      visited = delta >= 0 && (delta % p.step) == 0 && delta / p.step < p.nsteps;
    else
      visited = delta <= 0 && ((-delta) % (-p.step)) == 0 && delta / p.step < p.nsteps;
    if (visited) continue;
    const long long rem = idx - t * per_frame;
    const long long row = t * p.B + rem / n4;  // (frame, sequence)
    ((AT*)p.H)[idx] = ((const AT*)p.X)[row * p.ldX + rem % n4];
    if (rem < bn) {
      Elem<AT>::store(p.Y, (t * p.B + rem / p.n) * p.ldY + rem % p.n, 0.f);
      p.C[t * bn + rem] = 0.f;
    }
  }
}

// Before the MFMA kernels: clears status and flags, writes y0 into buffer 0 of every group's
// hidden-state exchange area (in B-operand order) and packs W into A-operand order.
//
// Packed W: fragment (m, sm, lane) holds, for row i = lane%16 of M-tile m and lane group
// kg = lane/16, the KE elements W[KM*sm + KE*kg + e][gate*n + 4*m + cell] with
// cell = i/4, gate = i%4 -- i.e. the 16 rows of an M-tile are the 4 gates of 4 adjacent cells,
// so that after the MFMA one lane holds all four gate pre-activations of one (cell, sequence).
template <typename AT>
__device__ __forceinline__ void prepare_mfma(const Lstm2Params& p, int n_flags) {
  constexpr int KE = Elem<AT>::KE;
  constexpr int KM = Elem<AT>::KM;
  const long long gtid = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  const long long gsz = (long long)gridDim.x * blockDim.x;
  for (long long i = gtid; i < 64; i += gsz) p.status[i] = 0;
  for (long long i = gtid; i < n_flags; i += gsz) p.flags[i] = 0;
  // y0 -> hx[g][0][kb][b_local][e]
  const long long bn = (long long)p.B * p.n;
  const long long hx_buf = (long long)p.n * p.Bp;  // elements of one buffer
  for (long long idx = gtid; idx < bn; idx += gsz) {
    const int b = (int)(idx / p.n), c = (int)(idx % p.n);
    const int g = b / p.Bg, bl = b % p.Bg;
    const long long dst = ((long long)g * p.hx_bufs) * hx_buf + ((long long)(c / KE) * p.Bp + bl) * KE + (c % KE);
    ((AT*)p.hx)[dst] = ((const AT*)p.y0)[idx];
  }
  if (p.hx_sentinel) {
    // buffers 1.. of every group: all ones = "not yet written"
    const long long words_per_buf = hx_buf * (long long)sizeof(AT) / 4;
    const long long total = (long long)p.groups_total * p.hx_bufs * words_per_buf;
    for (long long w = gtid; w < total; w += gsz)
      if ((w / words_per_buf) % p.hx_bufs != 0) ((unsigned*)p.hx)[w] = 0xFFFFFFFFu;
  }
  // W -> Wp
  const int S = p.n / KM;
  // One macro step (KM rows of W) x 16 M-tiles (64 cells, 4 gates) per turn of a block, through LDS: the rows come in
  // as 16-byte pieces of consecutive memory (the entries refuse a W that is not 16-byte aligned), the fragments leave as
  // 1 KB per M-tile.  (Element by element from memory a lane's 8 loads of a bf16 fragment touch 8 rows of W and use 2
  // bytes of every line they fetch: for n = 1024 that took 14 us, four times what moving 16 MB takes.)
  constexpr int ES = (int)sizeof(AT);
  constexpr int MB = 16, SEG = 4 * MB * ES;           // bytes of one (row, gate) of a tile
  constexpr int SEGP = SEG + (ES == 2 ? 8 : 16);     // padded so that the 16 (gate, cell) and 4 row groups of a
  constexpr int ROWP = 4 * SEGP + (ES == 2 ? 4 : 0);  // fragment's lanes fall into different banks
  constexpr int CPS = SEG / 16;
  __shared__ unsigned tile[KM * ROWP / 4];
  const int m_tiles = p.n / 4, m_blocks = (m_tiles + MB - 1) / MB;
  for (int t = (int)blockIdx.x; t < S * m_blocks; t += (int)gridDim.x) {
    const int sm = t % S, m0 = (t / S) * MB;
    for (int c = (int)threadIdx.x; c < KM * 4 * CPS; c += (int)blockDim.x) {
      const int part = c % CPS, gate = (c / CPS) % 4, k = c / (4 * CPS);
      const int cell = 4 * m0 + part * (16 / ES);
      if (cell < p.n) {
        const u32x4 v = *(const u32x4*)((const AT*)p.W + (long long)(KM * sm + k) * 4 * p.n + gate * p.n + cell);
        unsigned* dst = tile + (k * ROWP + gate * SEGP + part * 16) / 4;
        dst[0] = v[0]; dst[1] = v[1]; dst[2] = v[2]; dst[3] = v[3];
      }
    }
    __syncthreads();
    for (int fi = (int)threadIdx.x; fi < MB * 64; fi += (int)blockDim.x) {
      const int lane = fi & 63, ml = fi >> 6, i = lane & 15, kg = lane >> 4;
      if (m0 + ml < m_tiles) {
        const unsigned char* src = (const unsigned char*)tile + (KE * kg) * ROWP + (i & 3) * SEGP + (4 * ml + (i >> 2)) * ES;
        struct { AT v[KE]; } frag;
#pragma unroll
        for (int e = 0; e < KE; ++e) frag.v[e] = *(const AT*)(src + e * ROWP);
        *(u32x4*)((AT*)p.Wp + (((long long)(m0 + ml) * S + sm) * 64 + lane) * KE) = __builtin_bit_cast(u32x4, frag);
      }
    }
    __syncthreads();
  }
}

template <typename AT>
__global__ void k_prepare_mfma(Lstm2Params p, int n_flags) {
  prepare_mfma<AT>(p, n_flags);
}

// The same for all problems of a fused launch at once: blockIdx.y = problem.
template <typename AT>
__global__ void k_prepare_mfma_multi(Lstm2Multi multi, int n_flags) {
  prepare_mfma<AT>(multi.p[blockIdx.y], n_flags);
}

// Widths the matrix-core kernels do not take run zero-padded: dst[rows_dst][blocks][n_pad] takes src[rows_src][blocks][n]
// (rows_src <= rows_dst) and zeros elsewhere; ET is an unsigned integer of the element's size (bits are copied).
template <typename ET>
__global__ void k_pad_cells(const ET* __restrict__ src, ET* __restrict__ dst, long long rows_src, long long rows_dst, int blocks,
                            int n, int n_pad, long long src_pitch) {
  // src_pitch: elements from one row of src to the next (blocks * n when contiguous)
  const long long total = rows_dst * blocks * n_pad;
  for (long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
    const int j = (int)(idx % n_pad);
    const long long rb = idx / n_pad;  // row * blocks + block
    const long long row = rb / blocks;
    dst[idx] = (j < n && row < rows_src) ? src[row * src_pitch + (rb % blocks) * n + j] : (ET)0;
  }
}

// The inverse: dst[rows][blocks][n] (rows dst_pitch elements apart) from src[rows][blocks][n_pad].
template <typename ET>
__global__ void k_unpad_cells(const ET* __restrict__ src, ET* __restrict__ dst, long long rows, int blocks, int n, int n_pad,
                              long long dst_pitch) {
  const long long total = rows * blocks * n;
  for (long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
    const int j = (int)(idx % n);
    const long long rb = idx / n;
    dst[(rb / blocks) * dst_pitch + (rb % blocks) * n + j] = src[rb * n_pad + j];
  }
}

// Clears the status word for the generic path.
static __global__ void k_fill_u32(unsigned* dst, unsigned value, long long count) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < count;
       i += (long long)gridDim.x * blockDim.x)
    dst[i] = value;
}

// rows of row_words 32-bit words, pitch_words apart: := 0
static __global__ void k_clear_rows(unsigned* dst, long long rows, long long row_words, long long pitch_words) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < rows * row_words; i += (long long)gridDim.x * blockDim.x) {
    const long long r = i / row_words;
    dst[r * pitch_words + (i - r * row_words)] = 0u;
  }
}

// data[i] += bias[i % width]  (rows of `width` elements)
template <typename AT>
__global__ void k_add_bias(void* data, const void* bias, long long count, int width) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x)
    Elem<AT>::store(data, i, Elem<AT>::load(data, i) + Elem<AT>::load(bias, i % width));
}

static __global__ void k_clear_status(unsigned* status) {
  if (threadIdx.x < 64) status[threadIdx.x] = 0;
}

// Caller-side final output (returnn/tf/native_op.py:913-929): one workgroup per sequence finds the
// last visited frame (in processing order) with a non-zero mask and copies that row of Y, else y0.
template <typename AT>
__global__ void k_last_output(const void* Y, const void* y0, const float* mask, void* out, long long T, int B, int n,
                              int first, int step, int nsteps, long long ldY) {
  __shared__ int s_last;
  const int b = blockIdx.x;
  if (threadIdx.x == 0) s_last = -1;
  __syncthreads();
  int last = -1;
  for (int s = threadIdx.x; s < nsteps; s += blockDim.x) {
    const long long t = (long long)first + (long long)s * step;
    if ((int)mask[t * B + b] != 0) last = s;
  }
  if (last >= 0) atomicMax(&s_last, last);
  __syncthreads();
  last = s_last;
  const AT* src = (last >= 0) ? (const AT*)Y + (((long long)first + (long long)last * step) * B + b) * ldY
                              : (const AT*)y0 + (long long)b * n;
  for (int j = threadIdx.x; j < n; j += blockDim.x) ((AT*)out)[(long long)b * n + j] = src[j];
}

// ---------------------------------------------------------------------------------------------
// Generic per-step kernel: any B and n, one thread per (sequence, cell).  Accumulates X + y.W
// over ascending k in float32, the order of a plain sequential GEMM.
// Step s reads the carry buffer (s & 1) (y0 at s == 0) and writes buffer ((s + 1) & 1).
// ---------------------------------------------------------------------------------------------
template <typename AT>
__global__ void k_step_generic(Lstm2Params p, int s) {
  const long long bn = (long long)p.B * p.n;
  const long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  if (idx >= bn) return;
  const int n = p.n;
  const int b = (int)(idx / n), j = (int)(idx % n);
  const long long t = frame_of(p, s);
  const void* y_in = (s == 0) ? p.y0 : (const void*)((const AT*)p.ycarry + (size_t)(s & 1) * bn);
  void* y_out = (void*)((AT*)p.ycarry + (size_t)((s + 1) & 1) * bn);
  const float* c_in = (s == 0) ? p.c0 : p.C + (t - p.step) * bn;
  const size_t xoff = ((size_t)t * p.B + b) * 4 * n + j;       // in H
  const size_t xin = ((size_t)t * p.B + b) * (size_t)p.ldX + j;  // in X
  float g0 = Elem<AT>::load(p.X, xin);
  float g1 = Elem<AT>::load(p.X, xin + n);
  float g2 = Elem<AT>::load(p.X, xin + 2 * (size_t)n);
  float g3 = Elem<AT>::load(p.X, xin + 3 * (size_t)n);
  const size_t yrow = (size_t)b * n;
  for (int k = 0; k < n; ++k) {
    const float yk = Elem<AT>::load(y_in, yrow + k);
    const size_t w = (size_t)k * 4 * n + j;
    g0 += yk * Elem<AT>::load(p.W, w);
    g1 += yk * Elem<AT>::load(p.W, w + n);
    g2 += yk * Elem<AT>::load(p.W, w + 2 * (size_t)n);
    g3 += yk * Elem<AT>::load(p.W, w + 3 * (size_t)n);
  }
  const float m = p.mask[t * p.B + b];
  const float a0 = Act<AT>::tanh(g0), a1 = Act<AT>::sigmoid(g1), a2 = Act<AT>::sigmoid(g2), a3 = Act<AT>::sigmoid(g3);
  const float pc = c_in[idx];
  const float c = (pc * a2 + a0 * a1) * m + pc * (1.f - m);
  Elem<AT>::store(p.H, xoff, (p.op_flags & kOpH0IsCell) ? c : a0);
  Elem<AT>::store(p.H, xoff + n, a1);
  Elem<AT>::store(p.H, xoff + 2 * (size_t)n, a2);
  Elem<AT>::store(p.H, xoff + 3 * (size_t)n, a3);
  p.C[t * bn + idx] = c;
  const float y = Elem<AT>::round(Act<AT>::tanh(c) * a3 * m);
  Elem<AT>::store(p.Y, ((size_t)t * p.B + b) * (size_t)p.ldY + j, y);
  Elem<AT>::store(y_out, idx, (p.op_flags & kOpNoCarry) ? y : y + Elem<AT>::load(y_in, idx) * (1.f - m));
  if (s == p.nsteps - 1) p.d[idx] = c;
}

// ---------------------------------------------------------------------------------------------
// MFMA kernel.  Grid = groups * wgs_per_group workgroups of 256 threads.
//
// A group owns Bg batch rows; inside it workgroup rank r owns the MT*4 cells
// [4*MT*r, 4*MT*(r+1)) = MT M-tiles of 16 gate columns.  Per step every workgroup computes
// G^T[16*MT, 16*NT] = Wslice^T[16*MT, n] . h^T[n, 16*NT] with the k range dealt round-robin
// to the 4 wavefronts (macro step sm belongs to wave sm % 4), sums the four partial tiles
// through LDS, and the thread that owns (sequence, cell) applies gates, cell update and mask
// and publishes its new hidden value in B-operand order for everybody's next step.
//
// s_begin/s_end: steps run by this launch.  With s_end - s_begin > 1 the launch must be
// co-resident (cooperative launch): steps are separated by a flag wait, bounded by
// timeout_ticks; an expired wait sets status[0] and every later wait returns at once,
// so the grid always drains.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void map_block(const Lstm2Params& p, int bid, int& g, int& r) {
  const int NG = p.groups, G = p.wgs_per_group, X = p.xcds;
  // Consecutive workgroup ids go round-robin over the XCDs (each with its own L2).  Put a
  // group on as few XCDs as possible and give the workgroups of one XCD adjacent cells, so that
  // their partial cache-line reads of X and writes of Y/C/H meet in that XCD's L2.
  if (X > 1 && NG <= X && X % NG == 0 && G % (X / NG) == 0) {
    const int xpg = X / NG;
    const int x = bid % X, q = bid / X;
    g = x / xpg;
    r = (x % xpg) * (G / xpg) + q;
  } else if (X > 1 && NG % X == 0) {
    g = bid % NG;
    r = bid / NG;
  } else {
    g = bid / G;
    r = bid % G;
  }
}

__device__ __forceinline__ void wait_flags(const Lstm2Params& p, const unsigned* flags, int G, unsigned need,
                                           int lane) {
  unsigned long long t0 = 0;
  unsigned spins = 0;
  for (;;) {
    bool ok = true;
    for (int r = lane; r < G; r += 64)
      ok = ok && (__hip_atomic_load(flags + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= need);
    if (__all(ok)) break;
    if ((spins++ & 31u) == 0) {
      if (__hip_atomic_load(p.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
      const unsigned long long now = wall_clock64();
      if (spins == 1) {
        t0 = now;
      } else if (now - t0 > p.timeout_ticks) {
        __hip_atomic_store(p.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
    __builtin_amdgcn_s_sleep(1);
  }
  if (p.sync_policy & kAcquireFence) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

template <typename AT, int MT, int NT>
__global__ __launch_bounds__(kWgThreads) void k_lstm2_mfma(const Lstm2Params p, const int s_begin, const int s_end) {
  using E = Elem<AT>;
  constexpr int KE = E::KE;
  constexpr int KM = E::KM;
  constexpr int TILES = MT * NT;
  constexpr int EPT = (TILES + kWaves - 1) / kWaves;  // epilogue tiles per thread
  constexpr int U = (NT >= 4) ? 4 : 8;                // macro steps whose h fragments are in flight together

  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it in a scalar register
  const int n = p.n, S = n / KM;
  // A launch of one step uses every fragment of W once: it can take them from memory directly, with many small
  // workgroups per CU hiding the latency, instead of copying its slice to LDS first (p.w_direct).
  const bool direct = p.w_direct != 0;
  i32x4* Wl = (i32x4*)smem;                                                       // [MT][S][64] fragments (unless direct)
  f32x4* red = (f32x4*)(smem + (direct ? (size_t)0 : (size_t)MT * S * kTileBytes));  // [kWaves][TILES][64]

  int g, r;
  map_block(p, blockIdx.x, g, r);
  g += p.group_offset;
  const int b_base = g * p.Bg;
  const int rows = min(p.Bg, p.B - b_base);
  const bool persist = (s_end - s_begin) > 1;
  const long long bn = (long long)p.B * n;
  const size_t hx_buf_bytes = (size_t)n * p.Bp * sizeof(AT);
  unsigned char* hx_g = (unsigned char*)p.hx + (size_t)g * p.hx_bufs * hx_buf_bytes;
  const unsigned* flags_g = p.flags + (size_t)g * p.wgs_per_group;

  // W slice of this workgroup: global (already in fragment order) -> LDS, once per launch.
  const i32x4* Wsrc = (const i32x4*)p.Wp + (size_t)r * MT * S * 64;
  if (!direct)
    for (int i = tid; i < MT * S * 64; i += kWgThreads) Wl[i] = Wsrc[i];

  // State of the (sequence, cell) pairs this thread owns.
  float c_state[EPT], h_prev[EPT];
  int e_b[EPT], e_cell[EPT];
  bool e_valid[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = wave + kWaves * j;
    const int mt = e / NT, nt = e % NT;
    const int bl = 16 * nt + (lane & 15);
    e_cell[j] = 4 * (r * MT + mt) + (lane >> 4);
    e_b[j] = bl;
    e_valid[j] = (e < TILES) && (bl < rows);
    c_state[j] = 0.f;
    h_prev[j] = 0.f;
    if (e_valid[j]) {
      const long long bc = (long long)(b_base + bl) * n + e_cell[j];
      if (s_begin == 0) {
        c_state[j] = p.c0[bc];
        h_prev[j] = E::load(p.y0, bc);
      } else {
        c_state[j] = p.C[(frame_of(p, s_begin) - p.step) * bn + bc];
        const size_t ho = ((size_t)(e_cell[j] / KE) * p.Bp + bl) * KE + (e_cell[j] % KE);
        h_prev[j] = E::load(hx_g + (size_t)(s_begin & 1) * hx_buf_bytes, ho);
      }
    }
  }
  __syncthreads();

  const int kg = lane >> 4, jl = lane & 15;

  for (int s = s_begin; s < s_end; ++s) {
    const long long t = frame_of(p, s);

    // Gate inputs and mask of this step: independent of the recurrence, issued before the wait.
    float xg[EPT][4], msk[EPT];
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      msk[j] = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) xg[j][q] = 0.f;
      if (e_valid[j]) {
        const size_t xo = ((size_t)t * p.B + (b_base + e_b[j])) * (size_t)p.ldX + e_cell[j];
#pragma unroll
        for (int q = 0; q < 4; ++q) xg[j][q] = E::load(p.X, xo + (size_t)q * n);
        msk[j] = p.mask[t * p.B + b_base + e_b[j]];
      }
    }

    if (persist && s > s_begin) wait_flags(p, flags_g, p.wgs_per_group, (unsigned)s, lane);

    // Recurrent GEMM: this wave's share of k.
    f32x4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const unsigned char* hx_cur = hx_g + (size_t)(s & 1) * hx_buf_bytes;
    __amdgpu_buffer_rsrc_t hx_rs = __builtin_amdgcn_make_buffer_rsrc((void*)hx_cur, 0, 0x7fffffff, kBufFlags);
    const bool ld_coherent = persist && (p.sync_policy & kLoadCoherent);
    for (int sm0 = wave; sm0 < S; sm0 += kWaves * U) {
      i32x4 bf[U][NT], afd[U][MT];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int sm = sm0 + kWaves * u;
        if (sm < S) {
          if (direct) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) afd[u][mt] = Wsrc[(mt * S + sm) * 64 + lane];
          }
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const unsigned off = (unsigned)(((4 * sm + kg) * p.Bp + 16 * nt + jl) * kFragBytes);
            if (ld_coherent)
              bf[u][nt] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(hx_rs, off, 0, kAuxDevice));
            else
              bf[u][nt] = *(const i32x4*)(hx_cur + off);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int sm = sm0 + kWaves * u;
        if (sm < S) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const i32x4 af = direct ? afd[u][mt] : Wl[(mt * S + sm) * 64 + lane];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = E::mma(af, bf[u][nt], acc[mt][nt]);
          }
        }
      }
    }

    // Partial tiles -> LDS.
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) red[(wave * TILES + mt * NT + nt) * 64 + lane] = acc[mt][nt];
    __syncthreads();

    // Epilogue: gates, cell update, mask; publish the new hidden value first (critical path).
    unsigned char* hx_nxt = hx_g + (size_t)((s + 1) & 1) * hx_buf_bytes;
    __amdgpu_buffer_rsrc_t nx_rs = __builtin_amdgcn_make_buffer_rsrc((void*)hx_nxt, 0, 0x7fffffff, kBufFlags);
    const bool st_coherent = persist && (p.sync_policy & kStoreCoherent);
    float a_out[EPT][4], y_out[EPT];
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int e = wave + kWaves * j;
      if (e < TILES) {
        f32x4 gsum = red[(0 * TILES + e) * 64 + lane];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) gsum += red[(w * TILES + e) * 64 + lane];
        const float m = msk[j];
        const float a0 = Act<AT>::tanh(gsum[0] + xg[j][0]);
        const float a1 = Act<AT>::sigmoid(gsum[1] + xg[j][1]);
        const float a2 = Act<AT>::sigmoid(gsum[2] + xg[j][2]);
        const float a3 = Act<AT>::sigmoid(gsum[3] + xg[j][3]);
        const float pc = c_state[j];
        const float c = (pc * a2 + a0 * a1) * m + pc * (1.f - m);
        const float y = E::round(Act<AT>::tanh(c) * a3 * m);
        const float hn = (p.op_flags & kOpNoCarry) ? y : E::round(y + h_prev[j] * (1.f - m));
        c_state[j] = c;
        h_prev[j] = hn;
        y_out[j] = y;
        a_out[j][0] = (p.op_flags & kOpH0IsCell) ? c : a0;
        a_out[j][1] = a1;
        a_out[j][2] = a2;
        a_out[j][3] = a3;
        if (e_valid[j]) {
          const unsigned ho =
              (unsigned)((((e_cell[j] / KE) * p.Bp + e_b[j]) * KE + (e_cell[j] % KE)) * (int)sizeof(AT));
          if (st_coherent)
            E::store_coherent(nx_rs, ho, hn);
          else
            E::store(hx_nxt, ho / sizeof(AT), hn);
        }
      }
    }
    if (persist) {
      // Every thread's hidden-state stores have left the CU before the workgroup's flag goes up.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();  // also frees `red` for the next step
    if (persist && tid == 0) {
      if (p.sync_policy & kReleaseFence) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      __hip_atomic_store(p.flags + (size_t)g * p.wgs_per_group + r, (unsigned)(s + 1), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }

    // Outputs of the op (off the critical path).
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      if (e_valid[j]) {
        const long long bc = (long long)(b_base + e_b[j]) * n + e_cell[j];
        const size_t xo = ((size_t)t * p.B + (b_base + e_b[j])) * 4 * n + e_cell[j];
#pragma unroll
        for (int q = 0; q < 4; ++q) E::store(p.H, xo + (size_t)q * n, a_out[j][q]);
        p.C[t * bn + bc] = c_state[j];
        E::store(p.Y, ((size_t)t * p.B + (b_base + e_b[j])) * (size_t)p.ldY + e_cell[j], y_out[j]);
      }
    }
  }

  if (s_end == p.nsteps) {
    // after a wait that ran into its bound: NaN as the final cell state and in the last visited frame of Y
    const bool expired = wait_expired(p.status);
    const long long t_last = frame_of(p, p.nsteps - 1);
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      if (e_valid[j]) {
        const long long bc = (long long)(b_base + e_b[j]) * n + e_cell[j];
        p.d[bc] = expired ? __builtin_nanf("") : c_state[j];
        if (expired) E::store(p.Y, ((size_t)t_last * p.B + (b_base + e_b[j])) * (size_t)p.ldY + e_cell[j], __builtin_nanf(""));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Persistent kernel with the recurrent weights in registers, a barrier-free exchange and a
// decoupled input and output streams.
//
// Same decomposition and the same arithmetic per output element as k_lstm2_mfma (k dealt
// round-robin to 4 compute wavefronts, partial tiles summed in wave order), but:
//  * every compute wavefront keeps the A-operand fragments of its k share in registers for all
//    steps (MT * KSMAX fragments of 4 registers): a step reads no weights from LDS or memory;
//  * there is no flag barrier.  The hidden state travels through a ring of 4 buffers whose
//    elements validate themselves: a buffer starts as all-ones words ("not yet written", a NaN
//    pattern the producers never emit), every element is written exactly once per use by the
//    workgroup that owns the cell, and a consumer re-reads the fragments it needs until none
//    of their elements is all-ones.  One store -> load hop per step instead of store,
//    acknowledge, flag, poll, load.  The first read of step s+1 is issued right after the
//    hidden values of step s have gone out.
//    Step s reads buffer s%4, writes its outputs to (s+1)%4 and re-arms its own elements of
//    (s+3)%4 = (s-1)%4, which every workgroup has finished reading (this workgroup has seen
//    all outputs of step s-1).  A wavefront's re-arm stores are acknowledged (vmcnt(0) after its
//    next successful read) before its next hidden-value stores, which precede anybody's first
//    look at that buffer for step s+3, so a consumer can never mistake an old value for a new one.
//  * the op's streams are decoupled from the recurrence: X[t] and the mask are fetched four steps
//    ahead as 16-byte chunks spread over the workgroup, parked in registers, handed over through
//    LDS two steps before their own and read into the registers of the thread that needs them one
//    step before -- all of it while the workgroup waits for the exchange anyway; H[t], Y[t], C[t] are staged in LDS by the threads that compute them and written
//    out one step later, again 16 bytes per thread.  So the waits of the recurrence never contain
//    the HBM latency of a stream, and the streams are coalesced.  One workgroup barrier per step
//    (after the partial tiles are in LDS) orders everything.
//  * exchange scope: the memory side of the device (sc1 loads and stores), which is valid
//    wherever the workgroups of a group run.
// Waits are bounded as in k_lstm2_mfma.
// ---------------------------------------------------------------------------------------------
constexpr int kExDevice = 0;  // device-scope loads and stores: always valid
constexpr int kExLocal = 1;   // the whole group on one XCD: plain stores into that XCD's L2, loads that bypass the first-level cache
// measurement aid: a step without the exchange's reads -- no loads of the hidden state (the MFMAs run on zeros), no delay,
// no waiting; the new values are still stored (plain stores).  Results are WRONG; status is set to 2.
constexpr int kExNoWait = 3;

template <typename AT>
struct Sentinel;

template <>
struct Sentinel<float> {
  static __device__ __forceinline__ bool complete(i32x4 v) {
    const unsigned a = max(max((unsigned)v[0], (unsigned)v[1]), max((unsigned)v[2], (unsigned)v[3]));
    return a != 0xFFFFFFFFu;
  }
  // value as stored: NaNs are canonicalised so that no payload equals the sentinel
  static __device__ __forceinline__ unsigned bits(float v) { return (v != v) ? 0x7FC00000u : __builtin_bit_cast(unsigned, v); }
  template <int AUX>
  static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t rs, unsigned off, unsigned bits) {
    __builtin_amdgcn_raw_buffer_store_b32(bits, rs, off, 0, AUX);
  }
  static constexpr unsigned kSentinel = 0xFFFFFFFFu;
};

template <>
struct Sentinel<__bf16> {
  // Non-zero iff one of the two halfwords of x is 0xFFFF: the classic "has a zero lane" test on ~x
  // (exact for the any-lane question).
  static __device__ __forceinline__ unsigned has_ffff(unsigned x) {
    const unsigned y = ~x;
    return (y - 0x00010001u) & x & 0x80008000u;
  }
  static __device__ __forceinline__ bool complete(i32x4 v) {
    return (has_ffff((unsigned)v[0]) | has_ffff((unsigned)v[1]) | has_ffff((unsigned)v[2]) | has_ffff((unsigned)v[3])) == 0;
  }
  static __device__ __forceinline__ unsigned bits(float v) {
    return (v != v) ? 0x7FC0u : (unsigned)__builtin_bit_cast(unsigned short, (__bf16)v);
  }
  template <int AUX>
  static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t rs, unsigned off, unsigned bits) {
    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)bits, rs, off, 0, AUX);
  }
  static constexpr unsigned kSentinel = 0xFFFFu;
};

constexpr int kHxRing = 4;

template <int V>
struct IntTag {
  static constexpr int value = V;
};

// LDS layout of k_lstm2_regw (bytes), shared with the host for the launch.  The staging copies of X[t], H[t], Y[t] and
// C[t] keep the frame's order [row][gate][cell] with kRowPad bytes appended to every row: without them the rows of a
// workgroup's tile start 64, 128 or 256 bytes apart, the 16 lanes that touch the same cell of 16 rows all meet in the
// same banks, and three quarters of the kernel's LDS cycles were bank conflicts (SQ_LDS_BANK_CONFLICT).
constexpr unsigned kRowPad = 16;
struct RegwLds {
  unsigned red, xl, ml, hs, ys, cs, total;
  unsigned x_row, y_row, c_row;      // bytes from one row to the next in the X / H, Y and C copies
  unsigned x_copy, y_copy, c_copy;   // bytes of one copy (the X / H copy ends with a 16-byte slot nobody reads)
};
__host__ __device__ constexpr RegwLds regw_lds(int es, int MT, int NT) {
  RegwLds l{};
  const unsigned rows = 16u * NT, cells = 4u * MT;
  l.x_row = 4u * cells * es + kRowPad;
  l.y_row = cells * es + kRowPad;
  l.c_row = cells * 4u + kRowPad;
  l.x_copy = rows * l.x_row + 16u;
  l.y_copy = rows * l.y_row;
  l.c_copy = rows * l.c_row;
  unsigned off = 0;
  l.red = off; off += 2u * kWaves * MT * NT * kTileBytes;
  l.xl = off; off += 2u * l.x_copy;
  l.hs = off; off += 3u * l.x_copy;
  l.ys = off; off += (3u * l.y_copy + 15u) / 16u * 16u;
  l.cs = off; off += 3u * l.c_copy;
  l.ml = off; off += 2u * rows * 4u + 16u;  // two copies and a spare word
  l.total = off;
  return l;
}

// 16-byte (or 8-byte) chunk moves of the stream wavefront.
template <int CH>
struct Chunk;
template <>
struct Chunk<16> {
  typedef i32x4 T;
  static __device__ __forceinline__ T load(__amdgpu_buffer_rsrc_t rs, unsigned off) {
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0));
  }
  static __device__ __forceinline__ T fill(unsigned word) { return T{(int)word, (int)word, (int)word, (int)word}; }
  static __device__ __forceinline__ void store(T v, __amdgpu_buffer_rsrc_t rs, unsigned off) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, v), rs, off, 0, 0);
  }
};
template <>
struct Chunk<8> {
  typedef unsigned long long T;
  static __device__ __forceinline__ T load(__amdgpu_buffer_rsrc_t rs, unsigned off) {
    return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, 0));
  }
  static __device__ __forceinline__ T fill(unsigned word) { return ((T)word << 32) | word; }
  static __device__ __forceinline__ void store(T v, __amdgpu_buffer_rsrc_t rs, unsigned off) {
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(__attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned, v), rs, off, 0, 0);
  }
};

// Running maximum over the 16-bit (bf16) or 32-bit (float) lanes of the words of a fragment: a lane
// of the result is all-ones iff some element seen so far was the "not yet written" pattern.
template <typename AT>
struct LaneMax;
template <>
struct LaneMax<float> {
  static __device__ __forceinline__ unsigned fold(unsigned acc, unsigned x) { return max(acc, x); }
  static __device__ __forceinline__ bool has_sentinel(unsigned acc) { return acc == 0xFFFFFFFFu; }
};
template <>
struct LaneMax<__bf16> {
  static __device__ __forceinline__ unsigned fold(unsigned acc, unsigned x) {
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(u16x2, acc), __builtin_bit_cast(u16x2, x)));
  }
  static __device__ __forceinline__ bool has_sentinel(unsigned acc) {
    return (acc & 0xFFFFu) == 0xFFFFu || (acc >> 16) == 0xFFFFu;
  }
};

// Optional instrumentation (-DRTN_LSTM2_TRACE): wave 0 of every workgroup accumulates shader-clock
// cycles per phase of k_lstm2_regw's step and writes the 8 totals to trace[workgroup * 8 ..] at the end.
#ifdef RTN_LSTM2_TRACE
#define RTN_TRACE_DECL unsigned long long tr_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}; unsigned long long tr_last = clock64();
#define RTN_TRACE_MARK(k) { const unsigned long long tr_now = clock64(); tr_acc[k] += tr_now - tr_last; tr_last = tr_now; }
#define RTN_TRACE_ADD(k, v) { tr_acc[k] += (v); }
#define RTN_TRACE_FLUSH(p, bid) if ((p).trace && threadIdx.x == 0) { for (int k = 0; k < 8; ++k) (p).trace[(size_t)(bid) * 8 + k] = tr_acc[k]; }
#else
#define RTN_TRACE_DECL
#define RTN_TRACE_MARK(k)
#define RTN_TRACE_ADD(k, v)
#define RTN_TRACE_FLUSH(p, bid)
#endif

constexpr unsigned kOobOffset = 0xFFFFFF00u;  // a buffer offset beyond any frame: loads give 0, stores are dropped

// The XCD (accelerator die, with an L2 of its own) this wavefront runs on.
__device__ __forceinline__ unsigned xcc_id() {
  unsigned x;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
  return x & 0xFu;
}

// Which XCDs does the device deal the workgroups of a grid to?  Every workgroup adds the XCD it runs on to a bit mask.
static __global__ void k_probe_xcds(unsigned* mask) {
  if (threadIdx.x == 0) (void)__hip_atomic_fetch_or(mask, 1u << xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One thread per workgroup: are all `members` workgroups that share `words` on one XCD?  Every caller adds its XCD to the
// mask words[1] and then itself to the count words[0] (both cleared before the launch; device-scope atomics whose result
// is waited for, so the mask is complete when the count is).  The wait is bounded like every other (status[0] = 1 when it
// expires; the answer is then "no").  A group found on several XCDs leaves its mask in status[1] for the record.
__device__ __forceinline__ bool group_on_one_xcd(unsigned* words, unsigned members, unsigned* status, unsigned long long timeout_ticks) {
  if (members <= 1) return true;
  (void)__hip_atomic_fetch_or(words + 1, 1u << xcc_id(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  (void)__hip_atomic_fetch_add(words, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  unsigned long long t0 = 0;
  unsigned spins = 0;
  bool complete = true;
  while (__hip_atomic_load(words, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < members) {
    if ((spins++ & 15u) == 0) {
      if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { complete = false; break; }
      const unsigned long long now = wall_clock64();
      if (spins == 1) {
        t0 = now;
      } else if (now - t0 > timeout_ticks) {
        __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        complete = false;
        break;
      }
    }
    __builtin_amdgcn_s_sleep(2);
  }
  const unsigned mask = __hip_atomic_load(words + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const bool ok = complete && (mask & (mask - 1)) == 0;
  if (!ok) __hip_atomic_store(status + 1, mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return ok;
}

// HALF: the groups have at most 8 rows (NT == 1, MT even).  A tile then holds valid results in the lanes of rows 0..7
// only, and the pointwise part folds two tiles into one pass: lanes of rows 0..7 take tile 2u, lanes of rows 8..15 take
// rows 0..7 of tile 2u + 1, so that a thread owns one (sequence, cell) pair where the plain mapping gives it two, one
// of them of a row that does not exist.
template <typename AT, int MT, int NT, int KSMAX, bool HALF = false>
__global__ __launch_bounds__(kWgThreads) void k_lstm2_regw(const Lstm2Multi multi) {
  static_assert(!HALF || (NT == 1 && MT % 2 == 0), "half-tile mapping: one batch tile, an even number of cell tiles");
  // Which of the launch's problems and which (group, rank) this workgroup works on (uniform over the workgroup).
  int which, g, r;
  if (multi.local) {
    // Every batch group on ONE XCD, so that the hidden state is exchanged through that XCD's L2.  The dispatcher deals
    // workgroup ids round-robin to the XCDs: id = slot * xcds + xcd.  An XCD hosts the groups xcd, xcd + xcds, ...
    // of the launch (all problems counted through); that all members of a group really share an XCD is checked below.
    const int X = multi.xcds, G = multi.p[0].wgs_per_group, per = multi.p[0].groups;
    const int xcd = (int)blockIdx.x % X, slot = (int)blockIdx.x / X;
    const int gg = (slot / G) * X + xcd;
    which = gg / per;
    if (which >= multi.count) return;
    g = gg - which * per;
    r = slot % G;
  } else {
    which = (int)blockIdx.x / multi.wgs_each;
    const int bid = (int)blockIdx.x - which * multi.wgs_each;
    if (which >= multi.count || bid >= multi.grid) return;
    map_block(multi.p[which], bid, g, r);
  }
  const Lstm2Params p = multi.p[which];
  const int trace_id = which * p.groups * p.wgs_per_group + g * p.wgs_per_group + r;
  (void)trace_id;
  using E = Elem<AT>;
  using SN = Sentinel<AT>;
  using LM = LaneMax<AT>;
  constexpr int KE = E::KE;
  constexpr int KM = E::KM;
  constexpr int ES = (int)sizeof(AT);
  constexpr int TILES = MT * NT;
  constexpr int UNITS = HALF ? TILES / 2 : TILES;  // passes of the pointwise part over all wavefronts
  constexpr int EPT = (UNITS + kWaves - 1) / kWaves;
  constexpr int ROWS = 16 * NT;   // rows of the MFMA tiles (>= valid rows of the group)
  constexpr int CELLS = 4 * MT;   // cells owned by this workgroup
  constexpr RegwLds L = regw_lds(ES, MT, NT);

  extern __shared__ __align__(16) unsigned char smem[];
  typedef f32x4 RedBuf[kWaves][TILES][64];
  RedBuf* red = (RedBuf*)(smem + L.red);  // [2]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it in a scalar register
  const int n = p.n, S = n / KM;
  g += p.group_offset;
  const int b_base = g * p.Bg;
  const int rows = min(p.Bg, p.B - b_base);
  const long long bn = (long long)p.B * n;
  const int nsteps = p.nsteps;

  // ---- the op's streams: X[t], mask[t] in; H[t], Y[t], C[t] out, as 16-byte (8-byte) chunks spread
  // over the 256 threads.  X is fetched four steps ahead into registers and copied to LDS two steps
  // before its own (a barrier lies between that copy and its readers); the outputs are staged in LDS by the threads that compute them and written
  // out after the barrier of the following step.  Chunks of rows the group does not have carry an
  // out-of-range buffer offset: their loads return 0 and their stores are dropped, without a branch.
  float* Ml = (float*)(smem + L.ml);
  constexpr int SEG = CELLS * ES;               // contiguous bytes of one (row, gate) in X and H
  constexpr int CH = SEG < 16 ? 8 : 16;         // bytes moved per thread and chunk
  constexpr int CPS = SEG / CH;                 // chunks per (row, gate)
  constexpr int XCH = (ROWS * 4 * CPS + kWgThreads - 1) / kWgThreads;  // chunks per thread, X and H
  constexpr int CHY = SEG < 16 ? 8 : 16;        // one row of Y is SEG bytes too
  constexpr int YCH = (ROWS * (SEG / CHY) + kWgThreads - 1) / kWgThreads;
  constexpr int SEGC = CELLS * 4;               // one row of C (float)
  constexpr int CCH = (ROWS * (SEGC / 16) + kWgThreads - 1) / kWgThreads;
  typedef Chunk<CH> XC;
  typedef Chunk<CHY> YC;
  typedef Chunk<16> CC;
  const int cell0 = CELLS * r;
  unsigned xoff[XCH], hoff[XCH], yoff[YCH], coff[CCH];  // byte offsets inside one frame (kOobOffset: nothing to move); the rows of
                                                        // X and Y may lie further apart than those of H and C (ldX, ldY)
  unsigned xlds[XCH], ylds[YCH], clds[CCH];  // byte offsets inside one LDS copy
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int c = tid + kWgThreads * i;
    const int row = c / (4 * CPS), gate = (c / CPS) % 4, part = c % CPS;
    xoff[i] = row < rows ? (unsigned)(((long long)(b_base + row) * p.ldX + gate * n + cell0) * ES + part * CH) : kOobOffset;
    hoff[i] = row < rows ? (unsigned)((((b_base + row) * 4 * n) + gate * n + cell0) * ES + part * CH) : kOobOffset;
    // threads beyond the tile write to / read from the spare slot at the end of the copy
    xlds[i] = row < ROWS ? (unsigned)(row * L.x_row + gate * SEG + part * CH) : (unsigned)(ROWS * L.x_row);
  }
#pragma unroll
  for (int i = 0; i < YCH; ++i) {
    const int c = tid + kWgThreads * i;
    const int row = c / (SEG / CHY), part = c % (SEG / CHY);
    yoff[i] = row < rows ? (unsigned)(((long long)(b_base + row) * p.ldY + cell0) * ES + part * CHY) : kOobOffset;
    ylds[i] = (unsigned)(min(row, ROWS - 1) * L.y_row + part * CHY);
  }
#pragma unroll
  for (int i = 0; i < CCH; ++i) {
    const int c = tid + kWgThreads * i;
    const int row = c / (SEGC / 16), part = c % (SEGC / 16);
    coff[i] = row < rows ? (unsigned)(((b_base + row) * n + cell0) * 4 + part * 16) : kOobOffset;
    clds[i] = (unsigned)(min(row, ROWS - 1) * L.c_row + part * 16);
  }
  const unsigned moff = tid < rows ? (unsigned)((b_base + tid) * 4) : kOobOffset;
  const unsigned frame_x = (unsigned)((size_t)p.B * p.ldX * ES), frame_h = (unsigned)((size_t)p.B * 4 * n * ES),
                 frame_y = (unsigned)((size_t)p.B * p.ldY * ES), frame_c = (unsigned)(bn * 4), frame_m = (unsigned)(p.B * 4);
  typename XC::T xv[2][XCH];
  float mv[2] = {0.f, 0.f};
  // Frame pointers advance by a constant per step (signed: the op may run backwards in time).
  const long long step_x = (long long)p.step * frame_x, step_h = (long long)p.step * frame_h, step_y = (long long)p.step * frame_y,
                  step_c = (long long)p.step * frame_c, step_m = (long long)p.step * frame_m;
  auto fetch_x_at = [&](const unsigned char* xp, bool enabled, auto par_tag) {  // loads of one frame of X into register set PAR
    constexpr int PAR = decltype(par_tag)::value;
    // (a frame that does not exist: a buffer of no bytes, every load gives 0 without a memory access or a branch)
    __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void*)xp, 0, enabled ? frame_x : 0u, kBufFlags);
#pragma unroll
    for (int i = 0; i < XCH; ++i) xv[PAR][i] = XC::load(xr, xoff[i]);
  };
  auto fetch_m_at = [&](const unsigned char* mp, bool enabled, auto par_tag) {  // ... and of its mask row
    constexpr int PAR = decltype(par_tag)::value;
    __amdgpu_buffer_rsrc_t mr = __builtin_amdgcn_make_buffer_rsrc((void*)mp, 0, enabled ? frame_m : 0u, kBufFlags);
    mv[PAR] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(mr, moff, 0, 0));
  };
  auto fetch_at = [&](const unsigned char* xp, const unsigned char* mp, bool enabled, auto par_tag) {
    fetch_x_at(xp, enabled, par_tag);
    fetch_m_at(mp, enabled, par_tag);
  };
  auto fetch = [&](int s, auto par_tag) {  // issue the loads of X[t_s] and mask[t_s] into register set PAR
    const long long t = frame_of(p, s);
    fetch_at((const unsigned char*)p.X + (size_t)t * frame_x, (const unsigned char*)p.mask + (size_t)t * frame_m, true, par_tag);
  };
  auto put = [&](auto par_tag) {  // register set PAR -> LDS copy PAR
    constexpr int PAR = decltype(par_tag)::value;
    unsigned char* xl = smem + L.xl + PAR * L.x_copy;
#pragma unroll
    for (int i = 0; i < XCH; ++i) *(typename XC::T*)(xl + xlds[i]) = xv[PAR][i];
    Ml[tid < ROWS ? PAR * ROWS + tid : 2 * ROWS] = mv[PAR];  // (no branch: the other threads write to a spare word)
  };
  // Staged outputs of a step (LDS copy `copy` of three) -> registers -> H[t], Y[t], C[t]: in two halves, so that the
  // LDS reads can be issued ahead of a batch of MFMAs and the stores behind it.
  typename XC::T fh[XCH];
  typename YC::T fy[YCH];
  typename CC::T fc[CCH];
  auto flush_read_at = [&](unsigned hs_off, unsigned ys_off, unsigned cs_off) {  // byte offsets of the copies in LDS
    const unsigned char* hs = smem + hs_off;
    const unsigned char* ys = smem + ys_off;
    const unsigned char* cs = smem + cs_off;
#pragma unroll
    for (int i = 0; i < XCH; ++i) fh[i] = *(const typename XC::T*)(hs + xlds[i]);
#pragma unroll
    for (int i = 0; i < YCH; ++i) fy[i] = *(const typename YC::T*)(ys + ylds[i]);
#pragma unroll
    for (int i = 0; i < CCH; ++i) fc[i] = *(const typename CC::T*)(cs + clds[i]);
  };
  auto flush_read = [&](int copy) { flush_read_at(L.hs + copy * L.x_copy, L.ys + copy * L.y_copy, L.cs + copy * L.c_copy); };
  auto flush_write_h = [&](unsigned char* hp, bool enabled) {
    __amdgpu_buffer_rsrc_t hr = __builtin_amdgcn_make_buffer_rsrc((void*)hp, 0, enabled ? frame_h : 0u, kBufFlags);
#pragma unroll
    for (int i = 0; i < XCH; ++i) XC::store(fh[i], hr, hoff[i]);
  };
  auto flush_write_y = [&](unsigned char* yp, bool enabled) {
    __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc((void*)yp, 0, enabled ? frame_y : 0u, kBufFlags);
#pragma unroll
    for (int i = 0; i < YCH; ++i) YC::store(fy[i], yr, yoff[i]);
  };
  auto flush_write_c = [&](unsigned char* cp, bool enabled) {
    __amdgpu_buffer_rsrc_t cr = __builtin_amdgcn_make_buffer_rsrc((void*)cp, 0, enabled ? frame_c : 0u, kBufFlags);
#pragma unroll
    for (int i = 0; i < CCH; ++i) CC::store(fc[i], cr, coff[i]);
  };
  auto flush_write_at = [&](unsigned char* hp, unsigned char* yp, unsigned char* cp, bool enabled) {
    flush_write_h(hp, enabled);
    flush_write_y(yp, enabled);
    flush_write_c(cp, enabled);
  };
  auto flush_write = [&](int s) {
    const long long t = frame_of(p, s);
    flush_write_at((unsigned char*)p.H + (size_t)t * frame_h, (unsigned char*)p.Y + (size_t)t * frame_y, (unsigned char*)p.C + (size_t)t * frame_c, true);
  };

  // ---- the recurrence
  const unsigned hx_buf_bytes = (unsigned)((size_t)n * p.Bp * sizeof(AT));
  unsigned char* hx_g = (unsigned char*)p.hx + (size_t)g * kHxRing * hx_buf_bytes;
  __amdgpu_buffer_rsrc_t ring_rs = __builtin_amdgcn_make_buffer_rsrc((void*)hx_g, 0, kHxRing * hx_buf_bytes, kBufFlags);
  const int kg = lane >> 4, jl = lane & 15;
  const int ks_count = (S > wave) ? (S - wave + kWaves - 1) / kWaves : 0;  // macro steps of this wave

  // A-operand fragments of this wave's k share: registers, for the whole sequence.  Slots past the
  // wave's share hold zeros and are paired with any complete fragment, so the step has no branches.
  // With at most 8 rows per group (HALF) the lanes of rows 8-15 of a fragment would load nothing: they take the rows of
  // the NEXT macro step instead (PAIRED), so that a wavefront's share of h comes in with half the load instructions (a
  // CU's load path takes a wavefront's load instruction at about 16 clocks whatever its width, and the four wavefronts'
  // loads are what the wait for h consists of).  The odd macro step's rows reach the lanes of rows 0-7 through a
  // shift by 8 inside each group of 16 lanes.
  constexpr bool PAIRED = HALF && NT == 1 && KSMAX % 2 == 0;
  constexpr int NLD = PAIRED ? KSMAX / 2 : KSMAX;  // loads of B fragments per step
  i32x4 wreg[MT][KSMAX];
  unsigned foff[KSMAX][NT];  // where this lane's B-operand fragments are inside a ring buffer
#pragma unroll
  for (int ks = 0; ks < KSMAX; ++ks) {
    const bool mine = ks < ks_count;
    const int sm = mine ? wave + kWaves * ks : 0;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      wreg[mt][ks] = i32x4{0, 0, 0, 0};
      if (mine) wreg[mt][ks] = ((const i32x4*)p.Wp)[((size_t)(r * MT + mt) * S + sm) * 64 + lane];
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      // Lanes of rows the group does not have load nothing: an out-of-range offset gives zeros (a complete fragment)
      // without a memory access, so a group of few rows moves few bytes.
      foff[ks][nt] = (mine && 16 * nt + jl < rows) ? (unsigned)(((4 * sm + kg) * p.Bp + 16 * nt + jl) * kFragBytes) : kOobOffset;
    }
  }
  if constexpr (PAIRED) {
#pragma unroll
    for (int a = 0; a < NLD; ++a) {
      const int ks = 2 * a + ((jl >> 3) & 1);
      const bool mine = ks < ks_count;
      const int sm = mine ? wave + kWaves * ks : 0;
      foff[a][0] = (mine && (jl & 7) < rows) ? (unsigned)(((4 * sm + kg) * p.Bp + (jl & 7)) * kFragBytes) : kOobOffset;
    }
  }

  // The (sequence, cell) pairs whose state this thread keeps.
  float c_state[EPT], h_prev[EPT];
  bool e_valid[EPT];
  unsigned e_hoff[EPT];            // byte offset of the pair's element in an exchange buffer
  unsigned e_row[EPT], e_cl[EPT];  // row and cell inside the workgroup's tile
  unsigned e_tile[EPT], e_src[EPT];  // tile and lane of the partial sums of the pair
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int u = min(wave + kWaves * j, UNITS - 1);
    int e, bl, src;
    if (HALF) {
      e = 2 * u + ((lane >> 3) & 1);
      bl = lane & 7;
      src = (lane & 0x30) | bl;
    } else {
      e = u;
      bl = 16 * (e % NT) + (lane & 15);
      src = lane;
    }
    const int mt = e / NT;
    const int cell = 4 * (r * MT + mt) + (lane >> 4);
    e_tile[j] = (unsigned)e;
    e_src[j] = (unsigned)src;
    e_row[j] = (unsigned)bl;
    e_cl[j] = (unsigned)(4 * mt + (lane >> 4));
    e_valid[j] = (wave + kWaves * j < UNITS) && (bl < rows);
    e_hoff[j] = (unsigned)((((cell / KE) * p.Bp + bl) * KE + (cell % KE)) * ES);
    c_state[j] = 0.f;
    h_prev[j] = 0.f;
    if (e_valid[j]) {
      const long long bc = (long long)(b_base + bl) * n + cell;
      c_state[j] = p.c0[bc];
      h_prev[j] = E::load(p.y0, bc);
    }
  }

  // An XCD-local plan rests on all workgroups of the group being on one XCD.  Check it: every workgroup adds its XCD
  // to the group's mask and then itself to the group's count (two words the prepare kernel cleared; device-scope
  // atomics whose result is waited for, so the mask is complete when the count is); with one XCD in the mask the hidden
  // state travels through that XCD's L2 (plain stores, loads that bypass the first-level cache), else with device scope.
  __shared__ int s_local;
  if (multi.local && tid == 0)
    s_local = group_on_one_xcd(p.flags + (size_t)g * p.wgs_per_group, (unsigned)p.wgs_per_group, p.status, p.timeout_ticks) ? 1 : 0;

  auto run = [&](auto ex_tag) {
    constexpr int EX = decltype(ex_tag)::value;
    // Exchange loads always bypass the first-level cache (device scope).  Stores: through to memory (device scope), or,
    // when the whole group shares an XCD, plain stores that stay in that XCD's L2, where the loads find them.
    constexpr int AUXS = (EX == kExDevice) ? kAuxDevice : 0, AUXL = kAuxDevice;
    i32x4 bf[KSMAX][NT];
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) bf[ks][nt] = i32x4{0, 0, 0, 0};
    // Issue the loads of this wave's fragments of ring buffer s%4.  Lanes of rows the group does not have are switched
    // off (their registers keep the zeros from above: a complete fragment): the address unit spends its cycles on the
    // active lanes only, and a wavefront's eight loads are what a CU's address unit is busy with for most of the read.
    auto issue = [&](int s) {
      const unsigned soff = (unsigned)(s & (kHxRing - 1)) * hx_buf_bytes;
      asm volatile("" ::: "memory");  // other workgroups write this memory: really load again
      if constexpr (EX == kExNoWait) return;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        if ((PAIRED ? (jl & 7) : 16 * nt + jl) < rows) {
#pragma unroll
          for (int ks = 0; ks < NLD; ++ks)
            bf[ks][nt] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(ring_rs, foff[ks][nt], soff, AUXL));
        }
    };
    // This thread's gate inputs and mask of a step, read from the LDS copy PAR into register set PAR (as stored; they
    // are widened where they are used, so that the reads can all be in flight together).
    AT x_in[2][EPT][4];
    float m_in[2][EPT];
    auto load_gate_inputs = [&](auto par_tag) {
      constexpr int PAR = decltype(par_tag)::value;
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
        const unsigned char* xin = smem + L.xl + PAR * L.x_copy + e_row[j] * L.x_row + e_cl[j] * ES;
#pragma unroll
        for (int q = 0; q < 4; ++q) x_in[PAR][j][q] = *(const AT*)(xin + q * SEG);
        m_in[PAR][j] = Ml[PAR * ROWS + e_row[j]];
      }
    };
    // What the pointwise part needs of this step's gate inputs, the mask and the carried state, made ready in the shadow
    // of the MFMAs (they were read from LDS one step ago, the state is that of the step before): the gate inputs as
    // float32, 1 - mask and its products with the carried cell state and output.
    float x_f[EPT][4], m_f[EPT], keep_c[EPT], keep_h[EPT];
    auto widen_gate_inputs = [&](auto par_tag) {
      constexpr int PAR = decltype(par_tag)::value;
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) x_f[j][q] = (float)x_in[PAR][j][q];
        m_f[j] = m_in[PAR][j];
        const float om = 1.f - m_f[j];
        keep_c[j] = c_state[j] * om;
        keep_h[j] = h_prev[j] * om;
      }
    };
    RTN_TRACE_DECL
    unsigned char *h_out = nullptr, *y_out_p = nullptr, *c_out = nullptr;
    const unsigned char *x_next = nullptr, *m_next = nullptr;
    // in units of s_sleep(1), about 64 clocks; see below.  (A group that was planned for one XCD and found itself on
    // several takes the numbers of a spread plan.)
    const bool spread_after_all = multi.local && EX == kExDevice;
    int delay = EX == kExNoWait ? 0 : spread_after_all ? 20 : p.poll_delay;
    const int delay_inc = spread_after_all ? 2 : p.delay_inc;
    // One time step; PAR = s & 1 selects the register sets and the LDS copies of X, `stage` = s % 3 the copy that
    // takes this step's outputs.
    //
    // The step's critical path is: h_{s-1} arrives -> MFMAs -> partial tiles through LDS (the one barrier) -> gates ->
    // new hidden values out.  Everything else rides in the shadow of the MFMAs, which a wavefront issues at one per 16
    // clocks with nothing else to do in between: the outputs of step s-2 go from LDS to memory (their staging and this
    // point are separated by the barrier of step s-1), the gate inputs of step s+1 come from LDS into the other
    // register set, X[t_{s+2}] moves from registers to LDS and X[t_{s+4}] from memory into the registers that became
    // free.  LDS reads are issued ahead of a batch of MFMAs and used behind it.
    auto step = [&](int s, auto par_tag, int stage) {
      constexpr int PAR = decltype(par_tag)::value;
      // Where the step's staged outputs go and where those of step s-2 lie in LDS: scalar arithmetic done here, while the
      // read of h is in flight, and not among the first MFMAs (the empty assembly statement keeps it here).
      const int rd_copy = stage == 2 ? 0 : stage + 1;  // the copy of step s-2 is (s+1) % 3
      unsigned rd_h = L.hs + rd_copy * L.x_copy, rd_y = L.ys + rd_copy * L.y_copy, rd_c = L.cs + rd_copy * L.c_copy;
      unsigned st_h = L.hs + stage * L.x_copy, st_y = L.ys + stage * L.y_copy, st_c = L.cs + stage * L.c_copy;
      asm volatile("" : "+s"(rd_h), "+s"(rd_y), "+s"(rd_c), "+s"(st_h), "+s"(st_y), "+s"(st_c));

      // Complete this wave's share of h_{s-1}: if anything that came back is not written yet, read again.
      // (Four independent running maxima: a single chain of dependent packed operations needs a wait state after
      // every one of them.)
      unsigned long long t0 = 0;
      unsigned spins = 0;
      for (;;) {
        unsigned m[4] = {0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < NLD; ++ks)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int w = 0; w < 4; ++w) m[w] = LM::fold(m[w], (unsigned)bf[ks][nt][w]);
        const unsigned seen = LM::fold(LM::fold(m[0], m[1]), LM::fold(m[2], m[3]));
        if (EX == kExNoWait || !__any(LM::has_sentinel(seen))) break;
        if ((spins++ & 15u) == 0) {
          if (__hip_atomic_load(p.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
          const unsigned long long now = wall_clock64();
          if (spins == 1) {
            t0 = now;
          } else if (now - t0 > p.timeout_ticks) {
            __hip_atomic_store(p.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
        }
        issue(s);
      }
      RTN_TRACE_MARK(0)  // wait for h_{s-1}
      // Everything this wave stored before (re-arm stores included) is acknowledged, and X[t_{s+2}],
      // fetched two steps ago, is in its registers.
      // (The builtin rather than inline assembly, so that the compiler's own wait-count bookkeeping sees it.)
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      asm volatile("" ::: "memory");
      // The first read is held back by `delay`: a read that comes back incomplete costs an extra round trip, waiting too
      // long costs the wait itself.  Across XCDs a round trip is long, and the delay adapts: longer by `delay_inc` when a
      // read had to be repeated, shorter by one unit every (delay_dec_mask + 1) steps while none has; the repeat rate
      // settles where the two balance.  Within an XCD a repeat is cheap (a read from the L2 next
      // door), and what costs is wavefronts drifting apart, each on a delay of its own, where every step ends with the
      // slowest of them: there the delay is one number for all (delay_inc == 0).
      if (spins)
        delay = min(delay + delay_inc, 64);
      else if (delay_inc && (s & p.delay_dec_mask) == p.delay_dec_mask && delay > 0)
        --delay;
      RTN_TRACE_MARK(7)  // outstanding stores acknowledged
      RTN_TRACE_ADD(6, spins)

      RedBuf& redbuf = red[PAR];
      // PAIRED: ONE accumulator for every two tiles.  A group of at most 8 rows fills columns 0-7 of a tile and leaves
      // columns 8-15 to padding; with the B operand of tile 2u holding the rows in columns 0-7 and zeros in columns 8-15,
      // and that of tile 2u+1 the same rows in columns 8-15 and zeros in 0-7, both tiles' MFMAs can add into the same
      // accumulator: columns 0-7 collect tile 2u, columns 8-15 tile 2u+1 (the other tile contributes exact zeros, so
      // every sum is bit for bit what a tile of its own would hold).  Half the accumulators, half the partial tiles
      // through LDS -- written by all 64 lanes, in the very lane order the pointwise part reads them in.
      constexpr int NACC = PAIRED ? MT / 2 : MT;
      f32x4 acc[NACC][NT];
#pragma unroll
      for (int mt = 0; mt < NACC; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
      // Everything that is not on the path h -> MFMA -> gates -> h rides in the shadow of the MFMAs: all of it without
      // a branch (a frame that does not exist is a buffer of no bytes; LDS copies nobody reads may take anything), in
      // one block of straight-line code that the scheduler is told to weave.  A wavefront that has a SIMD to itself
      // issues its instructions one after the other, and a 16-clock MFMA takes two issue turns of 4 clocks, a vector
      // instruction one (k_mfma_issue with OTHERS = 0 ... 3 vector instructions behind every MFMA: an MFMA every
      // 16.2 / 16.6 / 16.7 / 20.7 clocks): two other instructions fit behind every MFMA for free, and a run of them
      // between two MFMAs drains the matrix core.
      // PAIRED: a loaded register holds macro step 2a in the lanes of rows 0-7 and step 2a+1 in the lanes of rows 8-15 of
      // every group of 16 lanes.  Four B operands are made of it: each step's rows in columns 0-7 (for the even tiles)
      // and in columns 8-15 (for the odd tiles), zeros in the other half -- a mask where the rows stay, a row shift by 8
      // lanes (data parallel primitive; lanes without a source take 0) where they move.
      if constexpr (PAIRED) {
        // The MFMAs go in chunks of NACC -- one per accumulator: (macro step, even tiles), (macro step, odd tiles), ... --
        // so that two MFMAs into the same accumulator are NACC apart.  The compiler's scheduler would otherwise line up
        // the MFMAs of one accumulator, each waiting for the one before; nothing moves from one chunk to another
        // (sched_barrier), and the step's other work is dealt to the chunks by hand: the B operand of the next chunk
        // (four vector instructions) and one piece of the stream work each, woven between the chunk's MFMAs.
        constexpr int NCH = 2 * KSMAX;
        const int keep_lo = (jl & 8) ? 0 : -1, keep_hi = ~keep_lo;
        auto operand = [&](int c) {  // chunk c: macro step c / 2, rows in columns 0-7 (even tiles) or 8-15 (odd tiles)
          const int ks = c >> 1, odd = c & 1;
          const i32x4 src = bf[ks >> 1][0];
          i32x4 r;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            if (!(ks & 1))
              r[w] = odd ? __builtin_amdgcn_update_dpp(0, src[w], 0x118 /* row_shr:8 */, 0xF, 0xF, true) : (src[w] & keep_lo);
            else
              r[w] = odd ? (src[w] & keep_hi) : __builtin_amdgcn_update_dpp(0, src[w], 0x108 /* row_shl:8 */, 0xF, 0xF, true);
          }
          return r;
        };
        i32x4 opnd = operand(0);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int ks = c >> 1, odd = c & 1;
          i32x4 opnd_next = opnd;
          if (c + 1 < NCH) opnd_next = operand(c + 1);
          // (eight instructions fit behind a chunk's four MFMAs, four of them the next operand's; with fewer chunks the last one takes the rest)
          auto at = [&](int want) { return c == (want < NCH ? want : NCH - 1); };
          if (at(0)) flush_read_at(rd_h, rd_y, rd_c);
          if (at(1)) load_gate_inputs(IntTag<1 - PAR>{});
          if (at(2)) put(par_tag);
          if (at(3)) flush_write_h(h_out, s >= 2);
          if (at(4)) flush_write_y(y_out_p, s >= 2);
          if (at(5)) flush_write_c(c_out, s >= 2);
          if (at(6)) fetch_x_at(x_next, s + 4 < nsteps, par_tag);
          if (at(7)) fetch_m_at(m_next, s + 4 < nsteps, par_tag);
          if (at(8)) widen_gate_inputs(par_tag);
#pragma unroll
          for (int u = 0; u < NACC; ++u) {
            acc[u][0] = E::mma(wreg[2 * u + odd][ks], opnd, acc[u][0]);
            __builtin_amdgcn_sched_group_barrier(0x008, sizeof(AT) == 2 ? 1 : 4, 0);  // the MFMA(s) of one fragment ...
            __builtin_amdgcn_sched_group_barrier(0x096, 2, 0);                        // ... then up to two of the rest (three: 0-1 % slower; four or five: 2-3 %)
          }
          __builtin_amdgcn_sched_barrier(0);
          opnd = opnd_next;
        }
      } else {
        flush_read_at(rd_h, rd_y, rd_c);
        load_gate_inputs(IntTag<1 - PAR>{});
        put(par_tag);
        flush_write_at(h_out, y_out_p, c_out, s >= 2);
        fetch_at(x_next, m_next, s + 4 < nsteps, par_tag);
        widen_gate_inputs(par_tag);
#pragma unroll
        for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              acc[mt][nt] = E::mma(wreg[mt][ks], bf[ks][nt], acc[mt][nt]);
              __builtin_amdgcn_sched_group_barrier(0x008, sizeof(AT) == 2 ? 1 : 4, 0);  // the MFMA(s) of one fragment ...
              __builtin_amdgcn_sched_group_barrier(0x096, 3, 0);                        // ... then up to three of the rest (VALU, SALU, VMEM, LDS)
            }
      }
      h_out += step_h; y_out_p += step_y; c_out += step_c; x_next += step_x; m_next += step_m;
      if constexpr (PAIRED) {
#pragma unroll
        for (int u = 0; u < NACC; ++u) redbuf[wave][u][lane] = acc[u][0];
      } else if (!HALF || (lane & 8) == 0) {  // (with at most 8 rows only the lanes of rows 0..7 hold columns anybody reads)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) redbuf[wave][mt * NT + nt][lane] = acc[mt][nt];
      }
      RTN_TRACE_MARK(1)  // MFMA with the streams in their shadow, partial tiles to LDS
      __syncthreads();  // the one barrier of a step: partial tiles, X[t_{s+2}] and the outputs of step s-1 are in LDS
      RTN_TRACE_MARK(2)  // barrier

      // Gates and cell update, then straight away the new hidden values.
      unsigned h_bits[EPT];
      float g_act[EPT][4], y_out[EPT];
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
        h_bits[j] = 0;
        if (UNITS % kWaves == 0 || wave + kWaves * j < UNITS) {  // wave-uniform
          // (all four partial tiles on their way before the first is used: the compiler, left alone, reads them one
          // after the other through one set of registers and pays the LDS latency three times)
          f32x4 part[kWaves];
#pragma unroll
          for (int w = 0; w < kWaves; ++w) part[w] = PAIRED ? redbuf[w][wave + kWaves * j][lane] : redbuf[w][e_tile[j]][e_src[j]];
          __builtin_amdgcn_sched_barrier(0);
          f32x4 gsum = part[0];
#pragma unroll
          for (int w = 1; w < kWaves; ++w) gsum += part[w];
          const float m = m_f[j];
          const float a0 = Act<AT>::tanh(gsum[0] + x_f[j][0]);
          const float a1 = Act<AT>::sigmoid(gsum[1] + x_f[j][1]);
          const float a2 = Act<AT>::sigmoid(gsum[2] + x_f[j][2]);
          const float a3 = Act<AT>::sigmoid(gsum[3] + x_f[j][3]);
          const float pc = c_state[j];
          const float c = (pc * a2 + a0 * a1) * m + keep_c[j];   // keep_c = pc * (1 - m)
          const float y = E::round(Act<AT>::tanh(c) * a3 * m);
          const float hn = (p.op_flags & kOpNoCarry) ? y : E::round(y + keep_h[j]);  // keep_h = h_prev * (1 - m)
          c_state[j] = c;
          h_prev[j] = hn;
          h_bits[j] = SN::bits(hn);
          g_act[j][0] = (p.op_flags & kOpH0IsCell) ? c : a0;
          g_act[j][1] = a1; g_act[j][2] = a2; g_act[j][3] = a3;
          y_out[j] = y;
        }
      }
      // New hidden values out; re-arm the elements everybody read one step ago.
      // (Rows the group does not have own slots of the exchange buffers too, so no lane is switched off.)
      {
        const unsigned nxt = (unsigned)((s + 1) & (kHxRing - 1)) * hx_buf_bytes;
        const unsigned arm = (unsigned)((s + 3) & (kHxRing - 1)) * hx_buf_bytes;
#pragma unroll
        for (int j = 0; j < EPT; ++j)
          if (UNITS % kWaves == 0 || wave + kWaves * j < UNITS) SN::template store<AUXS>(ring_rs, e_hoff[j] + nxt, h_bits[j]);
#pragma unroll
        for (int j = 0; j < EPT; ++j)
          if (UNITS % kWaves == 0 || wave + kWaves * j < UNITS) SN::template store<AUXS>(ring_rs, e_hoff[j] + arm, SN::kSentinel);
      }
      RTN_TRACE_MARK(3)  // gates, cell update, exchange stores
      // While the new hidden values travel: stage the op's outputs of this step (they leave two steps from now), and
      // after the delay issue the first read of the next step.
#pragma unroll
      for (int j = 0; j < EPT; ++j) {
        if (UNITS % kWaves == 0 || wave + kWaves * j < UNITS) {
          unsigned char* hq = smem + st_h + e_row[j] * L.x_row + e_cl[j] * ES;
#pragma unroll
          for (int q = 0; q < 4; ++q) *(AT*)(hq + q * SEG) = (AT)g_act[j][q];
          *(AT*)(smem + st_y + e_row[j] * L.y_row + e_cl[j] * ES) = (AT)y_out[j];
          *(float*)(smem + st_c + e_row[j] * L.c_row + e_cl[j] * 4) = c_state[j];
        }
      }
      if (s + 1 < nsteps) {
        for (int k = 0; k < delay; ++k) __builtin_amdgcn_s_sleep(1);
        issue(s + 1);
      }
      RTN_TRACE_MARK(4)  // staging, delay, first read of the next step
    };
    fetch(0, IntTag<0>{});
    if (nsteps > 1) fetch(1, IntTag<1>{});
    put(IntTag<0>{});
    if (nsteps > 1) put(IntTag<1>{});
    __syncthreads();
    load_gate_inputs(IntTag<0>{});
    if (nsteps > 2) fetch(2, IntTag<0>{});
    if (nsteps > 3) fetch(3, IntTag<1>{});
    __syncthreads();  // everybody has the gate inputs of step 0: its LDS copy may take X[t_2]
    issue(0);
    int stage = 0;
    // frames of the outputs of step s-2 and of the inputs of step s+4, as the loop reaches step s
    h_out = (unsigned char*)p.H + (frame_of(p, 0) - 2 * (long long)p.step) * (long long)frame_h;
    y_out_p = (unsigned char*)p.Y + (frame_of(p, 0) - 2 * (long long)p.step) * (long long)frame_y;
    c_out = (unsigned char*)p.C + (frame_of(p, 0) - 2 * (long long)p.step) * (long long)frame_c;
    x_next = (const unsigned char*)p.X + frame_of(p, 4) * (long long)frame_x;
    m_next = (const unsigned char*)p.mask + frame_of(p, 4) * (long long)frame_m;
    for (int s = 0; s < nsteps; s += 2) {
      step(s, IntTag<0>{}, stage);
      stage = stage == 2 ? 0 : stage + 1;
      if (s + 1 < nsteps) {
        step(s + 1, IntTag<1>{}, stage);
        stage = stage == 2 ? 0 : stage + 1;
      }
    }
    RTN_TRACE_ADD(6, (unsigned long long)delay << 40)
    RTN_TRACE_FLUSH(p, trace_id)
  };
  __syncthreads();  // s_local
  if (p.exchange == kExNoWait) {
    if (tid == 0) __hip_atomic_store(p.status, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    run(IntTag<kExNoWait>{});
  } else if (multi.local && s_local) {
    run(IntTag<kExLocal>{});
  } else {
    run(IntTag<kExDevice>{});
  }
  __syncthreads();  // the last step's outputs are staged
  if (nsteps >= 2) {
    flush_read((nsteps - 2) % 3);
    flush_write(nsteps - 2);
  }
  flush_read((nsteps - 1) % 3);
  // A wait that ran into its bound let the recurrence go on with values that are wrong without looking it.  Whoever
  // consumes the outputs without asking for the status must still notice: the workgroups that see the mark hand out
  // NaN as the final cell state and as the last visited frame of Y.
  const bool expired = wait_expired(p.status);
  if (expired) {
#pragma unroll
    for (int i = 0; i < YCH; ++i) fy[i] = YC::fill(kNanWords<AT>);
  }
  flush_write(nsteps - 1);

#pragma unroll
  for (int j = 0; j < EPT; ++j)
    if (e_valid[j]) p.d[(long long)(b_base + e_row[j]) * n + 4 * MT * r + e_cl[j]] = expired ? __builtin_nanf("") : c_state[j];
}


// Measurement aid: what the matrix cores of the device can do on the step's own instruction sequence when nothing has
// to come from another workgroup.  Every workgroup of the plan's grid runs `steps` steps of what k_lstm2_regw does
// between the arrival of h and the pointwise part: the B-operand fragments of its k share from LDS (the same
// fragments every step: there is no recurrence; with groups of at most 8 rows: as loaded pairs that are masked and
// shifted into the four operand forms, like the kernel does), MT * NT * KSMAX MFMAs per wavefront against W fragments held in
// registers, the partial tiles through LDS with the step's one barrier, and their sum in wave order (kept as a running
// value so that nothing can be dropped).  No exchange, no streams, no pointwise arithmetic.  The time of a launch over
// the op's algorithmic flops is the MFMA roofline a kernel of this decomposition could reach at most.
template <typename AT, int MT, int NT, int KSMAX, bool HALF>
__global__ __launch_bounds__(kWgThreads) void k_mfma_sequence(float* out, int steps) {
  using E = Elem<AT>;
  constexpr int TILES = MT * NT;
  constexpr int UNITS = HALF ? TILES / 2 : TILES;
  constexpr int EPT = (UNITS + kWaves - 1) / kWaves;
  extern __shared__ __align__(16) unsigned char smem[];
  typedef f32x4 RedBuf[kWaves][TILES][64];
  RedBuf* red = (RedBuf*)smem;                                                // [2]
  i32x4* Bl = (i32x4*)(smem + 2 * sizeof(RedBuf));                            // [kWaves][KSMAX][NT][64]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // operands: small numbers that differ per lane and slot (their values do not matter, their being there does)
  i32x4 wreg[MT][KSMAX];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      const AT v = (AT)(0.001f * (float)(1 + ((lane + 3 * mt + 5 * ks + 7 * wave) & 15)));
      AT frag[E::KE];
#pragma unroll
      for (int e = 0; e < E::KE; ++e) frag[e] = v;
      wreg[mt][ks] = __builtin_bit_cast(i32x4, frag);
    }
#pragma unroll
  for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      AT frag[E::KE];
#pragma unroll
      for (int e = 0; e < E::KE; ++e) frag[e] = (AT)(0.01f * (float)(1 + ((lane + ks + nt + e) & 7)));
      Bl[((wave * KSMAX + ks) * NT + nt) * 64 + lane] = __builtin_bit_cast(i32x4, frag);
    }
  __syncthreads();
  f32x4 total = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr bool PAIRED = HALF && NT == 1 && KSMAX % 2 == 0;  // as in k_lstm2_regw: two tiles share an accumulator
  constexpr int NLD = PAIRED ? KSMAX / 2 : KSMAX;
  constexpr int NACC = PAIRED ? MT / 2 : MT;
  auto step = [&](auto par_tag) {
    constexpr int PAR = decltype(par_tag)::value;
    RedBuf& redbuf = red[PAR];
    i32x4 bf[KSMAX][NT];
    asm volatile("" ::: "memory");  // read the fragments again every step
#pragma unroll
    for (int ks = 0; ks < NLD; ++ks)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) bf[ks][nt] = Bl[((wave * KSMAX + ks) * NT + nt) * 64 + lane];
    f32x4 acc[NACC][NT];
#pragma unroll
    for (int mt = 0; mt < NACC; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (PAIRED) {
      i32x4 b_lo[KSMAX + 1], b_hi[KSMAX + 1];
      const int keep_lo = (lane & 8) ? 0 : -1, keep_hi = ~keep_lo;
#pragma unroll
      for (int a = 0; a < NLD; ++a)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          b_lo[2 * a][w] = bf[a][0][w] & keep_lo;
          b_hi[2 * a][w] = __builtin_amdgcn_update_dpp(0, bf[a][0][w], 0x118 /* row_shr:8 */, 0xF, 0xF, true);
          b_lo[2 * a + 1][w] = __builtin_amdgcn_update_dpp(0, bf[a][0][w], 0x108 /* row_shl:8 */, 0xF, 0xF, true);
          b_hi[2 * a + 1][w] = bf[a][0][w] & keep_hi;
        }
#pragma unroll
      for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
        for (int odd = 0; odd < 2; ++odd)
#pragma unroll
          for (int u = 0; u < NACC; ++u) acc[u][0] = E::mma(wreg[2 * u + odd][ks], odd ? b_hi[ks] : b_lo[ks], acc[u][0]);
#pragma unroll
      for (int u = 0; u < NACC; ++u) redbuf[wave][u][lane] = acc[u][0];
    } else {
#pragma unroll
      for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = E::mma(wreg[mt][ks], bf[ks][nt], acc[mt][nt]);
      if (!HALF || (lane & 8) == 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) redbuf[wave][mt * NT + nt][lane] = acc[mt][nt];
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      if (UNITS % kWaves == 0 || wave + kWaves * j < UNITS) {
        const int u = wave + kWaves * j;
        const int e = HALF ? 2 * u + ((lane >> 3) & 1) : u;
        const int src = HALF ? ((lane & 0x30) | (lane & 7)) : lane;
        f32x4 part[kWaves];
#pragma unroll
        for (int w = 0; w < kWaves; ++w) part[w] = PAIRED ? redbuf[w][u][lane] : redbuf[w][e][src];
        __builtin_amdgcn_sched_barrier(0);
        f32x4 g = part[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) g += part[w];
        total += g;
      }
    }
  };
  for (int s = 0; s < steps; s += 2) {
    step(IntTag<0>{});
    if (s + 1 < steps) step(IntTag<1>{});
  }
  out[(size_t)blockIdx.x * kWgThreads + tid] = total[0] + total[1] + total[2] + total[3];
}

// Measurement aid: the matrix cores alone.  Every workgroup of the plan's grid issues, per step, the MT * NT * KSMAX MFMAs
// of one wavefront's share -- the plan's tile sequence, in the op's order (macro steps outside, tiles inside), W fragments
// and B fragments in registers -- and nothing else: no LDS, no barrier, no sum over the wavefronts, no loads.  (The
// accumulators start at zero in every step, as the op's do, and end in an empty assembly statement that stands for their
// use; the B fragments pass through another one every step, so that the compiler cannot take a step's work for a
// repetition of the last.  Accumulators that run on from step to step instead cost a round of register copies at the
// loop's back edge, a fifth of the step, that no kernel of the op has.)  The time of
// a launch over the op's algorithmic flops is what the matrix cores can reach on this tile sequence: the ceiling of the
// recurrent GEMM that no arrangement of the rest of the step can exceed.
// OTHERS > 0: that many vector instructions (register moves) behind every MFMA -- what a wavefront can issue in an
// MFMA's shadow before the matrix core has to wait for it.
template <typename AT, int MT, int NT, int KSMAX, int THREADS = kWgThreads, int OTHERS = 0>
__global__ __launch_bounds__(THREADS) void k_mfma_issue(float* out, int steps) {
  using E = Elem<AT>;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  i32x4 wreg[MT][KSMAX], bf[KSMAX][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      AT frag[E::KE];
#pragma unroll
      for (int e = 0; e < E::KE; ++e) frag[e] = (AT)(0.001f * (float)(1 + ((lane + 3 * mt + 5 * ks + 7 * wave + e) & 15)));
      wreg[mt][ks] = __builtin_bit_cast(i32x4, frag);
    }
#pragma unroll
  for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      AT frag[E::KE];
#pragma unroll
      for (int e = 0; e < E::KE; ++e) frag[e] = (AT)(0.01f * (float)(1 + ((lane + ks + nt + e) & 7)));
      bf[ks][nt] = __builtin_bit_cast(i32x4, frag);
    }
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};  // (steps == 0)
  int moved = 0;
  const unsigned long long clk0 = clock64(), wall0 = wall_clock64();
  for (int s = 0; s < steps; ++s) {
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) asm volatile("" : "+v"(bf[ks][nt]));
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          acc[mt][nt] = E::mma(wreg[mt][ks], bf[ks][nt], acc[mt][nt]);
          if constexpr (OTHERS > 0) {  // (fenced: the moves stay behind their MFMA)
            if constexpr (OTHERS == 1) asm volatile("v_mov_b32 %0, %1" : "=v"(moved) : "v"(lane));
            if constexpr (OTHERS == 2) asm volatile("v_mov_b32 %0, %1\n\tv_mov_b32 %0, %1" : "=v"(moved) : "v"(lane));
            if constexpr (OTHERS >= 3) asm volatile("v_mov_b32 %0, %1\n\tv_mov_b32 %0, %1\n\tv_mov_b32 %0, %1" : "=v"(moved) : "v"(lane));
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) asm volatile("" : "+a"(acc[mt][nt]));
  }
  f32x4 total = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) total += acc[mt][nt];
  // Thread 0 leaves the sum (so that nothing can be dropped), threads 1 and 2 what the loop took in shader clocks and in
  // ticks of the constant 100 MHz clock: their ratio is the clock rate the matrix cores ran at under this load.
  const unsigned long long clk1 = clock64(), wall1 = wall_clock64();
  float v = total[0] + total[1] + total[2] + total[3] + (float)moved;
  if (tid == 1) v = (float)(clk1 - clk0);
  if (tid == 2) v = (float)(wall1 - wall0);
  if (tid < kWgThreads) out[(size_t)blockIdx.x * kWgThreads + tid] = v;
}

// Measurement aid: the latency of handing a value from every workgroup to every other one, the way the persistent
// kernel hands over the hidden state (device-scope store, device-scope load until the value is there), with nothing
// else going on: G workgroups on G CUs; per round each stores its 256-byte block of ring buffer round%4 (value =
// round number) and reads all G blocks, 16 lanes per block, until every word carries the round number; one
// workgroup barrier per round.  A value from an earlier use of the buffer differs from the round number, so a
// stale read can only cost a retry.  G <= 16.  status[0] is set to 1 if a wait runs into `timeout_ticks`.
static __global__ __launch_bounds__(kWgThreads) void k_handover_latency(unsigned* ring, unsigned* status, int G, int rounds,
                                                                 unsigned long long timeout_ticks) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = blockIdx.x;
  const unsigned buf_bytes = (unsigned)G * 256u;
  __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)ring, 0, 4 * buf_bytes, kBufFlags);
  const int blk = wave * 4 + (lane >> 4);  // the block this lane reads a 16-byte piece of
  const unsigned roff = blk < G ? (unsigned)blk * 256u + (unsigned)(lane & 15) * 16u : kOobOffset;
  for (int s = 1; s <= rounds; ++s) {
    const unsigned base = (unsigned)(s & 3) * buf_bytes;
    const unsigned v = (unsigned)s;
    if (tid < 64) __builtin_amdgcn_raw_buffer_store_b32(v, rs, base + (unsigned)r * 256u + (unsigned)tid * 4u, 0, kAuxDevice);
    unsigned long long t0 = 0;
    unsigned spins = 0;
    for (;;) {
      asm volatile("" ::: "memory");
      const i32x4 x = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, roff, base, kAuxDevice));
      const bool ok = blk >= G || ((unsigned)x[0] == v && (unsigned)x[1] == v && (unsigned)x[2] == v && (unsigned)x[3] == v);
      if (__all(ok)) break;
      if ((spins++ & 15u) == 0) {
        if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
        const unsigned long long now = wall_clock64();
        if (spins == 1) {
          t0 = now;
        } else if (now - t0 > timeout_ticks) {
          __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
    }
    __syncthreads();
  }
}

}  // namespace rtn
