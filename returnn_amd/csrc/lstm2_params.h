// Parameter block shared by the host driver and the gfx950 kernels of the NativeLstm2 forward op.
#pragma once

#include <stdint.h>

namespace rtn {

// How the hidden state is made visible between workgroups in the persistent kernel.
// A valid policy has (store_coherent || release_fence) and (load_coherent || acquire_fence).
enum SyncBits : int {
  kStoreCoherent = 1,  // publish h with device-scope write-through stores
  kReleaseFence = 2,   // device-scope release fence (L2 write-back) before the flag store
  kLoadCoherent = 4,   // read h with device-scope loads that bypass non-coherent caches
  kAcquireFence = 8,   // device-scope acquire fence (cache invalidate) after the flag wait
};

// Variations of the recurrence shared with NativeLstm2's sibling ops.
enum OpFlags : int {
  kOpNoCarry = 1,    // the recurrent input of a frame is the OUTPUT of the frame before (0 where that frame was masked),
                     // not the last valid output carried over masked frames (LstmGenericBase, LstmLowMem)
  kOpH0IsCell = 2,   // the first block of H holds the cell state instead of tanh(cell-in) (LstmGenericBase)
  kOpRawDh = 8,      // gradient kernels: the error arriving from the frame processed before is added to the output's error
                     // unmasked (d_y = DY * mask + d_h) and the derivatives handed to the initial output are those of the
                     // first visited frame alone: the LstmLowMem gradient as the reference has it (returnn/native_op.py:679)
  kOpEndAtStart = 4, // host side only: with a negative step the loop runs from frame T-start-1 down to frame `start`,
                     // not down to frame 0 (LstmLowMem's loop bounds, returnn/native_op.py:827-833)
};

struct Lstm2Params {
  // inputs (device)
  const void* X;      // [T,B,4n] AT
  const void* W;      // [n,4n] AT (row major, as given by the caller)
  const void* y0;     // [B,n] AT
  const float* c0;    // [B,n]
  const float* mask;  // [T,B]
  // outputs (device)
  void* Y;   // [T,B,n] AT
  float* C;  // [T,B,n]
  void* H;   // [T,B,4n] AT
  float* d;  // [B,n]
  // workspace sections (device)
  unsigned* status;  // [64]   status[0] != 0: a bounded wait expired
  unsigned* flags;   // [groups_total*wgs_per_group] last published step (+1) of each workgroup
  void* hx;          // [groups_total][hx_bufs][n/KE][Bp][KE] AT: hidden state in MFMA B-operand order, ring of buffers
  void* Wp;          // [n/4][S][64][16 bytes]: W in MFMA A-operand order
  void* ycarry;      // [2][B][n] AT: hidden-state carry of the generic per-step kernels
  // sizes
  long long T;
  long long ldX;  // elements between the rows of X of two consecutive (frame, sequence) pairs: 4n when X is contiguous; more when
                  // the caller's rows are wider (e.g. [T*B, 8n]: the pre-projected gates of two directions side by side)
  long long ldY;  // the same for the rows of Y: n when contiguous (2n: the two directions of a layer write into one [T,B,2n] array)
  int B, n;
  int first;   // first visited frame
  int step;    // signed stride between visited frames
  int nsteps;  // number of visited frames
  // decomposition of the MFMA kernels
  int groups;         // independent batch groups worked on by this launch
  int group_offset;   // index of the launch's first group (a large batch runs as several persistent launches in turn)
  int groups_total;   // groups of the whole problem: the workspace sections are laid out for all of them
  int wgs_per_group;  // workgroups per group (each owns MT*4 cells)
  int Bg;             // batch rows per group
  int Bp;             // rows of one hx buffer (= 16*NT)
  int hx_bufs;        // buffers in the hx ring: 2 with the flag barrier, 4 with self-validating data
  int hx_sentinel;    // 1: buffers 1.. start filled with the "not yet written" bit pattern (all ones)
  int xcds;           // XCDs assumed for the blockIdx -> (group, rank) mapping
  int exchange;       // register kernel: 0 = normal operation; 3, 4 = measurement aids (see kExNoWait, kExProbe)
  int poll_delay;     // register kernel: s_sleep(1) repeats between the hidden-value stores and the first read of the next step
  int delay_inc;      // register kernel: units added to the delay after a repeated read; 0 = the delay stays as it is
  int delay_dec_mask; // register kernel: the delay adapts downwards by one unit every (mask + 1) steps without a repeated read
  unsigned long long* trace;  // optional [workgroups][8] cycle totals per phase (instrumented builds only)
  int op_flags;       // OpFlags: variations of the recurrence for the sibling ops (0 = NativeLstm2)
  int w_direct;       // per-step launches of the LDS kernel: 1 = W fragments go from memory straight to the matrix cores (no LDS copy)
  int zero;           // always 0; an operand the compiler cannot fold (idempotent atomics used as L2 reads)
  int sync_policy;    // SyncBits
  unsigned long long timeout_ticks;  // bound of one flag wait, in 100 MHz wall-clock ticks
};

// Several independent problems of one shape in one launch of the persistent register kernel: workgroups
// [k * wgs_each, k * wgs_each + grid) run problem k; the rest of each slice leaves at once.
constexpr int kMaxMulti = 4;
struct Lstm2Multi {
  int count;     // problems, 1..kMaxMulti
  int wgs_each;  // workgroup ids reserved per problem, a multiple of the XCD count (keeps the id -> XCD dealing in phase)
  int grid;      // workgroups a problem really uses (<= wgs_each)
  int local;     // 1: every batch group of every problem sits on one XCD (workgroup id = slot * xcds + xcd; the groups of
                 // the launch, all problems counted through, are dealt round-robin to the XCDs); wgs_each / grid unused
  int xcds;      // XCDs the workgroup ids are dealt to (local plans)
  int pad_;
  Lstm2Params p[kMaxMulti];
};

}  // namespace rtn
