// Which build of the persistent kernels serves which decomposition.  The kernels are templates with many
// instantiations; they are compiled in several parts, each a compilation of lstm2_kernel_tables.hip with another value
// of RTN_TABLE_PART, so that the parts build side by side.  The host code asks these functions for a kernel and launches
// it through the pointer.
#pragma once

#include "lstm2_bwd_kernels.h"
#include "lstm2_kernels.h"

namespace rtn {

typedef void (*RegwKernel)(const Lstm2Multi);
typedef void (*BwdRegwKernel)(const Lstm2BwdMulti);

// Forward register kernel k_lstm2_regw<AT, MT, NT, KSMAX, HALF>; null if the decomposition has no build.
// "lo": KSMAX of 2 or 4 macro steps per wavefront, "hi": 8 or 16.
RegwKernel regw_table_bf16_lo(int MT, int NT, int KSMAX, bool half);
RegwKernel regw_table_bf16_hi(int MT, int NT, int KSMAX, bool half);
RegwKernel regw_table_f32_lo(int MT, int NT, int KSMAX, bool half);
RegwKernel regw_table_f32_hi(int MT, int NT, int KSMAX, bool half);

// Persistent gradient kernel k_lstm2_bwd_regw<AT, KSB, MT, WV, 0, HALF>; KSB: fragments of W per tile and wavefront,
// MT: tiles of 16 values of k per workgroup, WV: wavefronts per workgroup.  "half": groups of at most 8 rows.
BwdRegwKernel bwd_regw_table_bf16_half(int KSB, int MT, int WV);
BwdRegwKernel bwd_regw_table_bf16_full(int KSB, int MT, int WV);
BwdRegwKernel bwd_regw_table_f32_half(int KSB, int MT, int WV);
BwdRegwKernel bwd_regw_table_f32_full(int KSB, int MT, int WV);
// The variants with half of a wavefront's share of W in registers and half in LDS (one tile per workgroup).
BwdRegwKernel bwd_regw_lds_table_bf16(int WV);
BwdRegwKernel bwd_regw_lds_table_f32(int WV);

inline RegwKernel regw_kernel(int dtype, int MT, int NT, int KSMAX, bool half) {
  const bool lo = KSMAX <= 4;
  if (dtype == 1 /* RTN_DTYPE_BF16 */) return lo ? regw_table_bf16_lo(MT, NT, KSMAX, half) : regw_table_bf16_hi(MT, NT, KSMAX, half);
  return lo ? regw_table_f32_lo(MT, NT, KSMAX, half) : regw_table_f32_hi(MT, NT, KSMAX, half);
}

}  // namespace rtn
