// The instantiations of the persistent kernels, in parts: this file is compiled once per value of RTN_TABLE_PART
// (see build.py), each compilation defines the table functions of one part (lstm2_kernel_tables.h).
#include <hip/hip_runtime.h>

#include "lstm2_kernel_tables.h"

#ifndef RTN_TABLE_PART
#error "compile with -DRTN_TABLE_PART=<1..8>"
#endif

namespace rtn {
namespace {

// Forward.  HI: the builds with 8 or 16 macro steps of the contraction per wavefront, else those with 2 or 4.
template <typename AT, bool HI>
RegwKernel regw_table(int MT, int NT, int KSMAX, bool half) {
  if (half) {
#define RTN_CASE(mt, ks) \
  if (MT == mt && NT == 1 && KSMAX == ks) return &k_lstm2_regw<AT, mt, 1, ks, true>;
    if constexpr (HI) {
      RTN_CASE(2, 8) RTN_CASE(2, 16)
      RTN_CASE(4, 8)
      RTN_CASE(8, 8)
    } else {
      RTN_CASE(2, 2) RTN_CASE(2, 4)
      RTN_CASE(4, 2) RTN_CASE(4, 4)
    }
#undef RTN_CASE
    return nullptr;
  }
#define RTN_CASE(mt, nt, ks) \
  if (MT == mt && NT == nt && KSMAX == ks) return &k_lstm2_regw<AT, mt, nt, ks>;
  if constexpr (HI) {
    RTN_CASE(1, 1, 8) RTN_CASE(1, 2, 8) RTN_CASE(1, 4, 8)
    RTN_CASE(2, 1, 8) RTN_CASE(2, 2, 8) RTN_CASE(2, 4, 8)
    RTN_CASE(4, 1, 8) RTN_CASE(4, 2, 8)
    RTN_CASE(8, 1, 8)
    RTN_CASE(1, 1, 16) RTN_CASE(1, 2, 16)
    RTN_CASE(2, 1, 16) RTN_CASE(2, 2, 16)
  } else {
    RTN_CASE(1, 1, 2) RTN_CASE(1, 2, 2) RTN_CASE(1, 4, 2)
    RTN_CASE(2, 1, 2) RTN_CASE(2, 2, 2) RTN_CASE(2, 4, 2)
    RTN_CASE(4, 1, 2) RTN_CASE(4, 2, 2)
    RTN_CASE(1, 1, 4) RTN_CASE(1, 2, 4) RTN_CASE(1, 4, 4)
    RTN_CASE(2, 1, 4) RTN_CASE(2, 2, 4) RTN_CASE(2, 4, 4)
    RTN_CASE(4, 1, 4) RTN_CASE(4, 2, 4)
  }
#undef RTN_CASE
  return nullptr;
}

// Gradient.
template <typename AT, bool HALF>
BwdRegwKernel bwd_regw_table(int KSB, int MT, int WV) {
#define RTN_CASE(ks, mt, wv) \
  if (KSB == ks && MT == mt && WV == wv) return &k_lstm2_bwd_regw<AT, ks, mt, wv, 0, HALF>;
  RTN_CASE(2, 1, 4) RTN_CASE(4, 1, 4) RTN_CASE(8, 1, 4) RTN_CASE(16, 1, 4) RTN_CASE(32, 1, 4)
  if constexpr (sizeof(AT) == 2) { RTN_CASE(64, 1, 4) }
  RTN_CASE(2, 2, 4) RTN_CASE(4, 2, 4) RTN_CASE(8, 2, 4) RTN_CASE(16, 2, 4) RTN_CASE(32, 2, 4)
  RTN_CASE(2, 4, 4) RTN_CASE(4, 4, 4) RTN_CASE(8, 4, 4) RTN_CASE(16, 4, 4)
  RTN_CASE(2, 1, 8) RTN_CASE(4, 1, 8) RTN_CASE(8, 1, 8) RTN_CASE(16, 1, 8)
  RTN_CASE(2, 2, 8) RTN_CASE(4, 2, 8) RTN_CASE(8, 2, 8) RTN_CASE(16, 2, 8)
  RTN_CASE(2, 4, 8) RTN_CASE(4, 4, 8) RTN_CASE(8, 4, 8) RTN_CASE(16, 4, 8)
  RTN_CASE(2, 1, 16) RTN_CASE(4, 1, 16) RTN_CASE(8, 1, 16)
  RTN_CASE(2, 2, 16) RTN_CASE(4, 2, 16) RTN_CASE(8, 2, 16)
  RTN_CASE(2, 4, 16) RTN_CASE(4, 4, 16) RTN_CASE(8, 4, 16)
#undef RTN_CASE
  return nullptr;
}

template <typename AT>
BwdRegwKernel bwd_regw_lds_table(int WV) {
  if (WV == 8) return &k_lstm2_bwd_regw<AT, 16, 1, 8, 16>;
  return &k_lstm2_bwd_regw<AT, 32, 1, 4, 32>;
}

}  // namespace

#if RTN_TABLE_PART == 1
RegwKernel regw_table_bf16_lo(int MT, int NT, int KSMAX, bool half) { return regw_table<__bf16, false>(MT, NT, KSMAX, half); }
#elif RTN_TABLE_PART == 2
RegwKernel regw_table_bf16_hi(int MT, int NT, int KSMAX, bool half) { return regw_table<__bf16, true>(MT, NT, KSMAX, half); }
#elif RTN_TABLE_PART == 3
RegwKernel regw_table_f32_lo(int MT, int NT, int KSMAX, bool half) { return regw_table<float, false>(MT, NT, KSMAX, half); }
#elif RTN_TABLE_PART == 4
RegwKernel regw_table_f32_hi(int MT, int NT, int KSMAX, bool half) { return regw_table<float, true>(MT, NT, KSMAX, half); }
#elif RTN_TABLE_PART == 5
BwdRegwKernel bwd_regw_table_bf16_half(int KSB, int MT, int WV) { return bwd_regw_table<__bf16, true>(KSB, MT, WV); }
#elif RTN_TABLE_PART == 6
BwdRegwKernel bwd_regw_table_bf16_full(int KSB, int MT, int WV) { return bwd_regw_table<__bf16, false>(KSB, MT, WV); }
BwdRegwKernel bwd_regw_lds_table_bf16(int WV) { return bwd_regw_lds_table<__bf16>(WV); }
#elif RTN_TABLE_PART == 7
BwdRegwKernel bwd_regw_table_f32_half(int KSB, int MT, int WV) { return bwd_regw_table<float, true>(KSB, MT, WV); }
#elif RTN_TABLE_PART == 8
BwdRegwKernel bwd_regw_table_f32_full(int KSB, int MT, int WV) { return bwd_regw_table<float, false>(KSB, MT, WV); }
BwdRegwKernel bwd_regw_lds_table_f32(int WV) { return bwd_regw_lds_table<float>(WV); }
#else
#error "RTN_TABLE_PART must be 1..8"
#endif

}  // namespace rtn
