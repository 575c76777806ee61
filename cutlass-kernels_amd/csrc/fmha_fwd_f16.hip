// FMHA forward, fp16 operands: tile shapes and dispatch.  The kernel is in fmha_fwd_kernel.h.
#include "fmha_fwd_kernel.h"

namespace cfk {
namespace {

// "small" = 4 waves x 32 query rows (two workgroups share a CU), "large" = 8 waves x 32 rows (one workgroup per CU,
// half the K/V traffic per query row); both run two waves per SIMD, except head dim 64, whose small tile fits three
// (154 registers) and is the faster one for it.
using Cfg64S = FmhaCfg<64, 64, 4, 3, false, false>;
using Cfg64L = FmhaCfg<64, 64, 8, 2, false, false>;
using Cfg128S = FmhaCfg<128, 64, 4, 2, false, false>;
using Cfg128L = FmhaCfg<128, 64, 8, 2, false, false>;
using Cfg256S = FmhaCfg<256, 32, 4, 1, false, false>;  // one wave per SIMD: Q (64) + O (128) registers fill half the file

// builds that also write the score tap (debug): small tile only
using Cfg64Tap = FmhaCfg<64, 64, 4, 2, false, false, false, true>;
using Cfg128Tap = FmhaCfg<128, 64, 4, 2, false, false, false, true>;
using Cfg256Tap = FmhaCfg<256, 32, 4, 1, false, false, false, true>;

template <class F>
bool dispatch(int head_dim, int sq, int bh, bool tap_s, F &&f) {
  if (tap_s) {
    switch (head_dim) {
      case 64: f(Cfg64Tap{}); return true;
      case 128: f(Cfg128Tap{}); return true;
      case 256: f(Cfg256Tap{}); return true;
      default: return false;
    }
  }
  switch (head_dim) {
    case 64: use_large_tile(sq, bh, false) ? f(Cfg64L{}) : f(Cfg64S{}); return true;
    case 128: use_large_tile(sq, bh) ? f(Cfg128L{}) : f(Cfg128S{}); return true;
    case 256: f(Cfg256S{}); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_f16(int head_dim, int sq, int skv, int bh, bool tap_s, FmhaPlan *p) {
  (void)skv;
  return dispatch(head_dim, sq, bh, tap_s, [&](auto cfg) { fill_fmha_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_f16(const FmhaArgs &a, int head_dim, hipStream_t s) {
  hipError_t e = hipErrorInvalidValue;
  dispatch(head_dim, a.Sq, a.B * a.H, a.s_tap != nullptr, [&](auto cfg) { e = launch_fmha_cfg<decltype(cfg)>(a, s); });
  return e;
}

}  // namespace cfk
