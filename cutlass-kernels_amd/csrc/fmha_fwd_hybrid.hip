// FMHA forward, hybrid precision: Q, K e4m3 (GEMM-I on the fp8 MFMA), P and V fp16 (GEMM-II on the fp16 MFMA) --
// what the reference's --prec-type=2 computes when built without -DGEMM2FP8 (src/fmha-pipeline/fmha_forward.cu:
// 446-450).  Tile shapes and dispatch; the kernel is in fmha_fwd_kernel.h.
#include "fmha_fwd_kernel.h"

namespace cfk {
namespace {

using Cfg64S = FmhaCfg<64, 64, 4, 3, true, false>;
using Cfg128S = FmhaCfg<128, 64, 4, 2, true, false>;
using Cfg128L = FmhaCfg<128, 64, 8, 2, true, false>;
using Cfg256S = FmhaCfg<256, 32, 4, 1, true, false>;

// builds that also write the score tap (debug): small tile only
using Cfg64Tap = FmhaCfg<64, 64, 4, 2, true, false, false, true>;
using Cfg128Tap = FmhaCfg<128, 64, 4, 2, true, false, false, true>;
using Cfg256Tap = FmhaCfg<256, 32, 4, 1, true, false, false, true>;

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
    case 64: f(Cfg64S{}); return true;
    case 128: use_large_tile(sq, bh) ? f(Cfg128L{}) : f(Cfg128S{}); return true;
    case 256: f(Cfg256S{}); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_hybrid(int head_dim, int sq, int skv, int bh, bool tap_s, FmhaPlan *p) {
  (void)skv;
  return dispatch(head_dim, sq, bh, tap_s, [&](auto cfg) { fill_fmha_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_hybrid(const FmhaArgs &a, int head_dim, hipStream_t s) {
  hipError_t e = hipErrorNotSupported;
  dispatch(head_dim, a.Sq, a.B * a.H, a.s_tap != nullptr, [&](auto cfg) { e = launch_fmha_cfg<decltype(cfg)>(a, s); });
  return e;
}

}  // namespace cfk
