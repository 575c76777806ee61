// FMHA forward, e4m3 operands for both GEMMs (the reference's -DGEMM2FP8 build): tile shapes and dispatch.
// The kernel, including the fp8 V-tile layout transform, is in fmha_fwd_kernel.h.
#include "fmha_fwd_kernel.h"

namespace cfk {
namespace {

using Cfg64S = FmhaCfg<64, 64, 4, 2, true, true>;
using Cfg128S = FmhaCfg<128, 64, 4, 2, true, true>;
using Cfg128L = FmhaCfg<128, 64, 8, 2, true, true>;
using Cfg256S = FmhaCfg<256, 64, 4, 1, true, true>;  // O (128) + S (64) + Q (32) registers: one wave per SIMD

template <class F>
bool dispatch(int head_dim, int sq, int bh, F &&f) {
  switch (head_dim) {
    case 64: f(Cfg64S{}); return true;
    case 128: use_large_tile(sq, bh, false) ? f(Cfg128L{}) : f(Cfg128S{}); return true;
    case 256: f(Cfg256S{}); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_fp8(int head_dim, int sq, int skv, int bh, int v_layout, FmhaPlan *p) {
  (void)skv;
  if (v_layout != 0) return false;
  return dispatch(head_dim, sq, bh, [&](auto cfg) { fill_fmha_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_fp8(const FmhaArgs &a, int head_dim, hipStream_t s) {
  if (a.v_layout != 0) return hipErrorNotSupported;
  hipError_t e = hipErrorNotSupported;
  dispatch(head_dim, a.Sq, a.B * a.H, [&](auto cfg) { e = launch_fmha_cfg<decltype(cfg)>(a, s); });
  return e;
}

}  // namespace cfk
