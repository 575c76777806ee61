// FMHA forward, e4m3 operands for both GEMMs (the reference's -DGEMM2FP8 build): tile shapes and dispatch.
// The kernel, including the fp8 V-tile layout transform, is in fmha_fwd_kernel.h.
#include "fmha_fwd_kernel.h"

namespace cfk {
namespace {

using Cfg64S = FmhaCfg<64, 64, 4, 3, true, true>;  // three waves per SIMD: the VALU-bound softmax gains from every extra wave
using Cfg128S = FmhaCfg<128, 64, 4, 2, true, true>;
using Cfg128L = FmhaCfg<128, 64, 8, 2, true, true>;
using Cfg256S = FmhaCfg<256, 64, 4, 1, true, true>;  // O (128) + S (64) + Q (32) registers: one wave per SIMD

// V pre-transposed to [B,D,H,S] (the reference's offline transpose, src/fmha-pipeline/fmha_forward.cu:514-532)
using Cfg64T = FmhaCfg<64, 64, 4, 2, true, true, true>;
using Cfg128T = FmhaCfg<128, 64, 4, 2, true, true, true>;
using Cfg256T = FmhaCfg<256, 64, 4, 1, true, true, true>;

// builds that also write the score tap (debug)
using Cfg64Tap = FmhaCfg<64, 64, 4, 2, true, true, false, true>;
using Cfg128Tap = FmhaCfg<128, 64, 4, 2, true, true, false, true>;
using Cfg256Tap = FmhaCfg<256, 64, 4, 1, true, true, false, true>;
using Cfg64TTap = FmhaCfg<64, 64, 4, 2, true, true, true, true>;
using Cfg128TTap = FmhaCfg<128, 64, 4, 2, true, true, true, true>;
using Cfg256TTap = FmhaCfg<256, 64, 4, 1, true, true, true, true>;

template <class F>
bool dispatch(int head_dim, int sq, int bh, int v_layout, bool tap_s, F &&f) {
  if (tap_s) {
    const bool t = v_layout == 1;
    switch (head_dim) {
      case 64: t ? f(Cfg64TTap{}) : f(Cfg64Tap{}); return true;
      case 128: t ? f(Cfg128TTap{}) : f(Cfg128Tap{}); return true;
      case 256: t ? f(Cfg256TTap{}) : f(Cfg256Tap{}); return true;
      default: return false;
    }
  }
  if (v_layout == 1) {
    switch (head_dim) {
      case 64: f(Cfg64T{}); return true;
      case 128: f(Cfg128T{}); return true;
      case 256: f(Cfg256T{}); return true;
      default: return false;
    }
  }
  switch (head_dim) {
    case 64: f(Cfg64S{}); return true;
    case 128: use_large_tile(sq, bh, false) ? f(Cfg128L{}) : f(Cfg128S{}); return true;
    case 256: f(Cfg256S{}); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_fp8(int head_dim, int sq, int skv, int bh, int v_layout, bool tap_s, FmhaPlan *p) {
  (void)skv;
  return dispatch(head_dim, sq, bh, v_layout, tap_s, [&](auto cfg) { fill_fmha_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_fp8(const FmhaArgs &a, int head_dim, hipStream_t s) {
  hipError_t e = hipErrorNotSupported;
  dispatch(head_dim, a.Sq, a.B * a.H, a.v_layout, a.s_tap != nullptr, [&](auto cfg) { e = launch_fmha_cfg<decltype(cfg)>(a, s); });
  return e;
}

}  // namespace cfk
