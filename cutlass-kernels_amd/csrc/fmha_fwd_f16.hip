// FMHA forward, fp16 operands: tile shapes and dispatch.  The kernels are in fmha_fwd_kernel.h (32x32 MFMAs) and
// fmha_fwd_kernel16.h (16x16x32 MFMAs).
#include "fmha_fwd_kernel16p.h"
#include "fmha_fwd_kernel_ks.h"

namespace cfk {
namespace {

// <head dim, keys per tile, waves, waves per SIMD, e4m3 Q/K, e4m3 P/V, V transposed, score tap, tiles per barrier,
//  K fragments read ahead of the barrier, 16x16x32 build>.  4 waves = 128 query rows (two workgroups share a CU),
// 8 waves = 256 rows (one workgroup per CU, half the K/V traffic per query row).  Two waves per SIMD, except head dim
// 64, whose 128-row tile fits three (the faster choice there).  Head dim 256 (one wave per SIMD) is built in
// fmha_fwd_f16_d256.hip, under a machine-scheduler strategy of its own; only its score-tap build is here.
using C64_128x64 = FmhaCfg<64, 64, 4, 3, false, false>;
using C64_256x64 = FmhaCfg<64, 64, 8, 2, false, false>;
using C64_128x128 = FmhaCfg<64, 64, 4, 2, false, false, false, false, 2>;
using C64_256x128 = FmhaCfg<64, 64, 8, 2, false, false, false, false, 2>;
using C128_128x64 = FmhaCfg<128, 64, 4, 2, false, false>;
using C128_256x64 = FmhaCfg<128, 64, 8, 2, false, false>;
using C128_256x64P = FmhaCfg<128, 64, 8, 2, false, false, false, false, 1, 4>;  // key length a multiple of 256
using C128_128x128 = FmhaCfg<128, 64, 4, 2, false, false, false, false, 2>;
using C128_256x128 = FmhaCfg<128, 64, 8, 2, false, false, false, false, 2>;
// The builds on 16x16x32 MFMAs, the automatic choice for big problems at head dims 64 and 128 (+6..10 % on N(0,1)
// data).  Head dim 128: two key tiles per barrier when the key length allows (+1..2 %: 1145-1157 against 1134
// TFLOP/s on B=8 H=16 S=2048).  Not built: the K fragment prefetch (registers spill), at head dim 64 256 rows (880
// against 919 TFLOP/s for 128 rows) and two tiles per barrier (950 against 1030: the LDS then holds two workgroups
// per CU, not three), head dim 256 (929 against 932 for the 32x32 build).
using N64_128x64 = FmhaCfg<64, 64, 4, 3, false, false, false, false, 1, 0, true>;
using N128_128x64 = FmhaCfg<128, 64, 4, 2, false, false, false, false, 1, 0, true>;
using N128_256x64 = FmhaCfg<128, 64, 8, 2, false, false, false, false, 1, 0, true>;
using N128_256x128 = FmhaCfg<128, 64, 8, 2, false, false, false, false, 2, 0, true>;
using N128_128x128 = FmhaCfg<128, 64, 4, 2, false, false, false, false, 2, 0, true>;
// ... and with the hand-scheduled main loop (key length a multiple of 256, at least 512)
using A128_256x128 = FmhaCfg<128, 64, 8, 2, false, false, false, false, 2, 0, true, true>;
using A64_256x128 = FmhaCfg<64, 64, 8, 2, false, false, false, false, 2, 0, true, true>;
using A128_128x128 = FmhaCfg<128, 64, 4, 1, false, false, false, false, 2, 0, true, true>;   // the same loops, 4 waves, one per SIMD
using A64_128x128 = FmhaCfg<64, 64, 4, 1, false, false, false, false, 2, 0, true, true>;

// ... and for small grids: 32 query rows per workgroup, the eight waves split the keys (fmha_fwd_kernel_ks.h)
using K64_32x64 = KsCfg<64, 8>;
using K128_32x64 = KsCfg<128, 8>;

// builds that also write the score tap (debug): 128-row tile only
using C64Tap = FmhaCfg<64, 64, 4, 2, false, false, false, true>;
using C128Tap = FmhaCfg<128, 64, 4, 2, false, false, false, true>;
using C256Tap = FmhaCfg<256, 32, 4, 1, false, false, false, true>;

using All64 = CfgList<C64_128x64, N64_128x64, C64_256x64, C64_128x128, C64_256x128, A64_256x128, A64_128x128, K64_32x64>;
using All128 = CfgList<C128_128x64, N128_128x64, C128_256x64P, C128_256x64, N128_256x64, C128_128x128, C128_256x128, N128_128x128, A128_256x128, A128_128x128, N128_256x128, K128_32x64>;

template <class F>
bool dispatch(int head_dim, int sq, int skv, int bh, bool tap_s, F &&f) {
  if (tap_s) {
    switch (head_dim) {
      case 64: f(C64Tap{}); return true;
      case 128: f(C128Tap{}); return true;
      case 256: f(C256Tap{}); return true;
      default: return false;
    }
  }
  switch (head_dim) {
    case 64: select_tile<All64, CfgList<K64_32x64, A64_256x128, A64_128x128, N64_128x64, C64_128x64>, C64_128x64>(sq, skv, bh, f); return true;
    case 128: select_tile<All128, CfgList<K128_32x64, A128_256x128, A128_128x128, N128_256x128, N128_256x64, N128_128x64, C128_256x64P, C128_256x64, C128_128x64>, C128_128x64>(sq, skv, bh, f); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_f16(int head_dim, int sq, int skv, int bh, bool tap_s, FmhaPlan *p) {
  if (head_dim == 256 && !tap_s) { plan_fmha_f16_d256(sq, skv, bh, p); return true; }
  return dispatch(head_dim, sq, skv, bh, tap_s, [&](auto cfg) { fill_fmha_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_f16(const FmhaArgs &a, int head_dim, hipStream_t s) {
  if (head_dim == 256 && !a.s_tap) return launch_fmha_f16_d256(a, s);
  hipError_t e = hipErrorInvalidValue;
  dispatch(head_dim, a.Sq, a.Skv, a.B * a.H, a.s_tap != nullptr, [&](auto cfg) { e = launch_fmha_cfg<decltype(cfg)>(a, s); });
  return e;
}

hipError_t prepare_fmha_f16() {
  hipError_t e = prepare_all(All64{});
  if (e == hipSuccess) e = prepare_all(All128{});
  if (e == hipSuccess) e = prepare_fmha_f16_d256();
  if (e == hipSuccess) e = prepare_all(CfgList<C64Tap, C128Tap, C256Tap>{});
  return e;
}

}  // namespace cfk
