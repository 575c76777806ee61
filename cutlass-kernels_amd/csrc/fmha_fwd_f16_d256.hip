// FMHA forward, fp16 operands, head dim 256: tile shapes and dispatch.  A translation unit of its own because these
// kernels run one wave per SIMD (Q and O fill half the register file) and are built with another machine-scheduler
// strategy than the rest of the library (Makefile: iterative-ilp).  With a single wave nothing but the wave's own
// instruction order hides LDS and MFMA latency, and the order that strategy finds is the faster one: 994-1001 against
// 928 TFLOP/s on B=2 H=8 S=8192 with N(0,1) tensors, 1206 against 1024 with constant tensors.  Every kernel with two or
// three waves per SIMD loses under it (registers spill), so it is not a library-wide flag.
#include "fmha_fwd_kernel16p.h"

namespace cfk {
namespace {

// <head dim, keys per tile, waves, waves per SIMD, e4m3 Q/K, e4m3 P/V, V transposed, score tap, tiles per barrier,
//  K fragments read ahead of the barrier>
using C256_128x32 = FmhaCfg<256, 32, 4, 1, false, false>;
using C256_128x32P = FmhaCfg<256, 32, 4, 1, false, false, false, false, 1, 4>;  // key length a multiple of 128
// 64-key tiles: under this file's scheduler strategy they no longer spill inside the loop (they did under the default
// one: 572 TFLOP/s), and run as fast as 32-key tiles (1003-1007 against 1010-1016 TFLOP/s on B=2 H=8 S=8192, two 32-key
// tiles per barrier 1010-1013): a choice for the tile sweep, not the automatic one.
using C256_128x64 = FmhaCfg<256, 64, 4, 1, false, false>;
// The hand-scheduled persistent build on 16x16x32 MFMAs (fmha_fwd_kernel16p.h; key length a multiple of 128, at least
// 256): two 32-key tiles per barrier, big problems only
using A256_128x64 = FmhaCfg<256, 32, 4, 1, false, false, false, false, 2, 0, true, true>;
using All256 = CfgList<C256_128x32P, C256_128x32, C256_128x64, A256_128x64>;
using Auto256 = CfgList<A256_128x64, C256_128x32P, C256_128x32>;

template <class F>
void dispatch(int sq, int skv, int bh, F &&f) {
  select_tile<All256, Auto256, C256_128x32>(sq, skv, bh, f);
}

}  // namespace

void plan_fmha_f16_d256(int sq, int skv, int bh, FmhaPlan *p) {
  dispatch(sq, skv, bh, [&](auto cfg) { fill_fmha_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_f16_d256(const FmhaArgs &a, hipStream_t s) {
  hipError_t e = hipErrorInvalidValue;
  dispatch(a.Sq, a.Skv, a.B * a.H, [&](auto cfg) { e = launch_fmha_cfg<decltype(cfg)>(a, s); });
  return e;
}

hipError_t prepare_fmha_f16_d256() { return prepare_all(All256{}); }

}  // namespace cfk
