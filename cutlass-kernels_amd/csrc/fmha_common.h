// Shared declarations of the gfx950 FMHA-forward kernels (host launchers + argument block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cfk {

// Argument block handed to every FMHA kernel (by value).  Tensors are [B, S, H, D] with D contiguous, the
// layout of the reference (src/fmha-pipeline/fmha_forward.cu:131-134, 151-152).
struct FmhaArgs {
  const void *q, *k, *v;
  void *o;
  float *row_max;    // optional [B,H,Sq] tap: running max, log2 domain (reference: miOut)
  float *row_sum;    // optional [B,H,Sq] tap: sum of exp2(t - max)     (reference: sPrimeOut)
  int32_t B, H, Sq, Skv;
  float scale_log2;  // softmax_scale * log2(e) * q_descale * k_descale
  float out_scale;   // v_descale (1 for fp16)
  int32_t v_layout;  // 0 = [B,S,H,D], 1 = [B,D,H,S]
};

struct FmhaPlan {
  int32_t block_m, block_n, lds_bytes, threads, grid;
};

// Each launcher validates nothing: the C-ABI layer has already checked shapes against the plan.
hipError_t launch_fmha_f16(const FmhaArgs &a, int head_dim, hipStream_t s);
hipError_t launch_fmha_fp8(const FmhaArgs &a, int head_dim, hipStream_t s);
bool plan_fmha_f16(int head_dim, int sq, int skv, int bh, FmhaPlan *p);
bool plan_fmha_fp8(int head_dim, int sq, int skv, int bh, int v_layout, FmhaPlan *p);

hipError_t launch_gemm_f16(int M, int N, int K, const void *A, const void *B, void *C, int layout, hipStream_t s);

// Workgroup id -> logical tile id.  Hardware deals consecutive workgroup ids round-robin over the 8 XCDs,
// each with a private L2.  Giving XCD x the contiguous range [x*n/8, (x+1)*n/8) keeps the query blocks
// of one (batch, head) -- which all re-read the same K/V -- on one L2.
__device__ __forceinline__ int xcd_remap(int wg, int n) {
  constexpr int kXcds = 8;
  const int per = n / kXcds;
  const int main_n = per * kXcds;
  if (wg >= main_n) return wg;  // ragged tail keeps its id
  return (wg % kXcds) * per + wg / kXcds;
}

}  // namespace cfk
