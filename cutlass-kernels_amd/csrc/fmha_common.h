// Shared declarations of the gfx950 FMHA-forward kernels (host launchers + argument block).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdlib>

namespace cfk {

// Argument block handed to every FMHA kernel (by value).  Tensors are [B, S, H, D] with D contiguous, the
// layout of the reference (src/fmha-pipeline/fmha_forward.cu:131-134, 151-152).
struct FmhaArgs {
  const void *q, *k, *v;
  void *o;
  float *row_max;    // optional [B,H,Sq] tap: running max, log2 domain (reference: miOut)
  float *s_tap;      // optional [B,H,Sq,Skv] tap: pre-softmax scores, natural domain     (reference: tensorS)
  float *row_sum;    // optional [B,H,Sq] tap: sum of exp2(t - max)     (reference: sPrimeOut)
  int32_t B, H, Sq, Skv;
  float scale_log2;  // softmax_scale * log2(e) * q_descale * k_descale
  float out_scale;   // v_descale (1 for fp16)
  float s_scale;     // softmax_scale * q_descale * k_descale (scales the score tap)
  int32_t v_layout;  // 0 = [B,S,H,D], 1 = [B,D,H,S]
  float tau;         // the softmax reference point moves when a tile's max exceeds it by more than this (log2 domain)
  int32_t track_only;  // no optimistic first pass over the keys (cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY, 1))
  int32_t direct_p;    // first pass with e4m3 P: codes without an exponential (cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, 1))
};

// cfk_set_option(CFK_OPT_PREDICTABLE_LATENCY, ...): also steers the choice of instantiation (fmha_fwd_kernel.h: select_tile)
bool predictable_latency();
// cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, ...): calls then launch the DirectCfg builds of the kernels with e4m3 P
bool fast_e4m3_weights();

struct FmhaPlan {
  int32_t block_m, block_n, lds_bytes, threads, grid;
  int32_t q_multiple;   // what the query length has to be a multiple of (block_m, or 32 where the last tile may be partly filled)
  int32_t kv_multiple;  // what the key length has to be a multiple of (block_n, or one key tile where the kernel has a tail)
  int32_t mfma;  // 32: 32x32 MFMA build, 16: 16x16x32 build
  char kernel[80];  // the instantiation, as profilers print it without namespaces: fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>
};

// Each launcher validates nothing: the C-ABI layer has already checked shapes against the plan.
// `tap_s` (plan) / a.s_tap (launch) selects the build of the kernel that also writes the score tap.
hipError_t launch_fmha_f16(const FmhaArgs &a, int head_dim, hipStream_t s);      // Q,K,V fp16
hipError_t launch_fmha_fp8(const FmhaArgs &a, int head_dim, hipStream_t s);      // Q,K,V e4m3, P e4m3
hipError_t launch_fmha_hybrid(const FmhaArgs &a, int head_dim, hipStream_t s);   // Q,K e4m3; P,V fp16
bool plan_fmha_f16(int head_dim, int sq, int skv, int bh, bool tap_s, FmhaPlan *p);
// fp16 at head dim 256 (without the score tap) lives in a translation unit of its own; launch_fmha_f16 and
// plan_fmha_f16 forward to these
hipError_t launch_fmha_f16_d256(const FmhaArgs &a, hipStream_t s);
void plan_fmha_f16_d256(int sq, int skv, int bh, FmhaPlan *p);
hipError_t prepare_fmha_f16_d256();
bool plan_fmha_fp8(int head_dim, int sq, int skv, int bh, int v_layout, bool tap_s, FmhaPlan *p);
bool plan_fmha_hybrid(int head_dim, int sq, int skv, int bh, bool tap_s, FmhaPlan *p);
// One-time set-up (dynamic-LDS limits) of every instantiation of a family on the current device; launches do it on
// demand, this makes it happen ahead of time.
hipError_t prepare_fmha_f16();
hipError_t prepare_fmha_fp8();
hipError_t prepare_fmha_hybrid();
hipError_t prepare_gemm();

// D = alpha * A.B + beta * C for `batch` packed problems; f32 selects float operands (layout 0 only), else fp16.
struct GemmArgs {
  const void *A, *B, *C;  // C may be null (beta is then ignored)
  void *D;
  int32_t M, N, K, batch, layout;
  bool f32;
  float alpha, beta;
};
hipError_t launch_gemm(const GemmArgs &g, hipStream_t s);

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

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))
// LDS pointer from an absolute LDS byte address (32-bit integer)
#define LDS_AT(T, addr) ((__attribute__((address_space(3))) T *)(uintptr_t)(addr))

// Asynchronous 16 B/lane global -> LDS copy: lane l writes LDS bytes [lds_addr + 16 l, +16) with the 16 bytes at
// its own global address.  Issued through inline asm on purpose: the compiler then does not track the copy, so it
// does not drain vmcnt before every later LDS read, and the copies of one pipeline step stay in flight until
// the explicit wait_lds_dma() in front of the step's closing barrier.  lds_addr must be wave-uniform.
// The instruction takes its LDS base from M0, which the statements overwrite.  "m0" is on their clobber lists so that
// the compiler sees a definition of M0 there and does not carry an M0 value of its own across a copy (it merges
// identical M0 initialisations otherwise); M0 being a reserved register, clang warns about the entry, hence the
// pragma.  (Saving and restoring M0 inside each statement instead, two scalar moves per copy, measured -0.4 .. -0.9 %
// on the attention kernels.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_dma16(const void *gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory", "m0");
}
// The same copy addressed as wave-uniform base (SGPR pair) + per-lane 32-bit byte offset: no 64-bit vector add per copy.
__device__ __forceinline__ void lds_dma16(const void *base, uint32_t lane_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_off), "s"(base)
               : "memory", "m0");
}
// ... and with the LDS address as the sum of two wave-uniform terms (a long-lived one, e.g. the wave's share of every
// tile, plus one that is a constant at most call sites): keeps one scalar register live instead of one per target.
__device__ __forceinline__ void lds_dma16(const void *base, uint32_t lane_off, uint32_t lds_a, uint32_t lds_b) {
  asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" ::"s"(lds_a), "s"(lds_b), "v"(lane_off), "s"(base)
               : "memory", "scc", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ void wait_lds_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// The lane number, computed on the spot (two v_mbcnt) from an operand the compiler cannot see through: neither kept in a
// register across the main loop nor hoisted out of the item loop.
__device__ __forceinline__ unsigned fresh_zero() {
  unsigned z = 0;
  asm volatile("" : "+v"(z));
  return z;
}
__device__ __forceinline__ int fresh_lane() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, fresh_zero())); }

// Exchange among the four lanes c, c+16, c+32, c+48 that share a query, without a lane number in a register and
// without the LDS: v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its
// second, v_permlane32_swap the same for 32-lane halves; with x in both operands the two results, combined, are the
// pairwise max / sum.  (Written as asm: this compiler's builtin hands back the first result twice.  The s_nop covers
// the wait states the instruction wants behind a vector write of its operands.)
__device__ __forceinline__ void swap_rows16(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_rows32(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}

__device__ __forceinline__ float quad_max(float x) {
  float a = x, b = x;
  swap_rows16(a, b);
  a = b = fmaxf(a, b);
  swap_rows32(a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float quad_sum(float x) {
  float a = x, b = x;
  swap_rows16(a, b);
  a = b = a + b;
  swap_rows32(a, b);
  return a + b;
}

}  // namespace cfk
