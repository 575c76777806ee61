// FMHA forward, fp8 e4m3 (OCP) operands for BOTH GEMMs, fp32 softmax/accumulate, fp16 output -- gfx950 only.
//
// Takes the place of the reference's fp8 path: the same kernels as the fp16 path instantiated with
// cutlass::float_e4m3_t and -DGEMM2FP8 (src/fmha-pipeline/fmha_forward.cu:446-450), its fp8 WGMMA selectors
// (ss_helper.h:3-94), the P down-cast (reg2reg.h:18-27), the fp8 register reorganisation ReorgCFp8toAFp8
// (reg2reg.h:45-108) and the offline V transpose / key permutation done by the driver (fmha_forward.cu:514-558).
//
// Machine mapping (see fmha_fwd_f16.hip for the shared ideas: transposed GEMMs, one query column per lane,
// deferred rescale, LDS-DMA double buffering, two S register sets):
//  * v_mfma_f32_32x32x64_f8f6f4 (fp8 x fp8, 64-deep K-step, 16 passes) for S^T = K.Q^T and O^T += V^T.P^T -- the
//    legacy 32x32x16 fp8 MFMA runs at the fp16 rate.  A lane holds 32 of the 64 contraction slots of a K-step in 8
//    VGPRs; which slot means which index is free as long as the A and the B operand agree.
//  * P: a lane's 32 accumulator values of a 64-key tile (two 32-key blocks x 16 registers) ARE its 32 B-operand
//    slots: slot t = key 32*(t/16) + 8*((t%16)/4) + 4*g + t%4.  They are cast with v_cvt_pk_fp8_f32 in register
//    order; nothing is shuffled across lanes and P never touches LDS.
//  * The fp8 V-tile layout transform: V stays [B,S,H,D] in HBM and row-major ([key][d], swizzled) in LDS.  The A
//    operand needs, per lane (d, g), the 32 bytes V[key(t, g)][d], t = 0..31 -- a byte-granular transpose plus the
//    key permutation above.  Four ds_read_b64_tr_b8 deliver exactly that: in a block of 16 lanes, lane L supplies
//    the address of (row L/2, 8-byte column group L%2) and lane i receives rows 0..7 of column i, so choosing
//    row e -> key 16u + 8*(e/4) + 4g + e%4 for load u applies the permutation for free.  (The reference either
//    transposes V on the host and shuffles P across the quad, or also permutes V on the host: FP8NOSHFL.)
//  * Per-tensor scales: q_descale*k_descale is folded into the exp2 scale, v_descale into the final 1/l.
//  * P is biased by 2^kPBias before the cast (the softmax reference point sits kPBias below the row max): P then
//    spans (0, 2^8] instead of (0, 1] and keeps probabilities down to 2^-17 of the row max out of e4m3's flush
//    zone.  The reference casts P in (0,1] directly (fmha_consumer.h:54); the bias cancels in O/l.
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "fmha_common.h"

namespace cfk {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int int8v __attribute__((ext_vector_type(8)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))

__device__ __forceinline__ void lds_dma16(const void *gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory");
}
__device__ __forceinline__ void wait_lds_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <int D_, int NWAVES_, int WPE_>
struct Fp8Cfg {
  static constexpr int D = D_, BN = 64, NWAVES = NWAVES_, WPE = WPE_;
  static constexpr int T = NWAVES * 64;
  static constexpr int BM = NWAVES * 32;
  static constexpr int PITCH = D;                        // bytes per LDS row
  static constexpr int TILE_BYTES = BN * PITCH;
  static constexpr int LDS_BYTES = 4 * TILE_BYTES;       // K stage 0/1, V stage 0/1
  static constexpr int CPR = D / 16;                     // 16-byte chunks per row
  static constexpr int RPI = 1024 / PITCH;               // rows per wave-wide 16 B/lane copy
  static constexpr int IPW = BN / RPI / NWAVES;          // copies per wave per tile
  static_assert(D == 64 || D == 128 || D == 256, "head dim");
  static_assert(BN % (RPI * NWAVES) == 0 && IPW >= 1, "tile must split evenly over the waves");
};

// XOR swizzles of the 16-byte chunk index of a row (rows are D bytes; LDS banks repeat every 256 B, so 256/D rows
// share a bank period).
//  K: ds_read_b128 by 16 consecutive rows at one chunk index -> the rows that share a position inside the bank
//     period (16*D/256 of them) need distinct XOR values.
//  V: ds_read_b64_tr_b8 by keys {4g..4g+3, 8+4g..8+4g+3} x 32 contiguous bytes -> keys that share a position
//     inside the bank period need distinct 32-byte slots; bit 0 stays clear so a 32-byte pair stays contiguous.
template <int D>
__device__ __forceinline__ int swz_k8(int row) {
  if (D == 64) return (row >> 2) & 3;
  if (D == 128) return (row >> 1) & 7;
  return ((row & 3) << 2) | ((row >> 2) & 3);
}
template <int D>
__device__ __forceinline__ int swz_v8(int row) {
  if (D == 64) return ((row >> 3) & 1) << 1;
  if (D == 128) return (((row >> 1) & 1) << 1) | (((row >> 3) & 1) << 2);
  return ((row & 3) | (((row >> 3) & 1) << 2)) << 1;
}

template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(C::WPE, C::WPE)))
fmha_fwd_fp8_kernel(const FmhaArgs a) {
  constexpr int D = C::D, BN = C::BN;
  constexpr int KB = BN / 32;   // 32-key blocks per tile
  constexpr int KS = D / 64;    // 64-deep K-steps of S^T
  constexpr int DB = D / 32;    // 32-row blocks of O^T
  constexpr float kTau = 8.0f;  // P <= 2^kTau before a rescale is forced (e4m3 max is 448)
  constexpr float kPBias = 7.0f;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  const int q_blocks = a.Sq / C::BM;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / q_blocks;
  const int qb = tile - bh * q_blocks;
  const int b = bh / a.H, h = bh - b * a.H;
  const int64_t ld = (int64_t)a.H * D;  // row stride in elements (= bytes)
  const char *Qp = (const char *)a.q + ((int64_t)b * a.Sq * a.H + h) * D;
  const char *Kp = (const char *)a.k + ((int64_t)b * a.Skv * a.H + h) * D;
  const char *Vp = (const char *)a.v + ((int64_t)b * a.Skv * a.H + h) * D;
  _Float16 *Op = (_Float16 *)a.o + ((int64_t)b * a.Sq * a.H + h) * D;
  const int q0 = qb * C::BM + wave * 32;
  const int n_tiles = a.Skv / BN;
  const float c_log2 = a.scale_log2;
  const uint32_t ld_bytes = (uint32_t)ld;
  const uint32_t tile_stride = (uint32_t)BN * ld_bytes;

  // ---- global -> LDS copies (see fmha_fwd_f16.hip): lane l fills slot (row l / CPR, position l % CPR) with
  // chunk position ^ swz(row)
  uint32_t goff_k[C::IPW], goff_v[C::IPW];
#pragma unroll
  for (int i = 0; i < C::IPW; ++i) {
    const int row = (i * C::NWAVES + wave) * C::RPI + lane / C::CPR;
    const int cp = lane % C::CPR;
    goff_k[i] = (uint32_t)row * ld_bytes + (uint32_t)((cp ^ swz_k8<D>(row)) * 16);
    goff_v[i] = (uint32_t)row * ld_bytes + (uint32_t)((cp ^ swz_v8<D>(row)) * 16);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
  auto load_tile = [&](const char *gbase, const uint32_t (&goff)[C::IPW], int jt, int lds_off) {
    const char *gt = gbase + (size_t)jt * tile_stride;
#pragma unroll
    for (int i = 0; i < C::IPW; ++i) lds_dma16(gt + goff[i], lds_base + lds_off + (i * C::NWAVES + wave) * 1024);
  };
  constexpr int K_ST0 = 0, V_ST0 = 2 * C::TILE_BYTES;

  // ---- Q: B operand of S^T.  Lane (r, g), K-step s holds the 32 bytes Q[q0 + r][64s + 32g .. +32).
  int8v qreg[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int4v *p = (const int4v *)(Qp + (int64_t)(q0 + r) * ld + 64 * s + 32 * g);
    const int4v lo = p[0], hi = p[1];
    qreg[s] = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }

  // ---- per-lane LDS read addresses (bytes, relative to a tile)
  // K operand, K-step s: row r (+32 kb), chunks 4s+2g and 4s+2g+1, each swizzled on its own
  int k_rd[KS][2];
#pragma unroll
  for (int s = 0; s < KS; ++s)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) k_rd[s][hh] = r * C::PITCH + (((4 * s + 2 * g + hh) ^ swz_k8<D>(r)) * 16);
  // V operand via ds_read_b64_tr_b8 (see the file comment)
  const int li = lane & 15;
  const int row_e = li >> 1;
  const int v_key = 8 * (row_e >> 2) + 4 * g + (row_e & 3);          // + 16 u
  int v_rd[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    const int c = 2 * db + ((lane >> 4) & 1);
    v_rd[db] = v_key * C::PITCH + ((c ^ swz_v8<D>(v_key)) * 16) + 8 * (li & 1);
  }

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
  float m_ref = -INFINITY, m_true = -INFINITY, l_run = 0.f;

  auto qk = [&](int k_off, f32x16 (&sacc)[KB]) {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[kb][v] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int4v lo = *(const int4v *)(smem + k_off + k_rd[s][0] + kb * 32 * C::PITCH);
        const int4v hi = *(const int4v *)(smem + k_off + k_rd[s][1] + kb * 32 * C::PITCH);
        const int8v ka = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        sacc[kb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka, qreg[s], sacc[kb], 0, 0, 0, 0, 0, 0);
      }
  };
  // row max of a finished S tile and the deferred rescale (online_softmax.h:123-165)
  auto row_max_and_rescale = [&](const f32x16 (&sacc)[KB]) {
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[kb][v]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * c_log2;
    m_true = fmaxf(m_true, mx);
    if (__builtin_amdgcn_ballot_w64(mx > m_ref + kTau) != 0) {
      const float m_new = fmaxf(m_ref, mx - kPBias);
      const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
      m_ref = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;
    }
  };
  // P = exp2(c*S - m_ref); row sum in fp32 before the down-cast (online_softmax.h:173-206); e4m3 in slot order
  auto softmax_exp = [&](const f32x16 (&sacc)[KB], int8v &pb) {
    float rs = 0.f;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float p[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          p[t] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][4 * w + t], c_log2, -m_ref));
          rs += p[t];
        }
        int packed = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], 0, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], packed, true);
        pb[kb * 4 + w] = packed;
      }
    l_run += rs;
  };
  auto pv = [&](int v_off, const int8v &pb) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      int8v va;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int2v x = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(int2v, smem + v_off + v_rd[db] + u * 16 * C::PITCH));
        va[2 * u] = x[0];
        va[2 * u + 1] = x[1];
      }
      oacc[db] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, pb, oacc[db], 0, 0, 0, 0, 0, 0);
    }
  };

  auto step = [&](auto parity, auto has_next, int j, f32x16 (&s_cur)[KB], f32x16 (&s_nxt)[KB]) {
    constexpr int P = decltype(parity)::value;
    constexpr bool HAS_NEXT = decltype(has_next)::value;
    const int jk = j + 2 < n_tiles ? j + 2 : n_tiles - 1;
    const int jv = j + 1 < n_tiles ? j + 1 : n_tiles - 1;
    load_tile(Kp, goff_k, jk, K_ST0 + P * C::TILE_BYTES);
    load_tile(Vp, goff_v, jv, V_ST0 + (P ^ 1) * C::TILE_BYTES);
    int8v pb;
    if (HAS_NEXT) qk(K_ST0 + (P ^ 1) * C::TILE_BYTES, s_nxt);
    softmax_exp(s_cur, pb);
    pv(V_ST0 + P * C::TILE_BYTES, pb);
    if (HAS_NEXT) row_max_and_rescale(s_nxt);
    wait_lds_dma();
    __syncthreads();
  };

  f32x16 s_a[KB], s_b[KB];
  load_tile(Kp, goff_k, 0, K_ST0);
  load_tile(Vp, goff_v, 0, V_ST0);
  load_tile(Kp, goff_k, n_tiles > 1 ? 1 : 0, K_ST0 + C::TILE_BYTES);
  wait_lds_dma();
  __syncthreads();
  qk(K_ST0, s_a);
  row_max_and_rescale(s_a);
  __syncthreads();

  using std::integral_constant;
  int j = 0;
  for (; j + 2 < n_tiles; j += 2) {
    step(integral_constant<int, 0>{}, integral_constant<bool, true>{}, j, s_a, s_b);
    step(integral_constant<int, 1>{}, integral_constant<bool, true>{}, j + 1, s_b, s_a);
  }
  if (j + 2 == n_tiles) {
    step(integral_constant<int, 0>{}, integral_constant<bool, true>{}, j, s_a, s_b);
    step(integral_constant<int, 1>{}, integral_constant<bool, false>{}, j + 1, s_b, s_a);
  } else {
    step(integral_constant<int, 0>{}, integral_constant<bool, false>{}, j, s_a, s_b);
  }

  // ---- epilogue: O = v_descale * O / l, fp16, [B,S,H,D]
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = a.out_scale / l_tot;
  const int qrow = q0 + r;
  _Float16 *orow = Op + (int64_t)qrow * ld;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half4 o4;
#pragma unroll
      for (int t = 0; t < 4; ++t) o4[t] = (_Float16)(oacc[db][4 * i + t] * inv);
      *(half4 *)(orow + db * 32 + 8 * i + 4 * g) = o4;
    }
  if (g == 0) {
    const int64_t si = ((int64_t)b * a.H + h) * a.Sq + qrow;
    if (a.row_max) a.row_max[si] = m_true;
    if (a.row_sum) a.row_sum[si] = l_tot * __builtin_amdgcn_exp2f(m_ref - m_true);
  }
}

template <class C>
hipError_t launch_cfg(const FmhaArgs &a, hipStream_t s) {
  static bool attr_done = false;
  auto kern = fmha_fwd_fp8_kernel<C>;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  const int grid = a.B * a.H * (a.Sq / C::BM);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::T), C::LDS_BYTES, s, a);
  return hipGetLastError();
}

using Cfg64S = Fp8Cfg<64, 4, 2>;
using Cfg128S = Fp8Cfg<128, 4, 2>;
using Cfg128L = Fp8Cfg<128, 8, 2>;
using Cfg256S = Fp8Cfg<256, 4, 1>;   // O (128) + S (64) + Q (32) registers: one wave per SIMD

bool use_large(int head_dim, int sq, int bh) {
  static const int forced = [] {
    const char *e = getenv("CFK_FMHA_TILE");
    if (!e) return -1;
    return e[0] == 's' ? 0 : e[0] == 'l' ? 1 : -1;
  }();
  if (head_dim != 128 || sq % 256 != 0 || forced == 0) return false;
  if (forced == 1) return true;
  return (long long)bh * (sq / 256) >= 512;
}

template <class C>
void fill_plan(int sq, int bh, FmhaPlan *p) {
  p->block_m = C::BM;
  p->block_n = C::BN;
  p->lds_bytes = C::LDS_BYTES;
  p->threads = C::T;
  p->grid = bh * (sq / C::BM);
}

template <class F>
bool dispatch(int head_dim, int sq, int bh, F &&f) {
  switch (head_dim) {
    case 64: f(Cfg64S{}); return true;
    case 128: use_large(head_dim, sq, bh) ? f(Cfg128L{}) : f(Cfg128S{}); return true;
    case 256: f(Cfg256S{}); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_fp8(int head_dim, int sq, int skv, int bh, int v_layout, FmhaPlan *p) {
  (void)skv;
  if (v_layout != 0) return false;
  return dispatch(head_dim, sq, bh, [&](auto cfg) { fill_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_fp8(const FmhaArgs &a, int head_dim, hipStream_t s) {
  if (a.v_layout != 0) return hipErrorNotSupported;
  hipError_t e = hipErrorNotSupported;
  dispatch(head_dim, a.Sq, a.B * a.H, [&](auto cfg) { e = launch_cfg<decltype(cfg)>(a, s); });
  return e;
}

}  // namespace cfk
