// FMHA forward, fp16 operands, fp32 softmax/accumulate, fp16 output -- gfx950 (MI355X) only.
//
// Takes the place of the reference's device kernels fmhaForwardPipelinedNoWspl / ...Wspl / fmhaForwardNoPipeline
// (src/fmha-pipeline/fmha_pipe_nows.h:72-331, fmha_pipe_ws.h:69-365, fmha_nopipe.h:43-342) and of their building
// blocks fmhaForwardConsumer (fmha_consumer.h:8-73), onlineSoftmaxAndRescale (online_softmax.h:87-207),
// applySoftmaxNormalizer (online_softmax.h:59-85) and the epilogue (fmha_epilogue.h:120-177).  Same mathematics,
// different machine mapping:
//
//  * One workgroup owns BM = NWAVES*NQ*32 query rows of one (batch, head); wave w owns NQ blocks of 32 rows.
//  * Both GEMMs run TRANSPOSED on v_mfma_f32_32x32x16_f16:
//        S^T[key, q] = K[key, :] . Q[q, :]      A = K tile from LDS, B = Q held in VGPRs for the whole kernel
//        O^T[d,  q] += V^T[d, key] . P^T[key, q] A = V tile read transposed from LDS, B = P straight from the
//                                                S^T accumulator registers.
//    In the 32x32 accumulator layout lane (q = lane%32, g = lane/32) holds rows 8*(v/4)+4*g+(v%4), v = 0..15, of
//    column q.  So one lane holds 16 keys of ONE query: row max / row sum are in-lane reductions plus a single
//    exchange with lane^32, the running max / sum / rescale factor are per-lane scalars, and P never moves
//    across lanes: the accumulator registers, cast to fp16, already ARE the B operand of the second MFMA under
//    a fixed permutation of the 16 keys of each K-step.  That permutation is applied to V instead (a GEMM is
//    invariant under a common permutation of its contraction index): it falls out of the addresses handed to
//    ds_read_b64_tr_b16, which delivers 4 consecutive keys of one head-dim column per lane.
//  * K/V tiles are staged global -> VGPR -> LDS, double buffered, one s_barrier per KV tile.  LDS rows are padded
//    (K by 16 B, V by 64 B) so that the ds_read_b128 / ds_read_b64_tr_b16 patterns spread over all banks.
//  * Workgroup ids are remapped so the query blocks of one head share an XCD's L2.
#include "fmha_common.h"

namespace cfk {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))

template <int D_, int BN_, int NQ_, int NWAVES_>
struct F16Cfg {
  static constexpr int D = D_, BN = BN_, NQ = NQ_, NWAVES = NWAVES_;
  static constexpr int T = NWAVES * 64;
  static constexpr int BM = NWAVES * NQ * 32;
  static constexpr int KSTR = D + 8;    // halves per LDS row of K (16 B pad)
  static constexpr int VSTR = D + 32;   // halves per LDS row of V (64 B pad)
  static constexpr int K_TILE = BN * KSTR;
  static constexpr int V_TILE = BN * VSTR;
  static constexpr int STAGE = K_TILE + V_TILE;          // halves
  static constexpr int LDS_BYTES = 2 * STAGE * 2;        // two stages
  static constexpr int CHUNKS = BN * D / 8;              // 16-byte chunks per tile
  static constexpr int CPT = CHUNKS / T;                 // chunks per thread
  static_assert(CHUNKS % T == 0, "tile must split evenly over the workgroup");
  static_assert(BN % 32 == 0 && D % 32 == 0, "tile shape");
};

__device__ __forceinline__ float xor32_max(float x) {
  return fmaxf(x, __shfl_xor(x, 32, 64));
}

template <class C>
__global__ void __launch_bounds__(C::T) fmha_fwd_f16_kernel(const FmhaArgs a) {
  constexpr int D = C::D, BN = C::BN, NQ = C::NQ;
  constexpr int KB = BN / 32;   // 32-key blocks per tile (M blocks of S^T)
  constexpr int KS = D / 16;    // K-steps of S^T
  constexpr int DB = D / 32;    // 32-row blocks of O^T
  constexpr int PS = BN / 16;   // K-steps of O^T
  extern __shared__ __attribute__((aligned(16))) _Float16 smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;

  const int q_blocks = a.Sq / C::BM;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / q_blocks;
  const int qb = tile - bh * q_blocks;
  const int b = bh / a.H, h = bh - b * a.H;
  const int64_t ld = (int64_t)a.H * D;  // row stride in elements
  const _Float16 *Qp = (const _Float16 *)a.q + ((int64_t)b * a.Sq * a.H + h) * D;
  const _Float16 *Kp = (const _Float16 *)a.k + ((int64_t)b * a.Skv * a.H + h) * D;
  const _Float16 *Vp = (const _Float16 *)a.v + ((int64_t)b * a.Skv * a.H + h) * D;
  _Float16 *Op = (_Float16 *)a.o + ((int64_t)b * a.Sq * a.H + h) * D;
  const int q0 = qb * C::BM + wave * (NQ * 32);

  // ---- Q: B operand of S^T, resident in VGPRs.  Lane (r, g) holds Q[q0 + 32nq + r][16s + 8g .. +8).
  half8 qreg[NQ][KS];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
    for (int s = 0; s < KS; ++s)
      qreg[nq][s] = *(const half8 *)(Qp + (int64_t)(q0 + nq * 32 + r) * ld + 16 * s + 8 * g);

  // ---- staging: thread t moves chunks c = i*T + t; chunk c = (row c / (D/8), 16-byte column c % (D/8))
  int4v kst[C::CPT], vst[C::CPT];
  auto issue_loads = [&](int j) {
#pragma unroll
    for (int i = 0; i < C::CPT; ++i) {
      const int c = i * C::T + tid;
      const int row = c / (D / 8), col = c % (D / 8);
      const int64_t off = (int64_t)(j * BN + row) * ld + col * 8;
      kst[i] = *(const int4v *)(Kp + off);
      vst[i] = *(const int4v *)(Vp + off);
    }
  };
  auto write_stage = [&](int stage) {
    _Float16 *ks = smem + stage * C::STAGE;
    _Float16 *vs = ks + C::K_TILE;
#pragma unroll
    for (int i = 0; i < C::CPT; ++i) {
      const int c = i * C::T + tid;
      const int row = c / (D / 8), col = c % (D / 8);
      *(int4v *)(ks + row * C::KSTR + col * 8) = kst[i];
      *(int4v *)(vs + row * C::VSTR + col * 8) = vst[i];
    }
  };

  f32x16 oacc[DB][NQ];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[db][nq][v] = 0.f;
  float m_run[NQ], l_run[NQ];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    m_run[nq] = -INFINITY;
    l_run[nq] = 0.f;
  }

  // per-lane constant parts of the LDS read addresses (in halves)
  const int k_rd = r * C::KSTR + 8 * g;
  // ds_read_b64_tr_b16: inside a block of 16 lanes, lane i must point at (row i/4, 4-element column group i%4);
  // it receives rows 0..3 of column i.  Lanes 16..31 take the next 16 columns, lanes 32..63 (g = 1) the keys +4.
  const int li = lane & 15;
  const int v_rd = (4 * g + (li >> 2)) * C::VSTR + 16 * ((lane >> 4) & 1) + 4 * (li & 3);

  const int n_tiles = a.Skv / BN;
  const float c_log2 = a.scale_log2;

  issue_loads(0);
  write_stage(0);
  __syncthreads();

  for (int j = 0; j < n_tiles; ++j) {
    const int stage = j & 1;
    if (j + 1 < n_tiles) issue_loads(j + 1);
    const _Float16 *ks = smem + stage * C::STAGE;
    const _Float16 *vs = ks + C::K_TILE;

    // ---- S^T = K . Q^T
    f32x16 sacc[KB][NQ];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
        for (int v = 0; v < 16; ++v) sacc[kb][nq][v] = 0.f;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const half8 ka = *(const half8 *)(ks + k_rd + kb * 32 * C::KSTR + 16 * s);
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
          sacc[kb][nq] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qreg[nq][s], sacc[kb][nq], 0, 0, 0);
      }

    // ---- online softmax (online_softmax.h:87-207), one query column per lane
    half8 pb[PS][NQ];
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float mx = sacc[0][nq][0];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[kb][nq][v]);
      mx = xor32_max(mx);
      const float m_new = fmaxf(m_run[nq], mx * c_log2);
      const float alpha = __builtin_amdgcn_exp2f(m_run[nq] - m_new);
      m_run[nq] = m_new;
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][nq][v], c_log2, -m_new));
          rs += p;  // row sum is taken in fp32 before the down-cast (online_softmax.h:173-206)
          pb[kb * 2 + v / 8][nq][v % 8] = (_Float16)p;
        }
      l_run[nq] = l_run[nq] * alpha + rs;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[db][nq][v] *= alpha;
    }

    // ---- O^T += V^T . P^T
#pragma unroll
    for (int ps = 0; ps < PS; ++ps)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const _Float16 *vp = vs + v_rd + (ps * 16) * C::VSTR + db * 32;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, vp));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, vp + 8 * C::VSTR));
        union {
          struct { short4v lo, hi; } s;
          half8 h;
        } va;
        va.s.lo = lo;
        va.s.hi = hi;
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
          oacc[db][nq] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va.h, pb[ps][nq], oacc[db][nq], 0, 0, 0);
      }

    if (j + 1 < n_tiles) write_stage(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: O = O / l (online_softmax.h:59-85), fp16, [B,S,H,D]
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    const float l_tot = l_run[nq] + __shfl_xor(l_run[nq], 32, 64);
    const float inv = a.out_scale / l_tot;
    const int qrow = q0 + nq * 32 + r;
    _Float16 *orow = Op + (int64_t)qrow * ld;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        half4 o4;
#pragma unroll
        for (int t = 0; t < 4; ++t) o4[t] = (_Float16)(oacc[db][nq][4 * i + t] * inv);
        *(half4 *)(orow + db * 32 + 8 * i + 4 * g) = o4;
      }
    if (g == 0) {
      const int64_t si = ((int64_t)b * a.H + h) * a.Sq + qrow;
      if (a.row_max) a.row_max[si] = m_run[nq];
      if (a.row_sum) a.row_sum[si] = l_tot;
    }
  }
}

template <class C>
hipError_t launch_cfg(const FmhaArgs &a, hipStream_t s) {
  static bool attr_done = false;  // one attribute call per instantiation and process
  auto kern = fmha_fwd_f16_kernel<C>;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  const int grid = a.B * a.H * (a.Sq / C::BM);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::T), C::LDS_BYTES, s, a);
  return hipGetLastError();
}

using Cfg64 = F16Cfg<64, 64, 1, 4>;
using Cfg128 = F16Cfg<128, 64, 1, 4>;
using Cfg256 = F16Cfg<256, 64, 1, 4>;

template <class C>
void fill_plan(int sq, int bh, FmhaPlan *p) {
  p->block_m = C::BM;
  p->block_n = C::BN;
  p->lds_bytes = C::LDS_BYTES;
  p->threads = C::T;
  p->grid = bh * (sq / C::BM);
}

}  // namespace

bool plan_fmha_f16(int head_dim, int sq, int skv, int bh, FmhaPlan *p) {
  (void)skv;
  switch (head_dim) {
    case 64: fill_plan<Cfg64>(sq, bh, p); return true;
    case 128: fill_plan<Cfg128>(sq, bh, p); return true;
    case 256: fill_plan<Cfg256>(sq, bh, p); return true;
    default: return false;
  }
}

hipError_t launch_fmha_f16(const FmhaArgs &a, int head_dim, hipStream_t s) {
  switch (head_dim) {
    case 64: return launch_cfg<Cfg64>(a, s);
    case 128: return launch_cfg<Cfg128>(a, s);
    case 256: return launch_cfg<Cfg256>(a, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace cfk
