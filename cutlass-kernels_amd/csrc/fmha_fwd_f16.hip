// FMHA forward, fp16 operands, fp32 softmax/accumulate, fp16 output -- gfx950 (MI355X) only.
//
// Takes the place of the reference's device kernels fmhaForwardPipelinedNoWspl / ...Wspl / fmhaForwardNoPipeline
// (src/fmha-pipeline/fmha_pipe_nows.h:72-331, fmha_pipe_ws.h:69-365, fmha_nopipe.h:43-342) and of their building
// blocks fmhaForwardProducer (fmha_producer.h:4-79), fmhaForwardConsumer (fmha_consumer.h:8-73),
// onlineSoftmaxAndRescale (online_softmax.h:87-207), applySoftmaxNormalizer (online_softmax.h:59-85) and the
// epilogue (fmha_epilogue.h:120-177).  Same mathematics, different machine mapping:
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
//  * K/V tiles go global -> LDS directly (global_load_lds_dwordx4, no VGPR staging), two stages each.  Rows are
//    unpadded; bank conflicts are avoided by XOR-swizzling the 16-byte chunks of a row, applied on the GLOBAL side
//    of the copy (lane i of a load always writes LDS slot i, but may fetch any chunk).
//  * Software pipeline (the reference overlaps only TMA with compute, its GEMMs drain the MMA pipe,
//    lib/gemm/gemm_tensor.hpp:14-25): iteration j issues S_{j+1} = K_{j+1}.Q^T on the MFMA pipe while the VALU
//    does exp2/row-sum/cast of S_j, then O += P_j.V_j while the VALU finds the row max of S_{j+1}.  S lives in two
//    register sets that swap roles every iteration (the loop is unrolled by two).
//  * Workgroup ids are remapped so the query blocks of one head share an XCD's L2.
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "fmha_common.h"

namespace cfk {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T *)(p))
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))

// Asynchronous 16 B/lane global -> LDS copy: lane l writes LDS bytes [lds_addr + 16 l, +16) with the 16 bytes at
// its own global address.  Issued through inline asm on purpose: the compiler then does not track the copy, so it
// does not drain vmcnt before every later LDS read, and the copies of one pipeline step stay in flight until
// the explicit wait_lds_dma() in front of the step's closing barrier.  lds_addr must be wave-uniform.
__device__ __forceinline__ void lds_dma16(const void *gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory");
}
__device__ __forceinline__ void wait_lds_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <int D_, int BN_, int NQ_, int NWAVES_, int WPE_ = 1>
struct F16Cfg {
  static constexpr int D = D_, BN = BN_, NQ = NQ_, NWAVES = NWAVES_;
  static constexpr int WPE = WPE_;                       // waves per SIMD the register budget is sized for
  static constexpr int T = NWAVES * 64;
  static constexpr int BM = NWAVES * NQ * 32;
  static constexpr int PITCH = D * 2;                    // bytes per LDS row (no padding)
  static constexpr int TILE_BYTES = BN * PITCH;
  static constexpr int LDS_BYTES = 4 * TILE_BYTES;       // K stage 0/1, V stage 0/1
  static constexpr int CPR = D / 8;                      // 16-byte chunks per row
  static constexpr int RPI = 1024 / PITCH;               // tile rows covered by one wave-wide 16 B/lane load
  static constexpr int IPW = BN / RPI / NWAVES;          // such loads per wave per tile
  static_assert(BN % (RPI * NWAVES) == 0, "tile must split evenly over the waves");
  static_assert(BN % 32 == 0 && D % 32 == 0 && (D == 64 || D == 128 || D == 256), "tile shape");
};

// XOR swizzles of the 16-byte chunk index within a row (LDS banks repeat every 256 B):
//  K is read with ds_read_b128 by 16 consecutive rows at one chunk index -> all 16 rows must land in distinct
//  256-byte bank groups; V is read with ds_read_b64_tr_b16 by 4 consecutive keys x 64 contiguous bytes.
template <int D>
__device__ __forceinline__ int swz_k(int row) {
  if (D == 64) return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  return ((row & 3) << 2) | ((row >> 2) & 3);
}
template <int D>
__device__ __forceinline__ int swz_v(int row) {
  if (D == 64) return ((row >> 1) & 1) << 2;
  return (row & 3) << 2;
}

template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(C::WPE, C::WPE)))
fmha_fwd_f16_kernel(const FmhaArgs a) {
  constexpr int D = C::D, BN = C::BN, NQ = C::NQ;
  constexpr int KB = BN / 32;   // 32-key blocks per tile (M blocks of S^T)
  constexpr int KS = D / 16;    // K-steps of S^T
  constexpr int DB = D / 32;    // 32-row blocks of O^T
  constexpr int PS = BN / 16;   // K-steps of O^T
  constexpr float kTau = 8.0f;  // deferred-rescale threshold (log2 domain): P <= 2^8 fits fp16
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
  const int64_t ld = (int64_t)a.H * D;  // row stride in elements
  const _Float16 *Qp = (const _Float16 *)a.q + ((int64_t)b * a.Sq * a.H + h) * D;
  const char *Kp = (const char *)((const _Float16 *)a.k + ((int64_t)b * a.Skv * a.H + h) * D);
  const char *Vp = (const char *)((const _Float16 *)a.v + ((int64_t)b * a.Skv * a.H + h) * D);
  _Float16 *Op = (_Float16 *)a.o + ((int64_t)b * a.Sq * a.H + h) * D;
  const int q0 = qb * C::BM + wave * (NQ * 32);
  const int n_tiles = a.Skv / BN;
  const float c_log2 = a.scale_log2;
  const uint32_t ld_bytes = (uint32_t)(ld * 2);
  const uint32_t tile_stride = (uint32_t)BN * ld_bytes;   // bytes between consecutive KV tiles in global memory

  // ---- global -> LDS copy.  Load i of wave w covers tile rows (i*NWAVES + w)*RPI .. +RPI; lane l writes the
  // LDS slot (row rr = l / CPR, chunk position cp = l % CPR) and fetches chunk cp ^ swz(row) of that row.
  uint32_t goff_k[C::IPW], goff_v[C::IPW];
#pragma unroll
  for (int i = 0; i < C::IPW; ++i) {
    const int row = (i * C::NWAVES + wave) * C::RPI + lane / C::CPR;
    const int cp = lane % C::CPR;
    goff_k[i] = (uint32_t)row * ld_bytes + (uint32_t)((cp ^ swz_k<D>(row)) * 16);
    goff_v[i] = (uint32_t)row * ld_bytes + (uint32_t)((cp ^ swz_v<D>(row)) * 16);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
  auto load_tile = [&](const char *gbase, const uint32_t (&goff)[C::IPW], int jt, int lds_off) {
    const char *gt = gbase + (size_t)jt * tile_stride;
#pragma unroll
    for (int i = 0; i < C::IPW; ++i) lds_dma16(gt + goff[i], lds_base + lds_off + (i * C::NWAVES + wave) * 1024);
  };
  constexpr int K_ST0 = 0, V_ST0 = 2 * C::TILE_BYTES;

  // ---- Q: B operand of S^T, resident in VGPRs.  Lane (r, g) holds Q[q0 + 32nq + r][16s + 8g .. +8).
  half8 qreg[NQ][KS];
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
    for (int s = 0; s < KS; ++s)
      qreg[nq][s] = *(const half8 *)(Qp + (int64_t)(q0 + nq * 32 + r) * ld + 16 * s + 8 * g);

  // ---- per-lane LDS read addresses (bytes, relative to a tile)
  // K operand, K-step s: row r (+32 kb), chunk (2s+g) ^ swz_k(r)
  int k_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) k_rd[s] = r * C::PITCH + (((2 * s + g) ^ swz_k<D>(r)) * 16);
  // V operand via ds_read_b64_tr_b16: inside a block of 16 lanes, lane i must point at (key i/4, 4 columns
  // 4*(i%4)..); it receives keys 0..3 of column i.  Lanes 16..31 take the next 16 columns, g = 1 the keys +4.
  const int li = lane & 15;
  const int v_key = 4 * g + (li >> 2);                               // + 16 ps + 8 h2
  const int v_col = 16 * ((lane >> 4) & 1) + 4 * (li & 3);           // + 32 db   (element index)
  int v_rd[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    const int c = (db * 32 + v_col) >> 3;
    v_rd[db] = v_key * C::PITCH + ((c ^ swz_v<D>(v_key)) * 16) + (v_col & 7) * 2;
  }

  f32x16 oacc[DB][NQ];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[db][nq][v] = 0.f;
  float m_ref[NQ], m_true[NQ], l_run[NQ];  // softmax reference point, true running max, running sum (log2 domain)
#pragma unroll
  for (int nq = 0; nq < NQ; ++nq) {
    m_ref[nq] = -INFINITY;
    m_true[nq] = -INFINITY;
    l_run[nq] = 0.f;
  }

  // S^T = K . Q^T for the K tile in LDS at byte offset k_off
  auto qk = [&](int k_off, f32x16 (&sacc)[KB][NQ]) {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
        for (int v = 0; v < 16; ++v) sacc[kb][nq][v] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const half8 ka = *(const half8 *)(smem + k_off + k_rd[s] + kb * 32 * C::PITCH);
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
          sacc[kb][nq] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qreg[nq][s], sacc[kb][nq], 0, 0, 0);
      }
  };
  // Row max of a finished S tile, and the deferred rescale (online_softmax.h:123-165).  The reference rescales O
  // and l by exp2(m_old - m_new) on every tile; any reference point m_ref works as long as exp2(t - m_ref) stays
  // representable, so m_ref only moves -- and O, l are only rescaled -- when the tile max exceeds it by more
  // than kTau.  The branch is wave-uniform.
  auto row_max_and_rescale = [&](const f32x16 (&sacc)[KB][NQ]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      float mx = sacc[0][nq][0];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[kb][nq][v]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * c_log2;
      m_true[nq] = fmaxf(m_true[nq], mx);
      if (__builtin_amdgcn_ballot_w64(mx > m_ref[nq] + kTau) != 0) {
        const float m_new = fmaxf(m_ref[nq], mx);
        const float alpha = __builtin_amdgcn_exp2f(m_ref[nq] - m_new);
        m_ref[nq] = m_new;
        l_run[nq] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int v = 0; v < 16; ++v) oacc[db][nq][v] *= alpha;
      }
    }
  };
  // P = exp2(c*S - m_ref), row sum in fp32 before the down-cast (online_softmax.h:173-206), cast to fp16 in the
  // B-operand register order of the second GEMM
  auto softmax_exp = [&](const f32x16 (&sacc)[KB][NQ], half8 (&pb)[PS][NQ]) {
#pragma unroll
    for (int nq = 0; nq < NQ; ++nq) {
      const float m_use = m_ref[nq];
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][nq][v], c_log2, -m_use));
          rs += p;
          pb[kb * 2 + v / 8][nq][v % 8] = (_Float16)p;
        }
      l_run[nq] += rs;
    }
  };
  // O^T += V^T . P^T for the V tile in LDS at byte offset v_off
  auto pv = [&](int v_off, const half8 (&pb)[PS][NQ]) {
#pragma unroll
    for (int ps = 0; ps < PS; ++ps)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const char *vp = smem + v_off + v_rd[db] + ps * 16 * C::PITCH;
        union {
          struct { short4v lo, hi; } s;
          half8 h;
        } va;
        va.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, vp));
        va.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, vp + 8 * C::PITCH));
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq)
          oacc[db][nq] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va.h, pb[ps][nq], oacc[db][nq], 0, 0, 0);
      }
  };

  // One pipeline step for tile j (parity P = j & 1).  On entry: s_cur = S_j is finished and its max is folded
  // into m_ref; K_{j+1} sits in K stage P^1 and V_j in V stage P.  HAS_NEXT is false for the last tile only.
  auto step = [&](auto parity, auto has_next, int j, f32x16 (&s_cur)[KB][NQ], f32x16 (&s_nxt)[KB][NQ]) {
    constexpr int P = decltype(parity)::value;
    constexpr bool HAS_NEXT = decltype(has_next)::value;
    // prefetch K_{j+2} into K stage P (last read by step j-1) and V_{j+1} into V stage P^1 (ditto); indices are
    // clamped at the end, which only rewrites a stage nobody reads any more
    const int jk = j + 2 < n_tiles ? j + 2 : n_tiles - 1;
    const int jv = j + 1 < n_tiles ? j + 1 : n_tiles - 1;
    load_tile(Kp, goff_k, jk, K_ST0 + P * C::TILE_BYTES);
    load_tile(Vp, goff_v, jv, V_ST0 + (P ^ 1) * C::TILE_BYTES);
    half8 pb[PS][NQ];
    if (HAS_NEXT) qk(K_ST0 + (P ^ 1) * C::TILE_BYTES, s_nxt);
    softmax_exp(s_cur, pb);
    pv(V_ST0 + P * C::TILE_BYTES, pb);
    if (HAS_NEXT) row_max_and_rescale(s_nxt);
    wait_lds_dma();   // this wave's copies have landed ...
    __syncthreads();  // ... and so have everybody else's; all reads of the stages about to be refilled are done
  };

  // ---- prologue: K_0, V_0, K_1 in flight; S_0 and its row max
  f32x16 s_a[KB][NQ], s_b[KB][NQ];
  load_tile(Kp, goff_k, 0, K_ST0);
  load_tile(Vp, goff_v, 0, V_ST0);
  load_tile(Kp, goff_k, n_tiles > 1 ? 1 : 0, K_ST0 + C::TILE_BYTES);
  wait_lds_dma();
  __syncthreads();
  qk(K_ST0, s_a);
  row_max_and_rescale(s_a);
  __syncthreads();  // every wave is done with K stage 0 before step 0 overwrites it

  using std::integral_constant;
  int j = 0;
  for (; j + 2 < n_tiles; j += 2) {
    step(integral_constant<int, 0>{}, integral_constant<bool, true>{}, j, s_a, s_b);
    step(integral_constant<int, 1>{}, integral_constant<bool, true>{}, j + 1, s_b, s_a);
  }
  if (j + 2 == n_tiles) {  // two tiles left: j (even) with a successor, then the last one
    step(integral_constant<int, 0>{}, integral_constant<bool, true>{}, j, s_a, s_b);
    step(integral_constant<int, 1>{}, integral_constant<bool, false>{}, j + 1, s_b, s_a);
  } else {                 // one tile left (even index)
    step(integral_constant<int, 0>{}, integral_constant<bool, false>{}, j, s_a, s_b);
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
      // taps are reported against the true row max, as the reference's miOut / sPrimeOut are
      if (a.row_max) a.row_max[si] = m_true[nq];
      if (a.row_sum) a.row_sum[si] = l_tot * __builtin_amdgcn_exp2f(m_ref[nq] - m_true[nq]);
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

// Tile shapes.  "small" = 4 waves x 32 query rows (two workgroups share a CU), "large" = 8 waves x 32 rows (one
// workgroup per CU, half the K/V traffic per query row); both run two waves per SIMD.
using Cfg64S = F16Cfg<64, 64, 1, 4, 2>;
using Cfg64L = F16Cfg<64, 64, 1, 8, 2>;
using Cfg128S = F16Cfg<128, 64, 1, 4, 2>;
using Cfg128L = F16Cfg<128, 64, 1, 8, 2>;
using Cfg256S = F16Cfg<256, 32, 1, 4, 1>;   // one wave per SIMD: Q (64) + O (128) registers alone fill half the file

enum class Shape { S, L };

// The reference fixes its tile shape at compile time (-DQBLKSIZE/-DKBLKSIZE, src/fmha-pipeline/shared_storage.h:4-15);
// here it is picked per call: the large tile needs seqlen_q % 256 == 0 and enough workgroups to fill 256 CUs twice.
// CFK_FMHA_TILE=small|large overrides the choice (tuning aid; ignored when the shape does not divide).
Shape pick_shape(int head_dim, int sq, int bh) {
  static const int forced = [] {
    const char *e = getenv("CFK_FMHA_TILE");
    if (!e) return -1;
    return e[0] == 's' ? 0 : e[0] == 'l' ? 1 : -1;
  }();
  if (head_dim == 256) return Shape::S;
  const bool large_ok = sq % 256 == 0;
  if (forced == 0 || !large_ok) return Shape::S;
  if (forced == 1) return Shape::L;
  return (long long)bh * (sq / 256) >= 512 ? Shape::L : Shape::S;
}

template <class C>
void fill_plan(int sq, int bh, FmhaPlan *p) {
  p->block_m = C::BM;
  p->block_n = C::BN;
  p->lds_bytes = C::LDS_BYTES;
  p->threads = C::T;
  p->grid = bh * (sq / C::BM);
}

// calls f.template operator()<Cfg>() for the configuration chosen for this problem
template <class F>
bool dispatch(int head_dim, int sq, int bh, F &&f) {
  const Shape sh = pick_shape(head_dim, sq, bh);
  switch (head_dim) {
    case 64: sh == Shape::L ? f(Cfg64L{}) : f(Cfg64S{}); return true;
    case 128: sh == Shape::L ? f(Cfg128L{}) : f(Cfg128S{}); return true;
    case 256: f(Cfg256S{}); return true;
    default: return false;
  }
}

}  // namespace

bool plan_fmha_f16(int head_dim, int sq, int skv, int bh, FmhaPlan *p) {
  (void)skv;
  return dispatch(head_dim, sq, bh, [&](auto cfg) { fill_plan<decltype(cfg)>(sq, bh, p); });
}

hipError_t launch_fmha_f16(const FmhaArgs &a, int head_dim, hipStream_t s) {
  hipError_t e = hipErrorInvalidValue;
  dispatch(head_dim, a.Sq, a.B * a.H, [&](auto cfg) { e = launch_cfg<decltype(cfg)>(a, s); });
  return e;
}

}  // namespace cfk
