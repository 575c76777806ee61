// The FMHA forward kernel for gfx950 (MI355X), one template for the three precision modes of the reference:
//   fp16            Q,K,V fp16                      (--prec-type=1)
//   fp8             Q,K,V e4m3, P cast to e4m3      (--prec-type=2 built with -DGEMM2FP8, fmha_forward.cu:446-450)
//   hybrid          Q,K e4m3; P,V fp16              (--prec-type=2 without GEMM2FP8, the reference's default fp8 build)
// always fp32 softmax / accumulation and fp16 output.
//
// Takes the place of the reference's device kernels fmhaForwardPipelinedNoWspl / ...Wspl / fmhaForwardNoPipeline
// (src/fmha-pipeline/fmha_pipe_nows.h:72-331, fmha_pipe_ws.h:69-365, fmha_nopipe.h:43-342) and of their building
// blocks fmhaForwardProducer (fmha_producer.h:4-79), fmhaForwardConsumer (fmha_consumer.h:8-73),
// onlineSoftmaxAndRescale (online_softmax.h:87-207), applySoftmaxNormalizer (online_softmax.h:59-85), convert_type /
// ReorgCFp8toAFp8 (reg2reg.h:18-108), the epilogue (fmha_epilogue.h:120-177), the tile constants
// (shared_storage.h:4-85) and the MMA selectors (ss_helper.h:3-94).  Same mathematics, different machine mapping:
//
//  * One workgroup owns BM = NWAVES*32 query rows of one (batch, head); a wave owns 32 rows; key tiles of BN keys.
//  * Both GEMMs run TRANSPOSED on 32x32 MFMAs (v_mfma_f32_32x32x16_f16, or v_mfma_f32_32x32x64_f8f6f4 for e4m3 -- the
//    legacy fp8 MFMA only runs at the fp16 rate):
//        S^T[key, q] = K[key, :] . Q[q, :]       A = K tile from LDS (ds_read_b128), B = Q resident in VGPRs
//        O^T[d,  q] += V^T[d, key] . P^T[key, q]  A = V tile read TRANSPOSED from LDS, B = P straight from the S^T
//                                                 accumulator registers.
//    In the 32x32 accumulator layout lane (q = lane%32, g = lane/32) holds rows 8*(v/4)+4*g+(v%4), v = 0..15, of
//    column q: one lane holds 16 keys of ONE query.  Row max / row sum are in-lane reductions plus one exchange with
//    lane^32; running max / sum / rescale factor are per-lane scalars; and the accumulator registers, cast to the P
//    precision, already ARE the B operand of the second MFMA under a fixed permutation of the keys of a K-step.  The
//    permutation is applied to V instead (a GEMM is invariant under a common permutation of its contraction index):
//    it falls out of the per-lane addresses handed to the LDS transpose reads.  P never crosses lanes, never touches
//    LDS (the reference shuffles across the quad, online_softmax.h:39-57 and reg2reg.h:71-107).
//      - fp16 V: ds_read_b64_tr_b16 hands a lane 4 consecutive keys of one head-dim column.
//      - e4m3 V, "the fp8 V-tile layout transform": the A operand needs per lane (d, g) the 32 bytes V[key(t,g)][d],
//        slot t = key 32*(t/16) + 8*((t%16)/4) + 4*g + t%4 -- a byte transpose plus that key permutation.  Four
//        ds_read_b64_tr_b8 deliver it: in a block of 16 lanes, lane L supplies the address of (row L/2, 8-byte column
//        group L%2) and lane i receives rows 0..7 of column i; row e of load u is pointed at key 16u+8(e/4)+4g+e%4.
//        V stays [B,S,H,D] in HBM: no host transpose (fmha_forward.cu:514-532), no host permutation (:534-558).
//  * K/V tiles go global -> LDS directly (global_load_lds_dwordx4, no VGPR staging), two stages each.  Rows are
//    unpadded; bank conflicts are removed by XOR-swizzling the 16-byte chunks of a row on the GLOBAL side of the
//    copy (lane i of a copy always writes LDS slot i, but may fetch any chunk).
//  * Software pipeline (the reference overlaps only TMA with compute; its GEMMs drain the MMA pipe,
//    lib/gemm/gemm_tensor.hpp:14-25): step j issues S_{j+1} = K_{j+1}.Q^T on the MFMA pipe while the VALU does
//    exp2 / row sum / cast of S_j, then O += P_j.V_j while the VALU finds the row max of S_{j+1}.  S lives in two
//    register sets that swap roles every step (the loop is unrolled by two).
//  * Deferred rescale: the reference rescales O and l by exp2(m_old - m_new) on every tile (online_softmax.h:
//    144-165).  Any reference point m_ref works as long as exp2(t - m_ref) stays representable, so m_ref only moves
//    -- and O, l are only rescaled -- when a tile max exceeds the maximum it was set from by more than a threshold
//    chosen by the host so that P <= 2^8 (exact range for fp16 and e4m3).  With e4m3 P the reference point
//    additionally sits 7 below the row max, so P spans (0, 2^8] instead of (0, 1] and probabilities down to 2^-17 of
//    the row max stay out of e4m3's flush zone (the reference casts P in (0,1] directly, fmha_consumer.h:54); the
//    bias cancels in O/l.
//      - e4m3 V given pre-transposed [B,D,H,S] (the reference's offline transpose): the tile is [d][key]; the K
//        tile is loaded row-permuted instead so that a lane's P slots are 32 contiguous keys and the V^T operand
//        is two plain ds_read_b128 (the counterpart of the reference's FP8NOSHFL key permutation, done on K, in
//        the copy, at no cost).
//  * Per-tensor fp8 scales: q_descale*k_descale is folded into the exp2 scale, v_descale into the final 1/l.
//  * Workgroup ids are remapped so the query blocks of one head share an XCD's L2.
#pragma once
#include <cstdio>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "fmha_common.h"

namespace cfk {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef int int8v __attribute__((ext_vector_type(8)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));

// what a pass over the keys does: track the running row max tile by tile (value), build e4m3 weights without an
// exponential (direct; only in a pass that does not track)
template <bool TRACK_, bool DIRECT_>
struct PassKind {
  static constexpr bool value = TRACK_, direct = DIRECT_;
  static_assert(!(TRACK_ && DIRECT_), "the direct codes belong to the pass with the fixed reference point");
};

template <int D_, int BN_, int NWAVES_, int WPE_, bool QK8_, bool PV8_, bool VT_ = false, bool TAP_S_ = false, int SUB_ = 1, int KPRE_ = 0,
          bool M16_ = false, bool ASM_ = false>
struct FmhaCfg {
  static constexpr int D = D_, BN = BN_, NWAVES = NWAVES_;
  static constexpr bool M16 = M16_;                             // the fp16 kernel on 16x16x32 MFMAs (fmha_fwd_kernel16.h)
  static constexpr bool ASM = ASM_;                             // ... with the hand-scheduled main loop (gen_fmha_loop16.py)
  static constexpr bool KSPLIT = false;                         // (true in KsCfg, fmha_fwd_kernel_ks.h: the waves split the keys)
  static constexpr int SUB = SUB_;                              // BN-key sub-tiles per barrier (1 or 2)
  static constexpr int KPRE = KPRE_;                            // K fragments of the next step read before the barrier
  static constexpr int NSLOT = KPRE ? 4 : 2 * SUB;              // LDS slots of one BN-key sub-tile of K
  static constexpr int NSLOT_V = 2 * SUB;                       // ... and of V
  static constexpr int WPE = WPE_;                              // waves per SIMD the register budget is sized for
  static constexpr bool QK8 = QK8_, PV8 = PV8_;                 // e4m3 (true) or fp16 (false) operands of GEMM-I / II
  static constexpr bool DIRECT = false;                         // (DirectCfg below)
  static constexpr bool VT = VT_;                               // V given pre-transposed, [B,D,H,S] (e4m3 only)
  static constexpr bool TAP_S = TAP_S_;                         // also write the pre-softmax scores (debug build)
  static constexpr int T = NWAVES * 64;
  static constexpr int BM = NWAVES * 32;
  static constexpr int K_PITCH = D * (QK8 ? 1 : 2);             // bytes per LDS row, no padding
  static constexpr int V_PITCH = VT ? BN : D * (PV8 ? 1 : 2);   // VT: the tile is [d][key], rows of BN bytes
  static constexpr int V_ROWS = VT ? D : BN;
  static constexpr int K_TILE = BN * K_PITCH, V_TILE = V_ROWS * V_PITCH;
  static constexpr int K_ST0 = 0, V_ST0 = NSLOT * K_TILE;       // LDS map: K slots, then V slots
  static constexpr int O_PITCH = D * 2 + 16;                    // epilogue: a wave's 32 fp16 output rows, padded
  static constexpr int STAGE_BYTES = NSLOT * K_TILE + NSLOT_V * V_TILE;
  static constexpr int O_BYTES = NWAVES * 32 * O_PITCH;
  // (the hand-scheduled build: 128 KB of K/V rings plus 32 KB; its 64 KB of output staging lie over the rings' upper
  // slots and those 32 KB: fmha_fwd_kernel16p.h;
  // ... the e4m3 one 64 KB of its own behind its 64 KB of rings, and a dword for the vote: fmha_fwd_kernel8p.h)
  static constexpr int LDS_BYTES = ASM ? (QK8 ? STAGE_BYTES + 65536 + 1024 : STAGE_BYTES + 32768) : STAGE_BYTES > O_BYTES ? STAGE_BYTES : O_BYTES;
  // one wave-wide 16 B/lane copy moves 1 KB = RPI rows; IPW copies per wave and tile
  static constexpr int K_RPI = 1024 / K_PITCH, K_IPW = BN / K_RPI / NWAVES;
  static constexpr int V_RPI = 1024 / V_PITCH, V_IPW = V_ROWS / V_RPI / NWAVES;
  static_assert(D == 64 || D == 128 || D == 256, "head dim");
  static_assert(SUB == 1 || SUB == 2, "sub-tiles per barrier");
  static_assert(!KPRE || SUB == 1, "K fragment prefetch is a variant of the one-tile step");
  static_assert(!ASM || ((M16 != (QK8 && PV8 && !VT)) && QK8 == PV8 && SUB == 2 &&
                         ((D == 128 && BN == 64 && NWAVES == 8 && WPE == 2) || (M16 && D <= 128 && BN == 64 && NWAVES == 4 && WPE == 1) ||
                          (QK8 && D == 128 && BN == 64 && NWAVES == 4 && WPE == 2) ||
                          (M16 && D == 256 && BN == 32 && NWAVES == 4 && WPE == 1) ||
                          (M16 && D == 64 && BN == 64 && NWAVES == 8 && WPE == 2))),
                "the hand-scheduled loops: fp16 on 16x16x32 MFMAs (head dims 64, 128, 256), e4m3 with V in [B,S,H,D] (128)");
  static_assert(BN % 32 == 0 && (!PV8 || BN == 64), "key tile: the e4m3 second GEMM has 64-deep K-steps");
  static_assert(!VT || PV8, "the pre-transposed layout is an e4m3-V layout");
  static_assert(K_IPW >= 1 && K_IPW * K_RPI * NWAVES == BN && V_IPW >= 1 && V_IPW * V_RPI * NWAVES == V_ROWS,
                "tile must split evenly over the waves");
};

// XOR swizzles of the 16-byte chunk index of an LDS row.  Banks repeat every 256 B, so 256/PITCH rows share a bank
// period (PITCH <= 256) or a row spans several (PITCH = 512).
//  rows read by ds_read_b128, 16 consecutive rows at one chunk index: rows at the same place in the bank period
//  need distinct values.
template <int PITCH>
__device__ __forceinline__ int swz_row(int row) {
  if (PITCH == 64) return (row >> 2) & 3;
  if (PITCH == 128) return (row >> 1) & 7;
  return ((row & 3) << 2) | ((row >> 2) & 3);
}
//  fp16 V read by ds_read_b64_tr_b16: 4 consecutive keys x 64 contiguous bytes.
template <int PITCH>
__device__ __forceinline__ int swz_v16(int row) {
  if (PITCH == 128) return ((row >> 1) & 1) << 2;
  return (row & 3) << 2;
}
//  e4m3 V read by ds_read_b64_tr_b8: keys {4g..4g+3, 8+4g..8+4g+3} x 32 contiguous bytes; bit 0 stays clear so a
//  32-byte pair stays contiguous.
template <int PITCH>
__device__ __forceinline__ int swz_v8(int row) {
  if (PITCH == 64) return ((row >> 3) & 1) << 1;
  if (PITCH == 128) return (((row >> 1) & 1) << 1) | (((row >> 3) & 1) << 2);
  return ((row & 3) | (((row >> 3) & 1) << 2)) << 1;
}

template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(C::WPE, C::WPE)))
fmha_fwd_kernel(const FmhaArgs a) {
  constexpr int D = C::D, BN = C::BN;
  constexpr bool QK8 = C::QK8, PV8 = C::PV8;
  constexpr int KB = BN / 32;                  // 32-key blocks per tile (M blocks of S^T)
  constexpr int KS = QK8 ? D / 64 : D / 16;    // K-steps of S^T
  constexpr int KH = QK8 ? 2 : 1;              // 16-byte LDS reads per K operand
  constexpr int DB = D / 32;                   // 32-row blocks of O^T
  constexpr int PS = PV8 ? BN / 64 : BN / 16;  // K-steps of O^T
  const float kTau = a.tau;                    // deferred-rescale threshold above the running max (log2 domain)
  // e4m3 P: the reference point sits this far below the row max (the weights reach up to 464 = 2^8.86).  The pass
  // that tracks the row max keeps it 7 below; the pass that does not (see the passes below) takes the first tile's max
  // itself -- that tile's weights lie in (0, 1], the range the reference's own algorithm casts all weights in -- which
  // leaves later maxima 8.8 binades = 6.1 standard deviations of N(0,1) scores.  (An earlier build sat 2 below that max:
  // two more bits for the smallest weights, which the output does not show -- rms error 6.806e-4 against 6.811e-4 at 4096
  // keys -- and 6.9 binades of head-room, which one in fourteen sets of N(0,1) tensors with 128 k rows exceeded in
  // some row, sending that row's workgroup through the second pass.)
  float p_bias = PV8 ? 7.0f : 0.0f;
  using QReg = std::conditional_t<QK8, int8v, half8>;
  using PReg = std::conditional_t<PV8, int8v, half8>;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;

  const int q_blocks = (a.Sq + C::BM - 1) / C::BM;   // the last query tile may be partly filled: whole waves of 32 rows
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / q_blocks;
  const int qb = tile - bh * q_blocks;
  const int b = bh / a.H, h = bh - b * a.H;
  const int64_t ld = (int64_t)a.H * D;  // row stride in elements
  constexpr int QES = QK8 ? 1 : 2, VES = PV8 ? 1 : 2;
  const char *Qp = (const char *)a.q + (((int64_t)b * a.Sq * a.H + h) * D) * QES;
  const char *Kp = (const char *)a.k + (((int64_t)b * a.Skv * a.H + h) * D) * QES;
  // V: [B,S,H,D] rows of the head at pitch H*D; pre-transposed [B,D,H,S]: rows d of the head at pitch H*Skv
  const char *Vp = C::VT ? (const char *)a.v + ((int64_t)b * D * a.H + h) * a.Skv
                         : (const char *)a.v + (((int64_t)b * a.Skv * a.H + h) * D) * VES;
  _Float16 *Op = (_Float16 *)a.o + ((int64_t)b * a.Sq * a.H + h) * D;
  // A wave behind the last query row still copies its share of every K/V tile and meets every barrier; it computes on
  // the last 32 rows (loads stay in bounds) and stores nothing.
  const bool live = qb * C::BM + wave * 32 < a.Sq;
  const int q0 = live ? qb * C::BM + wave * 32 : a.Sq - 32;
  const int n_tiles = a.Skv / BN;
  const float c_log2 = a.scale_log2;
  // global row pitch in bytes
  const uint32_t k_ld = (uint32_t)(ld * QES), v_ld = C::VT ? (uint32_t)a.H * (uint32_t)a.Skv : (uint32_t)(ld * VES);

  // ---- global -> LDS copies.  Copy i of wave w covers tile rows (i*NWAVES + w)*RPI .. +RPI; lane l writes LDS slot
  // (row l / CPR, chunk position l % CPR) and fetches chunk position ^ swz(row) of that row.
  uint32_t goff_k[C::K_IPW], goff_v[C::V_IPW];
#pragma unroll
  for (int i = 0; i < C::K_IPW; ++i) {
    constexpr int CPR = C::K_PITCH / 16;
    const int row = (i * C::NWAVES + wave) * C::K_RPI + lane / CPR;
    // Pre-transposed V wants a lane's 32 P slots to be 32 CONTIGUOUS keys.  Which key sits in which MFMA row of
    // S^T is free, so the K tile is loaded row-permuted: LDS row 32kb + 8w + 4g + j holds key 32g + 16kb + 4w + j
    // (then slot t of lane half g is key 32g + t).
    const int key = C::VT ? 32 * ((row >> 2) & 1) + 16 * (row >> 5) + 4 * ((row >> 3) & 3) + (row & 3) : row;
    goff_k[i] = (uint32_t)key * k_ld + (uint32_t)(((lane % CPR) ^ swz_row<C::K_PITCH>(row)) * 16);
  }
#pragma unroll
  for (int i = 0; i < C::V_IPW; ++i) {
    constexpr int CPR = C::V_PITCH / 16;
    const int row = (i * C::NWAVES + wave) * C::V_RPI + lane / CPR;
    const int sw = C::VT ? swz_row<C::V_PITCH>(row) : PV8 ? swz_v8<C::V_PITCH>(row) : swz_v16<C::V_PITCH>(row);
    goff_v[i] = (uint32_t)row * v_ld + (uint32_t)(((lane % CPR) ^ sw) * 16);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
  const uint32_t lds_wave = lds_base + wave * 1024;  // this wave's 1 KB share of every copy group
  auto load_k = [&](int jt, int stage) __attribute__((always_inline)) {
    const char *gt = Kp + (size_t)jt * ((size_t)BN * k_ld);
#pragma unroll
    for (int i = 0; i < C::K_IPW; ++i)
      lds_dma16(gt, goff_k[i], lds_wave, C::K_ST0 + stage * C::K_TILE + i * C::NWAVES * 1024);
  };
  auto load_v = [&](int jt, int stage) __attribute__((always_inline)) {
    const char *gt = C::VT ? Vp + (size_t)jt * BN : Vp + (size_t)jt * ((size_t)BN * v_ld);
#pragma unroll
    for (int i = 0; i < C::V_IPW; ++i)
      lds_dma16(gt, goff_v[i], lds_wave, C::V_ST0 + stage * C::V_TILE + i * C::NWAVES * 1024);
  };

  // ---- Q: B operand of S^T, resident in VGPRs.  fp16: lane (r, g), K-step s holds Q[q0+r][16s + 8g .. +8);
  // e4m3: the 32 bytes Q[q0+r][64s + 32g .. +32) (which contraction slot means which d is free as long as the K
  // operand uses the same map).
  QReg qreg[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    if constexpr (QK8) {
      const int4v *p = (const int4v *)(Qp + (int64_t)(q0 + r) * ld + 64 * s + 32 * g);
      const int4v lo = p[0], hi = p[1];
      qreg[s] = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    } else {
      qreg[s] = *(const half8 *)(Qp + ((int64_t)(q0 + r) * ld + 16 * s + 8 * g) * 2);
    }
  }

  // ---- per-lane LDS read addresses (absolute LDS byte addresses of slot 0; slots and sub-blocks are immediates)
  // K operand, K-step s: row r (+32 kb); fp16 chunk 2s+g, e4m3 chunks 4s+2g and 4s+2g+1 (each swizzled on its own)
  uint32_t k_rd[KS][KH];
#pragma unroll
  for (int s = 0; s < KS; ++s)
#pragma unroll
    for (int hh = 0; hh < KH; ++hh)
      k_rd[s][hh] = lds_base + C::K_ST0 + r * C::K_PITCH + ((((QK8 ? 4 : 2) * s + KH * g + hh) ^ swz_row<C::K_PITCH>(r)) * 16);
  // V operand: see the file comment.  li = lane within its block of 16.
  const int li = lane & 15;
  uint32_t v_rd[DB];
  uint32_t vt_rd[2] = {0, 0};
  if constexpr (C::VT) {  // row d = 32db + r of the [d][key] tile, chunks 2g and 2g+1 = keys 32g .. 32g+31
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) vt_rd[hh] = lds_base + C::V_ST0 + r * C::V_PITCH + (((2 * g + hh) ^ swz_row<C::V_PITCH>(r)) * 16);
#pragma unroll
    for (int db = 0; db < DB; ++db) v_rd[db] = 0;
  } else if constexpr (PV8) {
    const int row_e = li >> 1;
    const int v_key = 8 * (row_e >> 2) + 4 * g + (row_e & 3);  // + 16 u
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_rd[db] = lds_base + C::V_ST0 + v_key * C::V_PITCH + (((2 * db + ((lane >> 4) & 1)) ^ swz_v8<C::V_PITCH>(v_key)) * 16) + 8 * (li & 1);
  } else {
    const int v_key = 4 * g + (li >> 2);                       // + 16 ps + 8 h2
    const int v_col = 16 * ((lane >> 4) & 1) + 4 * (li & 3);   // + 32 db   (element index)
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_rd[db] = lds_base + C::V_ST0 + v_key * C::V_PITCH + ((((db * 32 + v_col) >> 3) ^ swz_v16<C::V_PITCH>(v_key)) * 16) + (v_col & 7) * 2;
  }

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
  // softmax reference point; this lane's running max of the raw scores (half of the query's keys); running sum;
  // raw-score threshold (m_ref + p_bias + kTau) / c above which the reference point moves
  float m_ref = -INFINITY, m_lane = -INFINITY, l_run = 0.f, thr_raw = -INFINITY;
  const float inv_c = 1.0f / c_log2;
  // e4m3 P: the row sum is taken on the MFMA pipe, which has cycles to spare there while the VALU does not.  One
  // 16x16x128 MFMA per 64 keys multiplies P^T (the same registers that feed the second GEMM) by a 0/1 matrix:
  // B lane (n = lane%16, block lane/16) is this kernel's lane (q = lane%32, g = lane/32), i.e. the 32 keys of query
  // n + 16*(block%2); A[m][block] = 1 iff block%2 == (m/4)%2, so output rows 4i..4i+3 of lane (n, i = lane/16) all
  // hold the sum over BOTH key halves of query n + 16*(i%2) = lane%32: every lane ends up with the sum of its own
  // query, no exchange needed.  It sums P as rounded to e4m3, the weights the second GEMM really applies.
  constexpr bool MFMA_SUM = PV8 && D <= 128;  // head dim 256 has no registers to spare, and twice the MFMA work per key
  constexpr bool DOT_SUM = !PV8;              // fp16 P: v_dot2_f32_f16 adds two rounded weights per instruction
  f32x4 l_acc = {0.f, 0.f, 0.f, 0.f};
  PReg sum_a;
  {
    const bool on = ((lane >> 4) & 1) == ((lane >> 2) & 1);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      if constexpr (PV8) sum_a[t] = on ? 0x38383838 : 0;  // e4m3 1.0 = 0x38
      else sum_a[t] = on ? (_Float16)1.0f : (_Float16)0.0f;
    }
  }

  // S^T = K . Q^T for the K tile in LDS stage `stage`
  constexpr int NPRE = C::KPRE;
  QReg kpre[NPRE ? NPRE : 1];
  auto read_kfrag = [&](uint32_t kt, int s, int kb) __attribute__((always_inline)) -> QReg {
    if constexpr (QK8) {
      const int4v lo = *LDS_AT(int4v, kt + k_rd[s][0] + kb * 32 * C::K_PITCH);
      const int4v hi = *LDS_AT(int4v, kt + k_rd[s][1] + kb * 32 * C::K_PITCH);
      return int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    } else {
      return *LDS_AT(half8, kt + k_rd[s][0] + kb * 32 * C::K_PITCH);
    }
  };
  // the first NPRE fragments (order: K-step major, 32-key block minor) of the K tile in slot `stage`
  auto prefetch_k = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
    for (int f = 0; f < NPRE; ++f) kpre[f] = read_kfrag(stage * C::K_TILE, f / KB, f % KB);
  };
  auto qk = [&](int stage, f32x16 (&sacc)[KB], bool use_pre = false) __attribute__((always_inline)) {
    const uint32_t kt = stage * C::K_TILE;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[kb][v] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        QReg ka;
        if (use_pre && s * KB + kb < NPRE) ka = kpre[s * KB + kb];
        else ka = read_kfrag(kt, s, kb);
        if constexpr (QK8) {
          sacc[kb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ka, qreg[s], sacc[kb], 0, 0, 0, 0, 0, 0);
        } else {
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qreg[s], sacc[kb], 0, 0, 0);
        }
      }
  };
  // Row max of a finished S tile and the deferred rescale (online_softmax.h:123-165).  The branch is wave-uniform.
  auto row_max_and_rescale = [&](const f32x16 (&sacc)[KB], int jt) __attribute__((always_inline)) {
    if (C::TAP_S && live) {  // the reference's -DCOPYOUTMM0 dump (fmha_consumer.h:31-42), here already scaled
      float *srow = a.s_tap + (((int64_t)b * a.H + h) * a.Sq + q0 + r) * (int64_t)a.Skv + (int64_t)jt * BN;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key0 = C::VT ? 32 * g + 16 * kb + 4 * i : 32 * kb + 8 * i + 4 * g;  // a lane's 4 consecutive keys
          f32x4 sv;
#pragma unroll
          for (int t = 0; t < 4; ++t) sv[t] = sacc[kb][4 * i + t] * a.s_scale;
          *(f32x4 *)(srow + key0) = sv;
        }
    }
    // The common case needs no exchange with the lane that holds the query's other keys: a lane only tests its own
    // half against the threshold, and the (rare, wave-uniform) slow path completes the max.
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = __builtin_fmaxf(mx, sacc[kb][v]);
    m_lane = __builtin_fmaxf(m_lane, mx);
    if (__builtin_amdgcn_ballot_w64(mx > thr_raw) != 0) {
      const float mfull = fmaxf(mx, __shfl_xor(mx, 32, 64)) * c_log2;
      const float m_new = fmaxf(m_ref, mfull - p_bias);
      const float alpha = __builtin_amdgcn_exp2f(m_ref - m_new);
      m_ref = m_new;
      thr_raw = (m_ref + p_bias + kTau) * inv_c;
      l_run *= alpha;
      if constexpr (MFMA_SUM) l_acc *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[db][v] *= alpha;
    }
  };
  // P = exp2(c*S - m_ref); row sum in fp32 before the down-cast (online_softmax.h:173-206); cast in the B-operand
  // register order of the second GEMM
  // DIRECT (DirectCfg builds: first pass with e4m3 P and the row sum on the matrix pipe, launched for callers that set
  // CFK_OPT_FAST_E4M3_WEIGHTS): the e4m3 code of a weight is built without an exponential.  Read as an integer, the code of a positive e4m3 number is 8 (log2 of it + 7) with the mantissa
  // interpolated linearly, so sat_u8(rne(8 (c S - m) + 56 - 0.46)) is exp2(c S - m) rounded to e4m3 up to that
  // interpolation (0.46: its mean; a fifth of the codes differ from the correctly rounded one, by one step; tests/
  // test_oracle.py pins the formula against the codec): one multiply-add and one v_cvt_pk_u8_f32 per score (4 issue
  // cycles each) in place of multiply-add, v_exp_f32 (8) and half a v_cvt_pk_fp8_f32 (8).  The conversion saturates at
  // 255: code 0x7F is NaN and reaches the row sum through the MFMA, codes from 0x80 on (negative numbers) are caught by
  // the OR of all P registers in p_flags.
  constexpr bool DIRECT_OK = C::DIRECT;
  static_assert(!C::DIRECT || (PV8 && MFMA_SUM), "direct codes: e4m3 P with the row sum on the matrix pipe");
  uint32_t p_flags = 0;
  auto softmax_exp = [&](auto direct, const f32x16 (&sacc)[KB], PReg (&pb)[PS]) __attribute__((always_inline)) {
    if constexpr (decltype(direct)::value && DIRECT_OK) {
      const float c8 = 8.0f * c_log2, m8 = 8.0f * m_ref - 55.54f;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          uint32_t code = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(sacc[kb][4 * w], c8, -m8), 0, 0u);
#pragma unroll
          for (int t = 1; t < 4; ++t) code = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(sacc[kb][4 * w + t], c8, -m8), t, code);
          p_flags |= code;
          pb[kb / 2][(kb % 2) * 4 + w] = (int)code;
        }
      return;
    }
    float rs = 0.f;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        float p[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          p[t] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][4 * w + t], c_log2, -m_ref));
          if constexpr (!MFMA_SUM && !DOT_SUM) rs += p[t];
        }
        if constexpr (PV8) {  // slot 16 kb + 4 w + t
          // the two converts overwrite both halves of the word: its old content is irrelevant, and handing in
          // the bits of p[0] (dead after this instruction) lets the result take p[0]'s register without a move
          int packed = __builtin_amdgcn_cvt_pk_fp8_f32(p[0], p[1], __builtin_bit_cast(int, p[0]), false);
          pb[kb / 2][(kb % 2) * 4 + w] = __builtin_amdgcn_cvt_pk_fp8_f32(p[2], p[3], packed, true);
        } else {              // K-step 2 kb + w / 2, slot 4 (w % 2) + t
#pragma unroll
          for (int t = 0; t < 4; ++t) pb[kb * 2 + w / 2][4 * (w % 2) + t] = (_Float16)p[t];
        }
      }
    if constexpr (DOT_SUM) {  // sum of P as rounded to fp16 (the weights the second GEMM applies), fp32 accumulation
      const half2v one2 = {(_Float16)1.0f, (_Float16)1.0f};
      float rs2 = 0.f;
#pragma unroll
      for (int ps = 0; ps < PS; ++ps)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const half2v pp = {pb[ps][2 * t], pb[ps][2 * t + 1]};
          if ((ps * 4 + t) & 1) rs2 = __builtin_amdgcn_fdot2(pp, one2, rs2, false);
          else rs = __builtin_amdgcn_fdot2(pp, one2, rs, false);
        }
      rs += rs2;
    }
    l_run += rs;
  };
  // the e4m3 V^T operand of K-step ps, d block db: four transpose reads (see the file comment)
  auto read_v8 = [&](uint32_t vt, int ps, int db) __attribute__((always_inline)) -> int8v {
    int8v va;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int2v x = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_AT(int2v, vt + v_rd[db] + (ps * 64 + u * 16) * C::V_PITCH));
      va[2 * u] = x[0];
      va[2 * u + 1] = x[1];
    }
    return va;
  };
  // O^T += V^T . P^T for the V tile in LDS stage `stage`
  auto pv = [&](uint32_t vt /* byte offset of the V slot */, const PReg (&pb)[PS]) __attribute__((always_inline)) {
    if constexpr (MFMA_SUM) {
#pragma unroll
      for (int ps = 0; ps < PS; ++ps) {
        if constexpr (PV8) l_acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(sum_a, pb[ps], l_acc, 0, 0, 0, 0, 0, 0);
        else l_acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(sum_a, pb[ps], l_acc, 0, 0, 0);
      }
    }
    if constexpr (PV8 && !C::VT && C::WPE == 2) {
      // two waves per SIMD: the operand of the next multiply is requested before the current multiply is issued, the
      // order pinned (left to itself the compiler reads, waits and multiplies one operand at a time: +0.8 %)
      int8v ring[2];
      ring[0] = read_v8(vt, 0, 0);
#pragma unroll
      for (int f = 0; f < PS * DB; ++f) {
        if (f + 1 < PS * DB) ring[(f + 1) & 1] = read_v8(vt, (f + 1) / DB, (f + 1) % DB);
        oacc[f % DB] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ring[f & 1], pb[f / DB], oacc[f % DB], 0, 0, 0, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      return;
    }
#pragma unroll
    for (int ps = 0; ps < PS; ++ps)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        if constexpr (C::VT) {
          const int4v lo = *LDS_AT(int4v, vt + vt_rd[0] + db * 32 * C::V_PITCH);
          const int4v hi = *LDS_AT(int4v, vt + vt_rd[1] + db * 32 * C::V_PITCH);
          const int8v va = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          oacc[db] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, pb[ps], oacc[db], 0, 0, 0, 0, 0, 0);
        } else if constexpr (PV8) {
          const int8v va = read_v8(vt, ps, db);
          oacc[db] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(va, pb[ps], oacc[db], 0, 0, 0, 0, 0, 0);
        } else {
          const uint32_t vp = vt + v_rd[db] + ps * 16 * C::V_PITCH;
          union {
            struct { short4v lo, hi; } s;
            half8 h;
          } va;
          va.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(short4v, vp));
          va.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(short4v, vp + 8 * C::V_PITCH));
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va.h, pb[ps], oacc[db], 0, 0, 0);
        }
      }
  };

  // e4m3 P: the three parts of a tile's work -- S_{j+1} = K.Q^T, the exponentials of S_j, O += P.V -- are kept apart as
  // blocks (scheduling fences) instead of being interleaved by the compiler.  The VALU is the busy unit of that kernel
  // (per key the softmax costs what it costs for fp16 P, the MFMA time is halved); with the blocks apart the two waves
  // of a SIMD overlap one wave's exponentials with the other's MFMAs: B=4 H=16 S=4096 D=128 2243-2334 against 2198-2269
  // TFLOP/s on N(0,1) tensors (two boxes), 2798 against 2664 on constant ones; head dim 64 +1.2 %.  One wave per SIMD
  // (head dim 256) gains most with the exponentials in front of the first GEMM: 2124 against 2050 (+0.8 % in the other
  // order).  With fp16 P the same fences lose (hybrid -2..-8 %, fp16 -2..-10 %): those kernels keep the compiler's order.
  constexpr bool FENCED = PV8;
  constexpr bool EXP_FIRST = PV8 && C::WPE == 1;
  auto fence = [&]() __attribute__((always_inline)) {
    if constexpr (FENCED) __builtin_amdgcn_sched_barrier(0);
  };
  // qk(next) and the exponentials of the current tile, in the order of the build
  auto qk_and_exp = [&](auto track, auto has_next, int k_stage, f32x16 (&s_nxt)[KB], f32x16 (&s_cur)[KB], PReg (&pb)[PS]) __attribute__((always_inline)) {
    constexpr bool HAS_NEXT = decltype(has_next)::value;
    constexpr std::integral_constant<bool, decltype(track)::direct> direct{};
    if constexpr (EXP_FIRST) {
      softmax_exp(direct, s_cur, pb);
      fence();
      if (HAS_NEXT) qk(k_stage, s_nxt);
    } else {
      if (HAS_NEXT) qk(k_stage, s_nxt);
      fence();
      softmax_exp(direct, s_cur, pb);
    }
    fence();
  };

  // One pipeline step for tile j (parity P = j & 1).  On entry: s_cur = S_j is finished and its max is folded into
  // m_ref; K_{j+1} sits in K stage P^1 and V_j in V stage P.  HAS_NEXT is false for the last tile only.
  auto step = [&](auto track, auto parity, auto has_next, int j, f32x16 (&s_cur)[KB], f32x16 (&s_nxt)[KB]) __attribute__((always_inline)) {
    constexpr bool TRACK = decltype(track)::value;
    constexpr int P = decltype(parity)::value;
    constexpr bool HAS_NEXT = decltype(has_next)::value;
    // prefetch K_{j+2} into K stage P (last read by step j-1) and V_{j+1} into V stage P^1 (ditto); the indices are
    // clamped at the end, which only rewrites a stage nobody reads any more
    load_k(j + 2 < n_tiles ? j + 2 : n_tiles - 1, P);
    load_v(j + 1 < n_tiles ? j + 1 : n_tiles - 1, P ^ 1);
    PReg pb[PS];
    qk_and_exp(track, has_next, P ^ 1, s_nxt, s_cur, pb);
    pv(P * C::V_TILE, pb);
    if (TRACK && HAS_NEXT) row_max_and_rescale(s_nxt, j + 1);
    wait_lds_dma();   // this wave's copies have landed ...
    __syncthreads();  // ... and so have everybody else's; all reads of the stages about to be refilled are done
  };

  // Two sub-tiles per barrier (SUB = 2): sub-tile s of K lives in K slot s % 4, sub-tile t of V in V slot t % 4.
  // Step J covers sub-tiles 2J and 2J+1.  On entry s_a = S_{2J} is finished and folded into m_ref; K sub-tiles
  // 2J+1, 2J+2 and V sub-tiles 2J, 2J+1 are in LDS.  The step refills the slots last read by step J-1: K sub-tiles
  // 2J+3, 2J+4 at its start, V sub-tiles 2J+2, 2J+3 between its halves.  LAST: sub-tile 2J+1 is the final one.
  auto step2 = [&](auto track, auto parity, auto last, int J, f32x16 (&s_a)[KB], f32x16 (&s_b)[KB]) __attribute__((always_inline)) {
    constexpr bool TRACK = decltype(track)::value;
    constexpr int P = decltype(parity)::value;
    constexpr bool LAST = decltype(last)::value;
    const int t0 = 2 * J, t_max = n_tiles - 1;
    load_k(t0 + 3 < t_max ? t0 + 3 : t_max, (2 * P + 3) % 4);
    load_k(t0 + 4 < t_max ? t0 + 4 : t_max, (2 * P) % 4);
    {
      PReg pb[PS];
      qk_and_exp(track, std::true_type{}, (2 * P + 1) % 4, s_b, s_a, pb);
      pv(((2 * P) % 4) * C::V_TILE, pb);
      if (TRACK) row_max_and_rescale(s_b, t0 + 1);
    }
    load_v(t0 + 2 < t_max ? t0 + 2 : t_max, (2 * P + 2) % 4);
    load_v(t0 + 3 < t_max ? t0 + 3 : t_max, (2 * P + 3) % 4);
    {
      PReg pb[PS];
      qk_and_exp(track, std::integral_constant<bool, !LAST>{}, (2 * P + 2) % 4, s_a, s_b, pb);
      pv(((2 * P + 1) % 4) * C::V_TILE, pb);
      if (TRACK && !LAST) row_max_and_rescale(s_a, t0 + 2);
    }
    wait_lds_dma();
    __syncthreads();
  };

  // K fragment prefetch (KPRE): K tile t lives in K slot t % 4 and is fetched two steps ahead, so the tile of the NEXT
  // step's S = K.Q^T is complete before this step's barrier and its first fragments are read into registers in front
  // of the barrier: the MFMA pipe restarts right behind it instead of waiting for LDS while all waves read at once.
  // The copies are issued after the step's K reads, off the restart path.
  auto step_p = [&](auto track, auto jmod4, auto has_next, int j, f32x16 (&s_cur)[KB], f32x16 (&s_nxt)[KB]) __attribute__((always_inline)) {
    constexpr bool TRACK = decltype(track)::value;
    constexpr int J4 = decltype(jmod4)::value;
    constexpr int P = J4 & 1;
    constexpr bool HAS_NEXT = decltype(has_next)::value;
    PReg pb[PS];
    if (HAS_NEXT) qk((J4 + 1) % 4, s_nxt, true);
    load_k(j + 3 < n_tiles ? j + 3 : n_tiles - 1, (J4 + 3) % 4);
    load_v(j + 1 < n_tiles ? j + 1 : n_tiles - 1, P ^ 1);
    softmax_exp(std::integral_constant<bool, decltype(track)::direct>{}, s_cur, pb);
    pv(P * C::V_TILE, pb);
    if (HAS_NEXT) {
      prefetch_k((J4 + 2) % 4);
      if (TRACK) row_max_and_rescale(s_nxt, j + 1);
    }
    wait_lds_dma();
    __syncthreads();
  };

  // ---- Two passes over the keys (e4m3 P).  The first one takes the row max of the first tile only and then trusts
  // the range of P: no row max, no comparison, no branch per tile (on N(0,1) data +14 % at head dims 64 and 128).  A
  // weight that leaves the range of e4m3 turns into NaN (v_cvt_pk_fp8_f32 has no infinity; it does so above 464) and
  // from there into a non-finite O and l for that query, which is looked for once, after the loop.
  // Only if some row of the workgroup shows it, the keys are walked again with the row max tracked tile by tile, the
  // reference's algorithm (online_softmax.h:123-165).  The taps need the true row max: they go straight to that pass,
  // and so do e4m3 weights on short key sequences (tau = 0: there the row's largest weight has to stay an exact power
  // of two, which only a reference point that follows the max gives).
  using std::integral_constant;
  f32x16 s_a[KB], s_b[KB];
  auto pass = [&](auto track) __attribute__((always_inline)) {
    constexpr bool TRACK = decltype(track)::value;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[db][v] = 0.f;
    m_ref = -INFINITY, m_lane = -INFINITY, l_run = 0.f, thr_raw = -INFINITY;
    l_acc = f32x4{0.f, 0.f, 0.f, 0.f};
    // (the direct codes have no subnormals -- everything below 2^-7 becomes 0 -- so that form keeps the reference point 2
    // below the first tile's max: a row whose first tile holds an unusually large score would lose the bulk of its keys)
    p_bias = PV8 ? (TRACK ? 7.0f : decltype(track)::direct ? 2.0f : 0.0f) : 0.0f;
    if constexpr (C::KPRE > 0) {
      // ---- prologue: K_0, K_1, K_2, V_0 in flight; S_0, its row max, first fragments of K_1.  n_tiles % 4 == 0.
      using T = integral_constant<bool, true>;
      using F = integral_constant<bool, false>;
      const int t_max = n_tiles - 1;
      load_k(0, 0);
      load_v(0, 0);
      load_k(1, 1);
      load_k(2 < t_max ? 2 : t_max, 2);
      wait_lds_dma();
      __syncthreads();
      qk(0, s_a);
      prefetch_k(1);
      row_max_and_rescale(s_a, 0);
      int j = 0;
      for (; j + 4 < n_tiles; j += 4) {
        step_p(track, integral_constant<int, 0>{}, T{}, j, s_a, s_b);
        step_p(track, integral_constant<int, 1>{}, T{}, j + 1, s_b, s_a);
        step_p(track, integral_constant<int, 2>{}, T{}, j + 2, s_a, s_b);
        step_p(track, integral_constant<int, 3>{}, T{}, j + 3, s_b, s_a);
      }
      step_p(track, integral_constant<int, 0>{}, T{}, j, s_a, s_b);
      step_p(track, integral_constant<int, 1>{}, T{}, j + 1, s_b, s_a);
      step_p(track, integral_constant<int, 2>{}, T{}, j + 2, s_a, s_b);
      step_p(track, integral_constant<int, 3>{}, F{}, j + 3, s_b, s_a);
    } else if constexpr (C::SUB == 2) {
      // ---- prologue: K_0, K_1, K_2, V_0, V_1 in flight; S_0 and its row max.  n_tiles is even and >= 2.
      const int t_max = n_tiles - 1;
      load_k(0, 0);
      load_v(0, 0);
      load_k(1, 1);
      load_k(2 < t_max ? 2 : t_max, 2);
      load_v(1, 1);
      wait_lds_dma();
      __syncthreads();
      qk(0, s_a);
      row_max_and_rescale(s_a, 0);
      __syncthreads();  // every wave is done with K slot 0 before step 0 overwrites it
      const int n_steps = n_tiles / 2;
      int J = 0;
      for (; J + 2 < n_steps; J += 2) {
        step2(track, integral_constant<int, 0>{}, integral_constant<bool, false>{}, J, s_a, s_b);
        step2(track, integral_constant<int, 1>{}, integral_constant<bool, false>{}, J + 1, s_a, s_b);
      }
      if (J + 2 == n_steps) {
        step2(track, integral_constant<int, 0>{}, integral_constant<bool, false>{}, J, s_a, s_b);
        step2(track, integral_constant<int, 1>{}, integral_constant<bool, true>{}, J + 1, s_a, s_b);
      } else {
        step2(track, integral_constant<int, 0>{}, integral_constant<bool, true>{}, J, s_a, s_b);
      }
    } else {
      // ---- prologue: K_0, V_0, K_1 in flight; S_0 and its row max
      load_k(0, 0);
      load_v(0, 0);
      load_k(n_tiles > 1 ? 1 : 0, 1);
      wait_lds_dma();
      __syncthreads();
      qk(0, s_a);
      row_max_and_rescale(s_a, 0);
      __syncthreads();  // every wave is done with K stage 0 before step 0 overwrites it

      int j = 0;
      for (; j + 2 < n_tiles; j += 2) {
        step(track, integral_constant<int, 0>{}, integral_constant<bool, true>{}, j, s_a, s_b);
        step(track, integral_constant<int, 1>{}, integral_constant<bool, true>{}, j + 1, s_b, s_a);
      }
      if (j + 2 == n_tiles) {  // two tiles left: j (even) with a successor, then the last one
        step(track, integral_constant<int, 0>{}, integral_constant<bool, true>{}, j, s_a, s_b);
        step(track, integral_constant<int, 1>{}, integral_constant<bool, false>{}, j + 1, s_b, s_a);
      } else {                 // one tile left (even index)
        step(track, integral_constant<int, 0>{}, integral_constant<bool, false>{}, j, s_a, s_b);
      }
    }

  };
  // (fp16 P gains nothing from the first pass -- its row max hides behind the second GEMM's MFMAs -- and skips it.)
  bool redo = !PV8 || C::TAP_S || a.row_max != nullptr || a.row_sum != nullptr || !(kTau > 0.f) || a.track_only != 0;
  if (!redo) {
    pass(PassKind<false, DIRECT_OK>{});
    const float l_chk = MFMA_SUM ? l_acc[0] : l_run;
    const bool bad = !(__builtin_fabsf(oacc[0][0]) < 3.0e38f) || !(l_chk < 3.0e38f) || (p_flags & 0x80808080u) != 0;
    redo = __syncthreads_or(bad) != 0;
  }
  if (redo) pass(PassKind<true, false>{});

  // ---- epilogue: O = out_scale * O / l (online_softmax.h:59-85), fp16, [B,S,H,D]; a lane holds 4 consecutive d
  const float l_tot = MFMA_SUM ? l_acc[0] : l_run + __shfl_xor(l_run, 32, 64);
  const float inv = a.out_scale / l_tot;
  const int qrow = q0 + r;
  // The accumulator layout gives a lane 4 consecutive d of ONE row: stored directly, a wave-wide store would touch
  // 32 rows with 16 bytes each.  The wave's 32 x D tile goes through its own LDS region instead (all staged tiles
  // are dead after the loop's last barrier) and leaves as whole rows, 16 bytes per lane.
  {
    char *ot = smem + wave * (32 * C::O_PITCH);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        half4 o4;
#pragma unroll
        for (int t = 0; t < 4; ++t) o4[t] = (_Float16)(oacc[db][4 * i + t] * inv);
        *(half4 *)(ot + r * C::O_PITCH + (db * 32 + 8 * i + 4 * g) * 2) = o4;
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    constexpr int LPR = D / 8;        // lanes per output row (16 bytes each)
    constexpr int RPP = 64 / LPR;     // rows per wave-wide store
    const int orow_l = lane / LPR, ochunk = lane % LPR;
#pragma unroll
    for (int pass = 0; pass < 32 / RPP; ++pass) {
      const int row = pass * RPP + orow_l;
      const int4v val = *(const int4v *)(ot + row * C::O_PITCH + ochunk * 16);
      if (live) *(int4v *)(Op + (int64_t)(q0 + row) * ld + ochunk * 8) = val;
    }
  }
  if (live && (a.row_max || a.row_sum)) {
    const float m_true = fmaxf(m_lane, __shfl_xor(m_lane, 32, 64)) * c_log2;
    if (g == 0) {
      const int64_t si = ((int64_t)b * a.H + h) * a.Sq + qrow;
      // taps are reported against the true row max, as the reference's miOut / sPrimeOut are (fmha_epilogue.h:7-46)
      if (a.row_max) a.row_max[si] = m_true;
      if (a.row_sum) a.row_sum[si] = l_tot * __builtin_amdgcn_exp2f(m_ref - m_true);
    }
  }
}

// One-time set-up of an instantiation: raise its dynamic-LDS limit.  Thread-safe (first calls of one shape from several
// host threads), and callable ahead of any launch (cfk_init) so that a first call under stream capture finds it done.
template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(C::WPE, C::WPE))) fmha_fwd_kernel16(const FmhaArgs a);
template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(2, 2))) fmha_fwd_kernel16p(const FmhaArgs a);
template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(2, 2))) fmha_fwd_kernel8p(const FmhaArgs a);
template <class C>
__global__ void __launch_bounds__(C::T) fmha_fwd_kernel_ks(const FmhaArgs a);

// the kernel an instantiation runs
// The same build with the e4m3 weights of the first pass written as codes, without an exponential (see softmax_exp in
// fmha_fwd_kernel and gen_fmha_loop8.py): what a call gets under cfk_set_option(CFK_OPT_FAST_E4M3_WEIGHTS, 1).
template <class C>
struct DirectCfg : C {
  static constexpr bool DIRECT = true;
};
template <class C>
constexpr bool has_direct_build = C::PV8 && C::D <= 128 && !C::TAP_S && !C::KSPLIT;

// What the query length has to be a multiple of: the compiler-scheduled 32x32 kernel (fmha_fwd_kernel) and the
// hand-scheduled kernels (fmha_fwd_kernel16p, fmha_fwd_kernel8p) take a last query tile filled to a whole number of
// waves (32 rows each), the other kernels whole tiles.  (The reference: whole
// tiles of its compile-time 64 or 128 rows, src/fmha-pipeline/shared_storage.h:4-15.)
template <class C>
constexpr int q_multiple = !C::KSPLIT && (C::ASM || !C::M16) ? 32 : C::BM;

template <class C>
constexpr auto fmha_kernel_of() {
  if constexpr (C::KSPLIT) return &fmha_fwd_kernel_ks<C>;
  else if constexpr (C::ASM && C::QK8) return &fmha_fwd_kernel8p<C>;
  else if constexpr (C::ASM) return &fmha_fwd_kernel16p<C>;
  else if constexpr (C::M16) return &fmha_fwd_kernel16<C>;
  else return &fmha_fwd_kernel<C>;
}

// Persistent workgroups (FmhaCfg::ASM): one per CU -- a multiple of the 8 XCDs, so that a workgroup's items stay on its
// XCD -- or one per item where there are no more items than CUs (any number: nobody takes a second item then).
inline int persistent_grid(int n_items) {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8) n = 256;
    return n / 8 * 8;
  }();
  return n_items <= cus ? n_items : cus;
}

template <class C>
hipError_t prepare_fmha_cfg() {
  static std::once_flag once;
  static hipError_t status = hipSuccess;
  std::call_once(once, [] {
    status = hipFuncSetAttribute((const void *)fmha_kernel_of<C>(), hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if constexpr (has_direct_build<C>) {
      const hipError_t e = hipFuncSetAttribute((const void *)fmha_kernel_of<DirectCfg<C>>(), hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
      if (status == hipSuccess) status = e;
    }
  });
  return status;
}

template <class C>
hipError_t launch_fmha_cfg(const FmhaArgs &a, hipStream_t s) {
  const hipError_t e = prepare_fmha_cfg<C>();
  if (e != hipSuccess) return e;
  const int items = a.B * a.H * ((a.Sq + C::BM - 1) / C::BM);
  const int grid = C::ASM ? persistent_grid(items) : items;
  if constexpr (has_direct_build<C>) {
    if (a.direct_p != 0) {
      hipLaunchKernelGGL(fmha_kernel_of<DirectCfg<C>>(), dim3(grid), dim3(C::T), C::LDS_BYTES, s, a);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL(fmha_kernel_of<C>(), dim3(grid), dim3(C::T), C::LDS_BYTES, s, a);
  return hipGetLastError();
}

template <class C>
void fill_fmha_plan(int sq, int bh, FmhaPlan *p) {
  p->block_m = C::BM;
  p->block_n = C::BN * C::SUB;
  p->kv_multiple = C::ASM && C::D != 256 ? C::BN : C::BN * C::SUB;
  p->q_multiple = q_multiple<C>;
  p->mfma = C::M16 ? 16 : 32;
  p->lds_bytes = C::LDS_BYTES;
  p->threads = C::T;
  p->grid = bh * ((sq + C::BM - 1) / C::BM);
  if constexpr (C::KSPLIT) {
    snprintf(p->kernel, sizeof p->kernel, "fmha_fwd_kernel_ks<%d,%d>", C::D, C::NWAVES);
    return;
  }
  snprintf(p->kernel, sizeof p->kernel, "%s<%d,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d>",
           C::ASM ? (C::QK8 ? "fmha_fwd_kernel8p" : "fmha_fwd_kernel16p") : C::M16 ? "fmha_fwd_kernel16" : "fmha_fwd_kernel", C::D, C::BN, C::NWAVES, C::WPE,
           (int)C::QK8, (int)C::PV8, (int)C::VT, (int)C::TAP_S, C::SUB, C::KPRE, (int)C::M16, (int)C::ASM);
  if constexpr (has_direct_build<C>) {
    if (fast_e4m3_weights()) strncat(p->kernel, "/direct", sizeof p->kernel - strlen(p->kernel) - 1);   // the DirectCfg build
  }
}

// ---- tile selection.  The reference fixes its tile at compile time (-DQBLKSIZE / -DKBLKSIZE,
// src/fmha-pipeline/shared_storage.h:4-15, swept by compile_run_all_config.sh:3-6); here every shape is built and one is
// picked per call.  CFK_FMHA_TILE=<query rows>x<keys>[/16|/16h|/32|/32h] (e.g. 256x128, or 256x64/16 for the build on
// 16x16x32 MFMAs, 256x128/16h and 256x128/32h for the fp16 / e4m3 ones with the hand-scheduled main loop, 32x64 for the
// key-split build), or small | large for the query rows alone, states a wish; a wish no instantiation can serve for the given shape is ignored.  CFK_FMHA_HANDLOOP=0 keeps
// the automatic choice off the hand-scheduled builds (for A/B measurements).
struct TileWish {
  int bm, bn;  // 0 = no wish
  int mfma;    // 16 or 32: the MFMA shape of the build (fp16 kernels come in both); 0 = no wish
  int hand;    // +1: the build with the hand-scheduled loop, -1: a compiler-scheduled build, 0 = no wish
};
inline TileWish tile_wish() {
  static const TileWish w = [] {
    TileWish t{0, 0, 0, 0};
    const char *e = getenv("CFK_FMHA_TILE");
    if (!e) return t;
    if (e[0] == 's') t.bm = 128;
    else if (e[0] == 'l') t.bm = 256;
    else {
      int bm = 0, bn = 0, mfma = 0;
      char suffix = 0;
      const int n = sscanf(e, "%dx%d/%d%c", &bm, &bn, &mfma, &suffix);
      if (n >= 2) {
        const bool shape = n >= 3 && (mfma == 16 || mfma == 32);
        t = TileWish{bm, bn, shape ? mfma : 0, !shape ? 0 : (n == 4 && suffix == 'h') ? 1 : -1};
      }
    }
    return t;
  }();
  return w;
}

template <class... Cs>
struct CfgList {};

// the shapes an instantiation can run: whole query tiles (fmha_fwd_kernel: whole waves), whole key steps (four key tiles per loop turn with the K
// fragment prefetch and in the e4m3 hand-scheduled loop; the hand-scheduled loops need eight tiles to fill and drain;
// two tiles with the two-tile step)
template <class C>
constexpr bool fits(int sq, int skv) {
  // (the hand-scheduled builds at head dims 64 and 128 take up to three tiles behind the last group of four outside
  // their loop)
  return sq % q_multiple<C> == 0 && skv % (C::BN * (C::ASM && C::D != 256 ? 1 : C::KPRE || C::ASM ? 4 : C::SUB)) == 0 &&
         (!C::ASM || skv >= 8 * C::BN);
}

// Where a hand-scheduled persistent build (one workgroup per CU, each walking its share of the work items) beats the
// one-workgroup-per-item builds: measured over problem sizes (driver/run_problem_sizes.sh; 300 launches each, N(0,1)
// data).  fp16 at head dim 256, where both kinds of build have 128-row items: at every item count from 1024 keys on
// (+25..30 % at 8192 keys, +10..20 % at 1024 and 2048; -1..-4 % at 512, -15 % at 256 keys: eight tiles, all head and
// tail).  fp16
// at head dims 64 and 128: from more 256-row items than half the CUs on (160 items +25 %, 256 items +23..28 %, 320 items
// +9 %; at 128 items a tie, at 96 -4 %: there the 128-row tile's twice as many workgroups count).  Up to 256 items of 128
// rows -- one round -- those head dims take the same loops in their 4-wave shape (128 rows, one wave per SIMD): +11..20 %
// over the compiler-scheduled 128-row builds from 1024 keys on (2048 keys +12 %, 8192 +20 %, 1024 +2..6 %, 512 -5 %).
// e4m3: the 8-wave shape from more than 128 items on (132 to 156 items +7..11 %, 160 and more +8..13 %; at 128 items -11 %) and only while the last round of items keeps
// four fifths of the workgroups busy (320 items -8 %, 384 items -5 %: the 128-row tile has twice the workgroups to even
// out the tail); up to 256 items of 128 rows the 4-wave shape (+9..20 % over the compiler-scheduled 128-row build).
// Those figures hold from 3072 keys on, where every e4m3 build starts with the pass that takes no row max per tile (3072
// keys: 4 waves +10..16 %; 8 waves +6..12 % at 288 to 480 items of 128 rows and 896 to 960, -3..-8 % at 576 to 768).  Below,
// the compiler-scheduled builds run their max-tracking pass only and are 19..50 % slower than this loop.
template <class C>
constexpr bool hand_loop_pays(long long items, int skv) {
  if (!C::QK8) {
    if (C::D == 256) return skv >= 1024;
    // (key tiles behind the last group of four run outside the generated loop, at three to four times a tile's time in it:
    // worth it from 2048 keys on and while they are few -- 2112 keys +9 %, 3008 keys with three of them 0..+27 %, 704 keys
    // with three -15 %, 1088 keys with one -9 %)
    const int n_tiles = skv / C::BN, n_left = n_tiles & 3;
    if (n_left != 0 && (n_tiles < 32 || n_left * 10 > n_tiles)) return false;
    return C::BM == 128 ? items <= 256 && skv >= 1024 : items > 128;
  }
  // (e4m3: the first pass sets its reference point from the first key tile, so a row's largest weight is not an exact
  // power of two as it is for a reference point that follows the running max; over few keys the rounding of that weight
  // does not average out -- cfk_api.hip has the figures -- so key lengths below 3072 take the max-tracking pass, which this
  // build only has as an unpipelined fall-back: there it runs by wish only (CFK_FMHA_TILE=256x128/32h or 128x128/32h;
  // 19..50 % faster than the max-tracking compiler-scheduled builds))
  if (skv < 3072) return false;
  // (tiles behind the last group of four, which run outside the generated loop, cost about what the loop gains: 3136
  // keys +4..6 %, 4160 / 4224 / 4288 keys -3 / -12 / -3 % with 8 waves and a tie with 4: taken below 4096 keys only)
  if (skv >= 4096 && skv % (4 * C::BN) != 0) return false;
  if (C::BM == 128) return items <= 256;   // (the 4-wave shape: one round of 128-row items)
  const long long rounds = (items + 255) / 256;
  return items > 128 && (rounds == 1 || items * 5 >= rounds * 256 * 4);
}

// (The compiler-scheduled fp16 256-row builds need key length to pay: B=8 H=27 S_q=1536 D=128 with 896 keys 723 TFLOP/s on
// 256 x 128 keys, 871 on 256 x 64, 947 on 128 x 64, all on 16x16x32 MFMAs; with 1536 keys 1036 / 1038 / 1014.  e4m3, B=8 H=32
// S_q=2048 D=128: 1024 keys 1445 on 256 x 128 against 1517 on 128 x 64, 1536 keys 1529 / 1573, 2048 keys 1702 / 1705.)
// Calls f with the first instantiation of the list that fits the shape and the wish.  Without a wish for the query
// rows, the hand-scheduled builds are taken where they pay (above), other tiles above 128 rows and the other 16x16x32
// builds (slower where launch and prologue dominate) only for big problems (size 2: enough workgroups to fill 256 CUs
// twice), and the key-split build only for small ones (size 0: its 32-row workgroups fit on the chip all at once).
template <class F, class... Cs>
bool first_fit(CfgList<Cs...>, int sq, int skv, long long bh, int size, TileWish w, F &&f) {
  bool done = false;
  auto try_one = [&](auto c) {
    using C = decltype(c);
    if (done || !fits<C>(sq, skv)) return;
    // (a 256-row tile whose last waves lie behind the last query row idles them: worth it while the hand-scheduled loop's
    // lead over a 128-row build -- 20..30 % for fp16, 7..9 % for e4m3 -- outweighs the idle share of the rows: up to a
    // quarter of them at head dim 128 (S_q=384: +6 %), an eighth at head dim 64 (S_q=640, a sixth idle: -4 %), a
    // sixteenth for e4m3)
    const long long padded = (long long)((sq + C::BM - 1) / C::BM) * C::BM;
    const bool tight = C::BM <= 128 || (padded - sq) * (C::QK8 ? 16 : C::D == 64 ? 8 : 4) <= padded;
    // (... and the fp16 256-row builds while what they lose -- to idle rows, to key tiles behind the last group of four
    // (each about 2.5 tile times more) and to a last round of work items that leaves CUs idle (the 128-row builds
    // lose about half as much to theirs) -- adds up to at most a quarter: over three draws of 100 problem sizes,
    // automatic choice against CFK_FMHA_HANDLOOP=0, every choice that lost more than the noise summed to 0.29 or more)
    bool stacked_ok = true;
    if (C::ASM && !C::QK8 && C::BM > 128) {
      const long long items = bh * (padded / C::BM), rounds = (items + 255) / 256;
      const int n_tiles = skv / C::BN, n_left = C::D == 256 ? 0 : n_tiles & 3;
      const double idle_rows = 1.0 - (double)sq / padded, tail = 2.5 * n_left / n_tiles;
      const double last_round = rounds > 1 ? 1.0 - (double)items / (rounds * 256) : 0.0;
      // (head dim 64: the larger lead; below 1024 keys, where the loop is all head and tail and the lead a few per cent, a
      // thin last round counts in full: 512 keys, 310 items -16 %)
      stacked_ok = n_tiles < 16 ? idle_rows + last_round <= 0.2 : idle_rows + tail + 0.5 * last_round <= (C::D == 64 ? 0.32 : 0.25);
    }
    // (the compiler-scheduled 256-row builds for e4m3 Q and K -- one 8-wave workgroup per CU -- against the 128-row tile, at
    // 2048 and 4096 keys: 128 items of 256 rows -20 %, 160 to 256 +2..8 %, 320 and 384 -7..-13 %, 512 +1..5 %, 576 -7..-10 %,
    // 768 0..+4 %: taken while their rounds of 256 workgroups fill)
    const long long items256 = bh * ((sq + 255) / 256), rounds256 = (items256 + 255) / 256;
    const bool fills256 = sq % 256 == 0 && items256 >= 160 && (rounds256 == 1 || items256 * 5 >= rounds256 * 256 * 4);
    const bool by_size = C::ASM ? tight && stacked_ok && hand_loop_pays<C>(bh * ((sq + C::BM - 1) / C::BM), skv)
                                : (C::QK8 && C::BM > 128 ? fills256 : !((C::BM > 128 || C::M16) && size != 2)) &&
                                      !(C::BM > 128 && skv < (C::PV8 ? 2048 : C::QK8 ? 0 : 1152));
    if (C::KSPLIT ? (w.bm ? C::BM != w.bm : size != 0) : (w.bm ? C::BM != w.bm : !by_size)) return;
    if (w.bn && C::BN * C::SUB != w.bn) return;
    if (w.mfma && (C::M16 ? 16 : 32) != w.mfma) return;
    if (w.hand && C::ASM != (w.hand > 0)) return;
    f(c);
    done = true;
  };
  (try_one(Cs{}), ...);
  return done;
}

// wish first (over every instantiation), then the automatic order, then -- for shapes nothing fits -- the fallback,
// whose tile the caller's divisibility check then names in its error
template <class All, class Auto, class Fallback, class F>
void select_tile(int sq, int skv, int bh, F &&f) {
  const bool big = sq % 256 == 0 && (long long)bh * (sq / 256) >= 512;
  const bool small = (long long)bh * ((sq + 31) / 32) <= 256 && skv >= 128;
  const int size = big ? 2 : small ? 0 : 1;
  const TileWish w = tile_wish();
  if ((w.bm || w.bn) && first_fit(All{}, sq, skv, bh, size, w, f)) return;
  static const bool no_hand = [] { const char *e = getenv("CFK_FMHA_HANDLOOP"); return e && e[0] == '0'; }();
  // (the hand-scheduled build is a two-pass kernel: not for callers that asked for a data-independent run time)
  if (first_fit(Auto{}, sq, skv, bh, size, TileWish{0, 0, 0, no_hand || predictable_latency() ? -1 : 0}, f)) return;
  f(Fallback{});
}

template <class... Cs>
hipError_t prepare_all(CfgList<Cs...>) {
  hipError_t e = hipSuccess;
  auto one = [&](auto c) {
    const hipError_t r = prepare_fmha_cfg<decltype(c)>();
    if (e == hipSuccess) e = r;
  };
  (one(Cs{}), ...);
  return e;
}

}  // namespace cfk
