// The fp16 FMHA forward kernel for small grids (KsCfg below): the waves of a workgroup split the KEYS, not the query
// rows.  A problem like B=1 H=8 S=512 D=64 gives the 128-row tile 32 workgroups for 256 CUs, each of which walks its
// eight key tiles one after the other: the run time is that chain of dependent steps (copy, barrier, S = K.Q^T, softmax,
// O += P.V), not arithmetic.  Here a workgroup owns 32 query rows (four times as many workgroups) and its NWAVES waves
// take the 64-key tiles round-robin (tile j goes to wave j % NWAVES), each with its own running max, row sum and O; the
// partial results meet in the LDS at the end (the merge of online_softmax.h:123-165 across waves instead of across
// tiles).  The chain per wave is then one eighth as long, and no barrier sits inside it.
//
// Mathematics, MFMA shape and register layouts are those of fmha_fwd_kernel16.h (16x16x32 MFMAs; lane (c, g) holds keys
// 16 kb + 4 g .. +3 of query 16 qb + c).  K fragments come straight from global memory in MFMA operand order (16 bytes
// per lane); V goes through a wave-private LDS tile (global->LDS copy, then transposing reads), so no wave waits for
// another before the merge.
#pragma once
#include "fmha_fwd_kernel16.h"

namespace cfk {

// The configuration of a key-split build: head dim, waves (= key tiles in flight per workgroup).  What it shares with
// FmhaCfg (tile formats, pitches) comes from there; a workgroup owns 32 query rows, every wave copies whole V tiles.
template <int D_, int NWAVES_>
struct KsCfg : FmhaCfg<D_, 64, NWAVES_, 1, false, false, false, false, 1, 0, true> {
  using Base = FmhaCfg<D_, 64, NWAVES_, 1, false, false, false, false, 1, 0, true>;
  static constexpr bool KSPLIT = true;
  static constexpr int BM = 32;
  static constexpr int V_IPW = Base::V_ROWS / Base::V_RPI;   // 1 KB copies per V tile, all by the wave that owns it
  // one V tile per wave (later its partial O, fp32: the same size) and 4 KB of per-query statistics
  static constexpr int LDS_BYTES = NWAVES_ * Base::V_TILE + 4096;
};

template <class C>
__global__ void __launch_bounds__(C::T) fmha_fwd_kernel_ks(const FmhaArgs a) {
  static_assert(C::KSPLIT && C::M16 && !C::QK8 && !C::PV8 && !C::VT && !C::TAP_S && C::BN == 64, "fp16, 64-key tiles");
  constexpr int D = C::D, BN = 64, W = C::NWAVES;
  constexpr int QB = 2, KB = BN / 16, KS = D / 32, DB = D / 16, PS = BN / 32;
  constexpr uint32_t kStats = W * C::V_TILE;   // behind the waves' tiles: m[W][32], l[W][32], true max [W][32]
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;

  const int q_blocks = a.Sq / 32;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / q_blocks;
  const int q0 = (tile - bh * q_blocks) * 32;
  const int b = bh / a.H, h = bh - b * a.H;
  const int64_t ld = (int64_t)a.H * D;  // row stride in elements
  const char *Qp = (const char *)a.q + (((int64_t)b * a.Sq * a.H + h) * D) * 2;
  const char *Kp = (const char *)a.k + (((int64_t)b * a.Skv * a.H + h) * D) * 2;
  const char *Vp = (const char *)a.v + (((int64_t)b * a.Skv * a.H + h) * D) * 2;
  _Float16 *Op = (_Float16 *)a.o + ((int64_t)b * a.Sq * a.H + h) * D;
  const int n_tiles = a.Skv / BN;
  const float c_log2 = a.scale_log2;
  const uint32_t k_ld = (uint32_t)(ld * 2);  // global row pitch in bytes
  const bool want_taps = a.row_max != nullptr || a.row_sum != nullptr;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

  // ---- this wave's V tile in the LDS: the whole 64 x D tile is copied by the wave itself, 1 KB (RPI rows) per copy
  const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
  const uint32_t v_tile = lds_base + wave * C::V_TILE;
  uint32_t goff_v[C::V_IPW];
#pragma unroll
  for (int i = 0; i < C::V_IPW; ++i) {
    constexpr int CPR = C::V_PITCH / 16;
    const int row = i * C::V_RPI + lane / CPR;
    goff_v[i] = (uint32_t)row * k_ld + (uint32_t)(((lane % CPR) ^ swz_v16n<C::V_PITCH>(row)) * 16);
  }
  uint32_t v_rd[DB];
  {
    const int v_key = 4 * g + (c >> 2);
    const int cg = c & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_rd[db] = v_tile + v_key * C::V_PITCH + (((2 * db + (cg >> 1)) ^ swz_v16n<C::V_PITCH>(v_key)) * 16) + (cg & 1) * 8;
  }

  half8 qreg[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int s = 0; s < KS; ++s) qreg[qb][s] = *(const half8 *)(Qp + ((int64_t)(q0 + 16 * qb + c) * ld + 32 * s + 8 * g) * 2);

  f32x4 oacc[DB][QB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) oacc[db][qb] = zero4;
  float m_ref[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) m_ref[qb] = -INFINITY, l_run[qb] = 0.f;

  for (int j = wave; j < n_tiles; j += W) {
    const char *vt = Vp + (size_t)j * ((size_t)BN * k_ld);
#pragma unroll
    for (int i = 0; i < C::V_IPW; ++i) lds_dma16(vt, goff_v[i], v_tile, i * 1024);
    // S^T = K . Q^T, K fragments straight from global memory: lane (c, g) of key block kb, K-step s: K[16 kb + c][32 s + 8 g .. +8)
    const char *kt = Kp + (size_t)j * ((size_t)BN * k_ld) + (size_t)c * k_ld + 16 * g;
    f32x4 s_[KB][QB];
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const half8 ka = *(const half8 *)(kt + (size_t)(16 * kb) * k_ld + 64 * s);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          s_[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qreg[qb][s], s == 0 ? zero4 : s_[kb][qb], 0, 0, 0);
      }
    // online softmax, reference point = running max (online_softmax.h:123-165); weights summed in fp32 before the cast
    // (online_softmax.h:173-206)
    half8 pb[QB][PS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx = s_[0][qb][0];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int t = 0; t < 4; ++t) mx = __builtin_fmaxf(mx, s_[kb][qb][t]);
      const float m_new = fmaxf(m_ref[qb], quad_max(mx) * c_log2);
      const float alpha = __builtin_amdgcn_exp2f(m_ref[qb] - m_new);
      m_ref[qb] = m_new;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db][qb] *= alpha;
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s_[kb][qb][t], c_log2, -m_new));
          rs += p;
          pb[qb][kb / 2][4 * (kb % 2) + t] = (_Float16)p;
        }
      l_run[qb] = l_run[qb] * alpha + rs;
    }
    wait_lds_dma();  // this wave's V tile has landed (nobody else reads it)
#pragma unroll
    for (int ps = 0; ps < PS; ++ps)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const uint32_t vp = v_rd[db] + ps * 32 * C::V_PITCH;
        union {
          struct { short4v lo, hi; } s2;
          half8 h;
        } va;
        va.s2.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(short4v, vp));
        va.s2.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(short4v, vp + 16 * C::V_PITCH));
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) oacc[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va.h, pb[qb][ps], oacc[db][qb], 0, 0, 0);
      }
    // the next turn's copy overwrites the tile: its transposing reads must have returned before that copy is issued
    // (the compiler may sink the MFMAs that consume them, and with them its own wait, below the copy's asm statement)
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  }

  // ---- the partial results meet: wave u leaves O_u (fp32, in its own tile region: lane-major, 16 bytes per lane and
  // block) and per query its reference point m_u and row sum l_u; a wave without tiles leaves m = -inf, l = 0, O = 0
  {
    f32x4 *op = (f32x4 *)(smem + wave * C::V_TILE);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) op[(db * QB + qb) * 64 + lane] = oacc[db][qb];
    float *st = (float *)(smem + kStats);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float l_tot = quad_sum(l_run[qb]);
      if (g == 0) {
        st[wave * 32 + 16 * qb + c] = m_ref[qb];
        st[(W + wave) * 32 + 16 * qb + c] = l_tot;
      }
    }
  }
  __syncthreads();
  // unit (db, qb) of the output goes to wave (db * QB + qb) % W
  const float *st = (const float *)(smem + kStats);
  for (int unit = wave; unit < DB * QB; unit += W) {
    const int db = unit / QB, qb = unit % QB;
    float m_all = -INFINITY;
#pragma unroll
    for (int u = 0; u < W; ++u) m_all = fmaxf(m_all, st[u * 32 + 16 * qb + c]);
    float l_all = 0.f;
    f32x4 o_all = zero4;
#pragma unroll
    for (int u = 0; u < W; ++u) {
      const float m_u = st[u * 32 + 16 * qb + c];
      const float w_u = m_u == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_u - m_all);
      l_all += st[(W + u) * 32 + 16 * qb + c] * w_u;
      o_all += ((const f32x4 *)(smem + u * C::V_TILE))[unit * 64 + lane] * w_u;
    }
    const float inv = a.out_scale / l_all;
    half4 o4;
#pragma unroll
    for (int t = 0; t < 4; ++t) o4[t] = (_Float16)(o_all[t] * inv);
    *(half4 *)(Op + (int64_t)(q0 + 16 * qb + c) * ld + 16 * db + 4 * g) = o4;
    if (want_taps && db == 0 && g == 0) {
      // the reference point follows the running max in every wave: the merged one is the true row max
      const int64_t si = ((int64_t)b * a.H + h) * a.Sq + q0 + 16 * qb + c;
      if (a.row_max) a.row_max[si] = m_all;
      if (a.row_sum) a.row_sum[si] = l_all;
    }
  }
}

}  // namespace cfk
