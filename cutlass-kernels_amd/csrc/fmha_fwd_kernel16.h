// The fp16 FMHA forward kernel on 16x16x32 MFMAs (v_mfma_f32_16x16x32_f16).  Same algorithm, LDS staging, pipeline
// (one or two key tiles per barrier) and epilogue as fmha_fwd_kernel.h, which it takes its configuration struct and
// host-side plumbing from; what differs is the MFMA shape, with it every register layout, and how the softmax notices
// that its reference point has to move: not by a row max per tile but by the row sum it needs anyway (softmax_tile
// below; 22 VALU instructions per wave and tile less, +3..6 % on N(0,1) data, results bit-identical).
//
// Why a second shape: on N(0,1) data this board is power-limited, and a register-only loop of 16x16x32 MFMAs sustains
// 1.89-1.90 PFLOP/s there against 1.69 for 32x32x16 (2.39 against 2.47 on constant operands): a multiply that is
// twice as deep per accumulator element moves half the accumulator bits per FLOP.  Measured on N(0,1) tensors against
// the 32x32 kernel, both with a row max per tile: B=8 H=16 S=2048 D=128 1107 against 1078 TFLOP/s, B=4 H=32 S=4096 D=64
// 919 against 875; on constant tensors, where nothing limits the clock, the 32x32 kernel is the faster one (1480
// against 1244): twice the MFMA instructions for the same VALU work leave fewer issue slots.  Head dim 256 gains
// nothing (929 against 932) and keeps the 32x32 kernel.
//
// Layouts (lane = 16 g + c, c = 0..15, g = 0..3):
//   A operand: row c of the 16-row block, contraction slots 8g .. 8g+7;   B operand: column c, slots 8g .. 8g+7;
//   accumulator: column c, rows 4g .. 4g+3.
// A wave still owns 32 query rows, as two 16-query blocks qb.  Both GEMMs run transposed:
//   S^T[key, q]  = K[key, :] . Q[q, :]       A = K fragment from LDS (one ds_read_b128 feeds both query blocks),
//                                            B = Q resident in VGPRs (slots = 8 consecutive d)
//   O^T[d, q]   += V^T[d, key] . P^T[key, q]  A = V read transposed from LDS (two ds_read_b64_tr_b16 feed both query
//                                            blocks), B = P straight from the S^T accumulators
// so lane (c, g) holds, of query 16 qb + c, keys 16 kb + 4g .. +3 of every 16-key block kb: a row max / row sum is an
// in-lane reduction plus an exchange among the four lanes c, c+16, c+32, c+48.  Two key blocks 2 ps, 2 ps + 1 make the
// eight contraction slots of K-step ps of the second GEMM: slot t of lane g is key 32 ps + 16 (t / 4) + 4 g + t % 4,
// and the V^T operand is fetched with that same key order (first transpose read at keys 4g .. 4g+3, second 16 further).
#pragma once
#include "fmha_fwd_kernel.h"

namespace cfk {

// fp16 V read by ds_read_b64_tr_b16 in this layout: a 32-lane half of the wave touches 8 consecutive keys x 32
// contiguous bytes (one 16-column block), which must spread over the 256-byte bank period; bit 0 stays clear so the
// 32 bytes stay contiguous.
// K rows read by ds_read_b128 with lane (c, g) at row c, chunk 4s+g: XOR with the row number itself is conflict-free
// here (measured; the swizzle of the 32x32 lane map costs 1.6 x the LDS cycles with this one).
template <int PITCH>
__device__ __forceinline__ int swz_k16n(int row) {
  return row & (PITCH / 16 - 1) & 15;
}
template <int PITCH>
__device__ __forceinline__ int swz_v16n(int row) {
  if (PITCH == 128) return ((row >> 1) & 3) << 1;
  return (row & 7) << 1;
}

template <class C>
__global__ void __launch_bounds__(C::T) __attribute__((amdgpu_waves_per_eu(C::WPE, C::WPE)))
fmha_fwd_kernel16(const FmhaArgs a) {
  static_assert(!C::QK8 && !C::PV8 && !C::VT && !C::TAP_S, "fp16 operands only, no score tap");
  constexpr int D = C::D, BN = C::BN;
  constexpr int QB = 2;        // 16-query blocks per wave
  constexpr int KB = BN / 16;  // 16-key blocks per tile (M blocks of S^T)
  constexpr int KS = D / 32;   // K-steps of S^T
  constexpr int DB = D / 16;   // 16-row blocks of O^T
  constexpr int PS = BN / 32;  // K-steps of O^T
  const float kTau = a.tau;    // deferred-rescale threshold above the running max (log2 domain)
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;

  const int q_blocks = a.Sq / C::BM;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / q_blocks;
  const int qblk = tile - bh * q_blocks;
  const int b = bh / a.H, h = bh - b * a.H;
  const int64_t ld = (int64_t)a.H * D;  // row stride in elements
  const char *Qp = (const char *)a.q + (((int64_t)b * a.Sq * a.H + h) * D) * 2;
  const char *Kp = (const char *)a.k + (((int64_t)b * a.Skv * a.H + h) * D) * 2;
  const char *Vp = (const char *)a.v + (((int64_t)b * a.Skv * a.H + h) * D) * 2;
  _Float16 *Op = (_Float16 *)a.o + ((int64_t)b * a.Sq * a.H + h) * D;
  const int q0 = qblk * C::BM + wave * 32;
  const int n_tiles = a.Skv / BN;
  const float c_log2 = a.scale_log2;
  const uint32_t k_ld = (uint32_t)(ld * 2), v_ld = k_ld;  // global row pitch in bytes

  // ---- global -> LDS copies, as in fmha_fwd_kernel.h: copy i of wave w covers tile rows (i*NWAVES + w)*RPI .. +RPI;
  // lane l writes LDS slot (row l / CPR, chunk position l % CPR) and fetches chunk position ^ swz(row) of that row.
  uint32_t goff_k[C::K_IPW], goff_v[C::V_IPW];
#pragma unroll
  for (int i = 0; i < C::K_IPW; ++i) {
    constexpr int CPR = C::K_PITCH / 16;
    const int row = (i * C::NWAVES + wave) * C::K_RPI + lane / CPR;
    goff_k[i] = (uint32_t)row * k_ld + (uint32_t)(((lane % CPR) ^ swz_k16n<C::K_PITCH>(row)) * 16);
  }
#pragma unroll
  for (int i = 0; i < C::V_IPW; ++i) {
    constexpr int CPR = C::V_PITCH / 16;
    const int row = (i * C::NWAVES + wave) * C::V_RPI + lane / CPR;
    goff_v[i] = (uint32_t)row * v_ld + (uint32_t)(((lane % CPR) ^ swz_v16n<C::V_PITCH>(row)) * 16);
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
    const char *gt = Vp + (size_t)jt * ((size_t)BN * v_ld);
#pragma unroll
    for (int i = 0; i < C::V_IPW; ++i)
      lds_dma16(gt, goff_v[i], lds_wave, C::V_ST0 + stage * C::V_TILE + i * C::NWAVES * 1024);
  };

  // ---- Q: B operand of S^T, resident in VGPRs: lane (c, g), query block qb, K-step s holds Q[q0+16qb+c][32s+8g .. +8)
  half8 qreg[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb)
#pragma unroll
    for (int s = 0; s < KS; ++s) qreg[qb][s] = *(const half8 *)(Qp + ((int64_t)(q0 + 16 * qb + c) * ld + 32 * s + 8 * g) * 2);

  // ---- per-lane LDS read addresses (absolute LDS byte addresses of slot 0; slots and blocks are immediates: the
  // swizzles only depend on the row within its 16- or 8-row group)
  uint32_t k_rd[KS];  // K operand, K-step s: row c (+16 kb), chunk 4s+g
#pragma unroll
  for (int s = 0; s < KS; ++s) k_rd[s] = lds_base + C::K_ST0 + c * C::K_PITCH + (((4 * s + g) ^ swz_k16n<C::K_PITCH>(c)) * 16);
  // V operand: within its block of 16 lanes, lane L hands the transpose read the address of (key L/4, columns
  // 4(L%4) .. +3) and receives keys 0..3 of column L; the block g reads keys 4g .. 4g+3 (+16 for the second read)
  uint32_t v_rd[DB];
  {
    const int v_key = 4 * g + (c >> 2);
    const int cg = c & 3;  // 4-column group inside the 16-column block: chunk cg/2, 8 bytes into it for odd cg
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_rd[db] = lds_base + C::V_ST0 + v_key * C::V_PITCH + (((2 * db + (cg >> 1)) ^ swz_v16n<C::V_PITCH>(v_key)) * 16) + (cg & 1) * 8;
  }

  f32x4 oacc[DB][QB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) oacc[db][qb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // per query block: softmax reference point (log2 domain); this lane's running max of the raw scores (a quarter of
  // the query's keys), kept for the taps only
  float m_ref[QB], m_lane[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) m_ref[qb] = -INFINITY, m_lane[qb] = -INFINITY;
  // Row sum: v_dot2_f32_f16 over this lane's quarter of each query's keys, of P as rounded to fp16 (the weights the
  // second GEMM applies), in fp32; the four quarters meet in the epilogue.
  float l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) l_run[qb] = 0.f;

  static_assert(C::KPRE == 0, "no K fragment prefetch in this kernel");
  const float sum_cap = __builtin_amdgcn_exp2f(kTau);
  const bool want_taps = a.row_max != nullptr || a.row_sum != nullptr;
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  // S^T = K . Q^T for the K tile in LDS slot `stage`
  auto qk = [&](int stage, f32x4 (&sacc)[KB][QB]) __attribute__((always_inline)) {
    const uint32_t kt = stage * C::K_TILE;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const half8 ka = *LDS_AT(half8, kt + k_rd[s] + kb * 16 * C::K_PITCH);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          sacc[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qreg[qb][s], s == 0 ? zero4 : sacc[kb][qb], 0, 0, 0);
      }
  };
  // this lane's max over its quarter of the keys of query block qb: a chain of three-operand maxima
  auto lane_max = [&](const f32x4 (&sacc)[KB][QB], int qb) __attribute__((always_inline)) -> float {
    float mx = __builtin_fmaxf(sacc[0][qb][0], sacc[0][qb][1]);
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int t = kb ? 0 : 2; t < 4; t += 2) mx = __builtin_fmaxf(__builtin_fmaxf(mx, sacc[kb][qb][t]), sacc[kb][qb][t + 1]);
    return mx;
  };
  // Move the reference point of every query up to the row max of `sacc` (if that is above it) and re-base O and l
  // (online_softmax.h:123-165); for the first tile the old reference point is -inf and O and l are zero.
  auto rebase = [&](const f32x4 (&sacc)[KB][QB]) __attribute__((always_inline)) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float mx = lane_max(sacc, qb);
      float mfull = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mfull = fmaxf(mfull, __shfl_xor(mfull, 32, 64));
      const float m_new = fmaxf(m_ref[qb], mfull * c_log2);
      const float alpha = __builtin_amdgcn_exp2f(m_ref[qb] - m_new);
      m_ref[qb] = m_new;
      l_run[qb] *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db][qb] *= alpha;
    }
  };
  // P = exp2(c*S - m_ref), cast to fp16 in the B-operand register order of the second GEMM, and the tile's row sums of
  // P as rounded (the weights the second GEMM applies), in fp32
  auto exp_and_sum = [&](const f32x4 (&sacc)[KB][QB], half8 (&pb)[QB][PS], float (&rsum)[QB]) __attribute__((always_inline)) {
    const half2v one2 = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          pb[qb][kb / 2][4 * (kb % 2) + t] = (_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][qb][t], c_log2, -m_ref[qb]));
      float rs = 0.f, rs2 = 0.f;
#pragma unroll
      for (int ps = 0; ps < PS; ++ps)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const half2v pp = {pb[qb][ps][2 * t], pb[qb][ps][2 * t + 1]};
          if (t & 1) rs2 = __builtin_amdgcn_fdot2(pp, one2, rs2, false);
          else rs = __builtin_amdgcn_fdot2(pp, one2, rs, false);
        }
      rsum[qb] = rs + rs2;
    }
  };
  // The softmax of key tile jt.  No row max is taken in the common case: a weight that leaves the fp16 range (or
  // merely exceeds 2^tau) shows in the row sum, which is needed anyway.  An infinite or large sum sends the wave to
  // the (wave-uniform, rare) slow path: the scores are gone by then (the exponentials overwrote them; keeping them
  // would cost 32 registers), so it recomputes them with K fragments fetched straight from global memory, moves the
  // reference point up to their row max and takes the exponentials again.
  auto softmax_tile = [&](int jt, const f32x4 (&sacc)[KB][QB], half8 (&pb)[QB][PS]) __attribute__((always_inline)) {
    if (want_taps) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) m_lane[qb] = __builtin_fmaxf(m_lane[qb], lane_max(sacc, qb));
    }
    float rsum[QB];
    exp_and_sum(sacc, pb, rsum);
    bool over = false;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) over = over || !(rsum[qb] < sum_cap);
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(over) != 0, 0)) {
      f32x4 sr[KB][QB];
      // (the empty statement keeps the address arithmetic of this path inside it: hoisted out of the loop it would
      // occupy ten registers for all of the kernel)
      int cc = c, gg = g;
      asm volatile("" : "+v"(cc), "+v"(gg));
      const char *kt = Kp + (size_t)jt * ((size_t)BN * k_ld) + (size_t)cc * k_ld + 16 * gg;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          const half8 ka = *(const half8 *)(kt + (size_t)(16 * kb) * k_ld + 64 * s);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb)
            sr[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qreg[qb][s], s == 0 ? zero4 : sr[kb][qb], 0, 0, 0);
        }
      rebase(sr);
      exp_and_sum(sr, pb, rsum);
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) l_run[qb] += rsum[qb];
  };
  // O^T += V^T . P^T for the V tile at LDS byte offset vt
  auto pv = [&](uint32_t vt, const half8 (&pb)[QB][PS]) __attribute__((always_inline)) {
#pragma unroll
    for (int ps = 0; ps < PS; ++ps)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const uint32_t vp = vt + v_rd[db] + ps * 32 * C::V_PITCH;
        union {
          struct { short4v lo, hi; } s;
          half8 h;
        } va;
        va.s.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(short4v, vp));
        va.s.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_AT(short4v, vp + 16 * C::V_PITCH));
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) oacc[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va.h, pb[qb][ps], oacc[db][qb], 0, 0, 0);
      }
  };

  // One pipeline step for tile j (parity P = j & 1), as in fmha_fwd_kernel.h: on entry s_cur = S_j is finished, K_{j+1}
  // sits in K stage P^1 and V_j in V stage P.
  auto step = [&](auto parity, auto has_next, int j, f32x4 (&s_cur)[KB][QB], f32x4 (&s_nxt)[KB][QB]) __attribute__((always_inline)) {
    constexpr int P = decltype(parity)::value;
    constexpr bool HAS_NEXT = decltype(has_next)::value;
    load_k(j + 2 < n_tiles ? j + 2 : n_tiles - 1, P);
    load_v(j + 1 < n_tiles ? j + 1 : n_tiles - 1, P ^ 1);
    half8 pb[QB][PS];
    if (HAS_NEXT) qk(P ^ 1, s_nxt);
    softmax_tile(j, s_cur, pb);
    pv(P * C::V_TILE, pb);
    wait_lds_dma();
    __syncthreads();
  };

  // Two key tiles per barrier (SUB = 2), slot bookkeeping as in fmha_fwd_kernel.h: tile t of K and of V lives in slot
  // t % 4; step J covers tiles 2J and 2J+1 and refills the slots last read by step J-1.
  auto step2 = [&](auto parity, auto last, int J, f32x4 (&s_a)[KB][QB], f32x4 (&s_b)[KB][QB]) __attribute__((always_inline)) {
    constexpr int P = decltype(parity)::value;
    constexpr bool LAST = decltype(last)::value;
    const int t0 = 2 * J, t_max = n_tiles - 1;
    load_k(t0 + 3 < t_max ? t0 + 3 : t_max, (2 * P + 3) % 4);
    load_k(t0 + 4 < t_max ? t0 + 4 : t_max, (2 * P) % 4);
    {
      half8 pb[QB][PS];
      qk((2 * P + 1) % 4, s_b);
      softmax_tile(t0, s_a, pb);
      pv(((2 * P) % 4) * C::V_TILE, pb);
    }
    load_v(t0 + 2 < t_max ? t0 + 2 : t_max, (2 * P + 2) % 4);
    load_v(t0 + 3 < t_max ? t0 + 3 : t_max, (2 * P + 3) % 4);
    {
      half8 pb[QB][PS];
      if (!LAST) qk((2 * P + 2) % 4, s_a);
      softmax_tile(t0 + 1, s_b, pb);
      pv(((2 * P + 1) % 4) * C::V_TILE, pb);
    }
    wait_lds_dma();
    __syncthreads();
  };

  using std::integral_constant;
  f32x4 s_a[KB][QB], s_b[KB][QB];
  if constexpr (C::SUB == 2) {
    const int t_max = n_tiles - 1;
    load_k(0, 0);
    load_v(0, 0);
    load_k(1, 1);
    load_k(2 < t_max ? 2 : t_max, 2);
    load_v(1, 1);
    wait_lds_dma();
    __syncthreads();
    qk(0, s_a);
    rebase(s_a);
    __syncthreads();  // every wave is done with K slot 0 before step 0 overwrites it
    const int n_steps = n_tiles / 2;
    int J = 0;
    for (; J + 2 < n_steps; J += 2) {
      step2(integral_constant<int, 0>{}, integral_constant<bool, false>{}, J, s_a, s_b);
      step2(integral_constant<int, 1>{}, integral_constant<bool, false>{}, J + 1, s_a, s_b);
    }
    if (J + 2 == n_steps) {
      step2(integral_constant<int, 0>{}, integral_constant<bool, false>{}, J, s_a, s_b);
      step2(integral_constant<int, 1>{}, integral_constant<bool, true>{}, J + 1, s_a, s_b);
    } else {
      step2(integral_constant<int, 0>{}, integral_constant<bool, true>{}, J, s_a, s_b);
    }
  } else {
    load_k(0, 0);
    load_v(0, 0);
    load_k(n_tiles > 1 ? 1 : 0, 1);
    wait_lds_dma();
    __syncthreads();
    qk(0, s_a);
    rebase(s_a);
    __syncthreads();  // every wave is done with K stage 0 before step 0 overwrites it
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
  }

  // ---- epilogue: O = out_scale * O / l (online_softmax.h:59-85), fp16, [B,S,H,D].  A lane holds 4 consecutive d of
  // one query per block; the wave's 32 x D tile goes through its own LDS region (all staged tiles are dead after the
  // loop's last barrier) and leaves as whole rows, 16 bytes per lane.
  float l_tot[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    l_tot[qb] = l_run[qb] + __shfl_xor(l_run[qb], 16, 64);
    l_tot[qb] += __shfl_xor(l_tot[qb], 32, 64);
  }
  {
    char *ot = smem + wave * (32 * C::O_PITCH);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float inv = a.out_scale / l_tot[qb];
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        half4 o4;
#pragma unroll
        for (int t = 0; t < 4; ++t) o4[t] = (_Float16)(oacc[db][qb][t] * inv);
        *(half4 *)(ot + (16 * qb + c) * C::O_PITCH + (db * 16 + 4 * g) * 2) = o4;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    constexpr int LPR = D / 8;     // lanes per output row (16 bytes each)
    constexpr int RPP = 64 / LPR;  // rows per wave-wide store
    const int orow_l = lane / LPR, ochunk = lane % LPR;
#pragma unroll
    for (int pass = 0; pass < 32 / RPP; ++pass) {
      const int row = pass * RPP + orow_l;
      const int4v val = *(const int4v *)(ot + row * C::O_PITCH + ochunk * 16);
      *(int4v *)(Op + (int64_t)(q0 + row) * ld + ochunk * 8) = val;
    }
  }
  if (want_taps) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float m_true = fmaxf(m_lane[qb], __shfl_xor(m_lane[qb], 16, 64));
      m_true = fmaxf(m_true, __shfl_xor(m_true, 32, 64)) * c_log2;
      if (g == 0) {
        const int64_t si = ((int64_t)b * a.H + h) * a.Sq + q0 + 16 * qb + c;
        // taps are reported against the true row max, as the reference's miOut / sPrimeOut are (fmha_epilogue.h:7-46)
        if (a.row_max) a.row_max[si] = m_true;
        if (a.row_sum) a.row_sum[si] = l_tot[qb] * __builtin_amdgcn_exp2f(m_ref[qb] - m_true);
      }
    }
  }
}

}  // namespace cfk
