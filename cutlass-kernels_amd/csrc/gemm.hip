// Dense (batched) GEMM D = alpha * A.B + beta * C with fp32 accumulation and an fp32 epilogue, D row-major M x N, for
// fp16 operands (v_mfma_f32_32x32x16_f16) and fp32 operands (v_mfma_f32_32x32x2_f32) -- gfx950 only.
//
// Secondary bench on the FMHA tile engine: the same LDS-DMA staging with XOR-swizzled rows and 32x32 MFMA tiles.
// Takes the place of gemm_device/gemm of the reference's CuTe example (src/cute-gemm-tma-gma/gemm.cu:57-463: TMA load
// of one A and one B tile, one synchronous WGMMA batch per K-tile, no pipelining; its type 1 is float, type 3 half,
// :677-684; batch count L with packed strides, :519-521) and of the CUTLASS-API example with its alpha / beta
// epilogue (src/cutlass-gemm/gemm.cu:87-140, 318-324).  Layouts: TN = A is M x K and B is N x K, both K-contiguous
// (the reference's form, :362-380); NN (fp16 only) = B is K x N, N-contiguous (the literal C = A.B), whose B operand is
// read with ds_read_b64_tr_b16 exactly as V is in the attention kernel.  The reference writes C column-major
// (:386-389); C and D are row-major here.  gfx950 has no tf32/xf32 MFMA: fp32 operands multiply in full fp32.
//
// Workgroup = 4 waves (one per SIMD) on a 256 x 256 macro tile; wave (wm, wn) of a 2 x 2 grid owns 128 x 128 of C as
// 4 x 4 MFMA blocks, its 256 accumulator registers in the AGPR half of the register file.  K tiles are 32 deep and go
// through a ring of four LDS stages (32 KB each: A 16 KB + B 16 KB): the copy of tile kt+3 is issued, one 1 KB piece
// after every four MFMAs, while tile kt multiplies.  Measured on MI355X, M=N=K=8192: the spread-out copies are worth
// +15 % when the operands are constant (1.50 PFLOP/s; copies issued back to back fill the memory pipeline's queue and
// stall the wave, and with one wave per SIMD the MFMA pipe with it); with U(-1,1) operands the board is power-limited
// and every variant lands at 1.10-1.16 PFLOP/s.  The MFMA computes the TRANSPOSED block (rows = n, columns = m) so
// that a lane ends up with 4 consecutive n of one row m: 8-byte row-major stores.
#include <type_traits>

#include <mutex>

#include "fmha_common.h"

namespace cfk {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256;

// K-contiguous rows of PITCH bytes (128: two rows per 256-byte bank period; 64: four): 16 consecutive rows at one
// 16-byte chunk index must spread over all banks -> rows at the same place in the period get distinct XOR values
template <int PITCH>
__device__ __forceinline__ int swz_k(int row) { return PITCH == 128 ? (row >> 1) & 7 : (row >> 2) & 3; }
// 512-byte rows read with ds_read_b64_tr_b16 (4 consecutive k x 64 contiguous bytes)
__device__ __forceinline__ int swz512(int row) { return (row & 3) << 2; }

// WN = waves along n (2 along m always): 2 -> 4 waves of 128 x 128, one per SIMD (the shipped shape; a third less
// LDS traffic per MFMA than 4 -> 8 waves of 128 x 64, two per SIMD).
// T = element type of A, B, C, D (_Float16 or float); BKB = bytes of a K-contiguous tile row (32 halves or 16
// floats at 64), NS = LDS stages (copies run NS-1 tiles ahead of the multiply).  blockIdx.y = problem of a batch.
template <class T, bool NN, int WN, int BKB, int NS>
__global__ void __launch_bounds__(2 * WN * 64) __attribute__((amdgpu_waves_per_eu(WN / 2, WN / 2)))
gemm_kernel(const T *__restrict__ A, const T *__restrict__ B, const T *__restrict__ Cin, T *__restrict__ D, int M, int N,
            int K, float alpha, float beta) {
  constexpr bool F32 = sizeof(T) == 4;
  constexpr int ES = sizeof(T);
  constexpr int BK = BKB / ES;
  static_assert(!(F32 && NN), "the N-contiguous B layout is built for fp16 only");
  using Frag = std::conditional_t<F32, f32x4, half8>;  // 16 bytes of a row: the operand of one K-step
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  constexpr int NWAVES = 2 * WN;
  constexpr int NB = BN / WN / 32;     // 32-column blocks per wave
  constexpr int PITCH = BKB;           // bytes per K-contiguous LDS row
  constexpr int A_TILE = BM * PITCH;   // TN: B tile likewise (n rows); NN: BK rows (k) of 512 B
  constexpr int STAGE = 2 * A_TILE;
  constexpr int CPW = A_TILE / 1024 / NWAVES;  // 1 KB copies per wave and operand tile
  constexpr int RPC = 1024 / PITCH;    // rows per copy
  constexpr int KS = PITCH / 32;       // K-steps per tile: 32 bytes of a row (one 16-byte fragment per lane half) each
  const int wm = wave / WN, wn = wave % WN;

  // tile order: groups of 8 tile rows, column-major inside a group, so concurrently running workgroups share A and
  // B panels in L2; workgroup ids are first remapped so that each XCD owns a contiguous range of that order
  const int tiles_n = N / BN, tiles_m = M / BM;
  int t = xcd_remap(blockIdx.x, gridDim.x);
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int grp = t / per_group;
  const int first_m = grp * GROUP;
  const int rows_in_group = tiles_m - first_m < GROUP ? tiles_m - first_m : GROUP;
  const int in_grp = t - grp * per_group;
  const int tm = first_m + in_grp % rows_in_group;
  const int tn = in_grp / rows_in_group;
  const int m0 = tm * BM, n0 = tn * BN;

  const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
  const int64_t batch = blockIdx.y;  // packed strides M*K, N*K, M*N (reference: gemm.cu:519-521)
  A += batch * M * K;
  B += batch * N * K;
  D += batch * M * N;
  if (Cin) Cin += batch * M * N;
  const char *Ap = (const char *)(A + (int64_t)m0 * K);
  const char *Bp = NN ? (const char *)(B + n0) : (const char *)(B + (int64_t)n0 * K);

  // ---- global -> LDS copies, 16 B per lane, 1 KB per wave-wide copy
  // A (and B in TN): 8 rows of 128 B per copy; 32 copies per tile, 4 per wave.
  uint32_t goff_a[CPW], goff_b[CPW];
#pragma unroll
  for (int i = 0; i < CPW; ++i) {
    const int row = (i * NWAVES + wave) * RPC + lane / (PITCH / 16);
    const int cp = lane % (PITCH / 16);
    goff_a[i] = (uint32_t)row * (uint32_t)(K * ES) + (uint32_t)((cp ^ swz_k<PITCH>(row)) * 16);
    if (!NN) {
      goff_b[i] = goff_a[i];
    } else {  // B tile is BK rows (k) of 512 B (256 n): 2 rows per copy
      const int krow = (i * NWAVES + wave) * 2 + (lane >> 5);
      const int cpb = lane & 31;
      goff_b[i] = (uint32_t)krow * (uint32_t)(N * 2) + (uint32_t)((cpb ^ swz512(krow)) * 16);
    }
  }
  auto load_stage = [&](int kt, int stage) {
    const char *ga = Ap + (size_t)kt * PITCH;
    const char *gb = NN ? Bp + (size_t)kt * BK * (size_t)(N * 2) : Bp + (size_t)kt * PITCH;
#pragma unroll
    for (int i = 0; i < CPW; ++i) lds_dma16(ga + goff_a[i], lds_base + stage * STAGE + (i * NWAVES + wave) * 1024);
#pragma unroll
    for (int i = 0; i < CPW; ++i) lds_dma16(gb + goff_b[i], lds_base + stage * STAGE + A_TILE + (i * NWAVES + wave) * 1024);
  };

  // ---- LDS read addresses.  K-step s: lane (r, g) needs bytes 32s + 16g .. +16 of its row (fp16: k = 16s + 8g .. +8;
  // fp32: k = 8s + 4g .. +4, used one element per 32x32x2 MFMA: which contraction slot means which k is free as long
  // as A and B agree).
  int a_rd[KS], b_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    a_rd[s] = (wm * 128 + r) * PITCH + (((2 * s + g) ^ swz_k<PITCH>(r)) * 16);               // + 32 rows per m block
    b_rd[s] = A_TILE + (wn * NB * 32 + r) * PITCH + (((2 * s + g) ^ swz_k<PITCH>(r)) * 16);  // + 32 rows per n block (TN)
  }
  // NN: B^T operand via ds_read_b64_tr_b16 from [k][n] rows (see the V operand of the attention kernel)
  const int li = lane & 15;
  const int bk_row = 8 * g + (li >> 2);                                // + 16 s + 4 h2: slot t of lane g is k = 16s + 8g + t, as in A
  const int bn_col = wn * NB * 32 + 16 * ((lane >> 4) & 1) + 4 * (li & 3);  // + 32 nb
  int bt_rd[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int c = (bn_col + 32 * nb) >> 3;
    bt_rd[nb] = A_TILE + bk_row * 512 + ((c ^ swz512(bk_row)) * 16) + (bn_col & 7) * 2;
  }

  f32x16 acc[4][NB];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mb][nb][v] = 0.f;

  const int k_tiles = K / BK;
  // operand fetch for K-step s of the tile in LDS stage `st`
  auto fetch = [&](const char *st, int s, Frag (&aop)[4], Frag (&bop)[NB]) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if (!NN) {
        bop[nb] = *(const Frag *)(st + b_rd[s] + nb * 32 * PITCH);
      } else {
        if constexpr (!F32) {
          union {
            struct { short4v lo, hi; } p;
            half8 h;
          } u;
          const char *bp = st + bt_rd[nb] + s * 16 * 512;
          u.p.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, bp));
          u.p.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, bp + 4 * 512));
          bop[nb] = u.h;
        }
      }
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) aop[mb] = *(const Frag *)(st + a_rd[s] + mb * 32 * PITCH);
  };
  // One copy (index c of the 2*CPW a wave issues per tile: first the A ones, then the B ones) of the tile at
  // ga / gb into stage `fill`
  auto load_copy = [&](const char *ga, const char *gb, int fill, int c) {
    if (c < CPW) lds_dma16(ga + goff_a[c], lds_base + fill * STAGE + (c * NWAVES + wave) * 1024);
    else lds_dma16(gb + goff_b[c - CPW], lds_base + fill * STAGE + A_TILE + ((c - CPW) * NWAVES + wave) * 1024);
  };
  // The multiplies of one K-step, with the copies [c0, c1) of the tile being prefetched spread between them: the
  // L1 takes a 1 KB copy apart into sixteen 64-byte accesses, so copies issued back to back fill the memory
  // pipeline's queue and stall the wave (and with it the MFMA pipe) at the next one.
  auto mma = [&](const Frag (&aop)[4], const Frag (&bop)[NB], const char *ga, const char *gb, int fill, int c0, int c1) {
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {  // transposed block: MFMA rows = n (B operand first), columns = m
        if constexpr (F32) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(bop[nb][e], aop[mb][e], acc[mb][nb], 0, 0, 0);
        } else {
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bop[nb], aop[mb], acc[mb][nb], 0, 0, 0);
        }
      }
#pragma unroll
      for (int c = c0 + mb; c < c1; c += 4) load_copy(ga, gb, fill, c);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Copies per wave and tile, and how they spread over the K-steps of the tile that is multiplied meanwhile.  With
  // two stages the tile being copied is needed right after this tile's barrier, so its copies go with the first KS-1
  // steps; with more stages they go with all KS steps and the wait leaves the younger tiles in flight.
  constexpr int CPT = 2 * CPW;
  constexpr int PER_STEP = NS == 2 ? (CPT + KS - 2) / (KS - 1) : CPT / KS;
  constexpr int IN_FLIGHT = NS == 2 ? 0 : (NS - 3) * CPT + (KS - 1) * PER_STEP;
  auto wait_tile = [&]() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT) : "memory"); };
#pragma unroll
  for (int t0 = 0; t0 < NS - 1; ++t0) load_stage(t0 < k_tiles ? t0 : k_tiles - 1, t0);
  wait_lds_dma();
  __syncthreads();
  Frag aop[2][4], bop[2][NB];  // two operand register sets: K-step s+1 is fetched while K-step s multiplies
  fetch(smem, 0, aop[0], bop[0]);
  int stage = 0;
  for (int kt = 0; kt < k_tiles; ++kt) {
    // the stage the previous tile was read from (its last reads were issued before that tile's barrier) is refilled
    // with tile kt+NS-1 (clamped at the end: a surplus copy rewrites a stage nobody reads any more)
    const int fill = stage == 0 ? NS - 1 : stage - 1;
    const int ld_t = kt + NS - 1 < k_tiles ? kt + NS - 1 : k_tiles - 1;
    const char *ga = Ap + (size_t)ld_t * PITCH;
    const char *gb = NN ? Bp + (size_t)ld_t * BK * (size_t)(N * 2) : Bp + (size_t)ld_t * PITCH;
    const char *st = smem + stage * STAGE;
    const int nstage = stage + 1 == NS ? 0 : stage + 1;
    // sched_barrier(0): the compiler's scheduler would otherwise sink each fetch down to its first use and expose
    // the LDS latency in front of every multiply
#pragma unroll
    for (int s2 = 0; s2 + 1 < KS; ++s2) {
      fetch(st, s2 + 1, aop[(s2 + 1) & 1], bop[(s2 + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      mma(aop[s2 & 1], bop[s2 & 1], ga, gb, fill, s2 * PER_STEP, (s2 + 1) * PER_STEP < CPT ? (s2 + 1) * PER_STEP : CPT);
    }
    wait_tile();
    __syncthreads();  // the next tile has landed for everybody
    // first K-step of the next tile is fetched before the last multiply of this one
    fetch(smem + nstage * STAGE, 0, aop[0], bop[0]);
    __builtin_amdgcn_sched_barrier(0);
    mma(aop[(KS - 1) & 1], bop[(KS - 1) & 1], ga, gb, fill, NS == 2 ? CPT : (KS - 1) * PER_STEP, CPT);
    stage = nstage;
  }
  wait_lds_dma();  // no copy may still be writing LDS when the workgroup retires

  // ---- epilogue: D = alpha * acc + beta * C in fp32 (src/cutlass-gemm/gemm.cu:318-324); lane (m = r, g) holds
  // n = 8i + 4g + j of each block: 4 consecutive elements of a row per access
  using Out4 = std::conditional_t<F32, f32x4, half4>;
  const bool with_c = Cin != nullptr && beta != 0.f;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    const int64_t row_off = (int64_t)(m0 + wm * 128 + mb * 32 + r) * N + n0 + wn * NB * 32;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t off = row_off + nb * 32 + 8 * i + 4 * g;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = alpha * acc[mb][nb][4 * i + j];
        if (with_c) {
          const Out4 c4 = *(const Out4 *)(Cin + off);
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] += beta * (float)c4[j];
        }
        Out4 o4;
#pragma unroll
        for (int j = 0; j < 4; ++j) o4[j] = (T)v[j];
        *(Out4 *)(D + off) = o4;
      }
  }
}

template <class T, bool NN>
struct GemmLaunch {
  static constexpr int WN = 2, BKB = 64, NS = 4;
  static constexpr int LDS_BYTES = NS * 2 * BM * BKB;
  static constexpr auto kern = gemm_kernel<T, NN, WN, BKB, NS>;
  // one-time set-up, thread-safe and callable ahead of any launch
  static hipError_t prepare() {
    static std::once_flag once;
    static hipError_t status = hipSuccess;
    std::call_once(once, [] {
      status = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    });
    return status;
  }
  static hipError_t launch(const GemmArgs &g, hipStream_t s) {
    const hipError_t e = prepare();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((g.M / BM) * (g.N / BN), g.batch), dim3(2 * WN * 64), LDS_BYTES, s, (const T *)g.A,
                       (const T *)g.B, (const T *)g.C, (T *)g.D, g.M, g.N, g.K, g.alpha, g.beta);
    return hipGetLastError();
  }
};

}  // namespace

hipError_t launch_gemm(const GemmArgs &g, hipStream_t s) {
  if (g.f32) return g.layout == 0 ? GemmLaunch<float, false>::launch(g, s) : hipErrorNotSupported;
  return g.layout == 0 ? GemmLaunch<_Float16, false>::launch(g, s) : GemmLaunch<_Float16, true>::launch(g, s);
}

hipError_t prepare_gemm() {
  hipError_t e = GemmLaunch<float, false>::prepare();
  if (e == hipSuccess) e = GemmLaunch<_Float16, false>::prepare();
  if (e == hipSuccess) e = GemmLaunch<_Float16, true>::prepare();
  return e;
}

}  // namespace cfk
