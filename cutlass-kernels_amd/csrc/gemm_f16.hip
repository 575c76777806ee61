// Dense GEMM C = A.B, fp16 operands, fp32 accumulate, fp16 C (row-major M x N) -- gfx950 only.
//
// Secondary bench on the FMHA tile engine: the same LDS-DMA staging with XOR-swizzled rows, the same
// v_mfma_f32_32x32x16_f16 tiles.  Takes the place of gemm_device/gemm of the reference's CuTe example
// (src/cute-gemm-tma-gma/gemm.cu:57-463: TMA load of one A and one B tile, one synchronous WGMMA batch per K-tile,
// no pipelining).  Layouts: TN = A is M x K and B is N x K, both K-contiguous (the reference's form, :362-380);
// NN = B is K x N, N-contiguous (the literal C = A.B), whose B operand is read with ds_read_b64_tr_b16 exactly as V
// is in the attention kernel.  The reference writes C column-major (:386-389); C is row-major here.
//
// Workgroup = 8 waves on a 256 x 256 macro tile, BK = 64, two LDS stages (A 32 KB + B 32 KB each).  Wave (wm, wn)
// of a 2 x 4 grid owns 128 x 64 of C as 4 x 2 MFMA blocks.  The MFMA computes the TRANSPOSED block
// (rows = n, columns = m) so that a lane ends up with 4 consecutive n of one row m: 8-byte row-major stores.
#include <type_traits>

#include "fmha_common.h"

namespace cfk {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64, NWAVES = 8, T = NWAVES * 64;
constexpr int A_TILE = BM * BK * 2;            // 32 KB, rows of 128 B (K-contiguous)
constexpr int B_TILE = BN * BK * 2;            // 32 KB: TN rows of 128 B (n rows); NN rows of 512 B (k rows)
constexpr int STAGE = A_TILE + B_TILE;
constexpr int LDS_BYTES = 2 * STAGE;

// 128-byte rows (two rows per 256-byte bank period): 16 consecutive rows at one 16-byte chunk index must spread
// over all banks -> the 8 rows of equal parity get 8 distinct XOR values
__device__ __forceinline__ int swz128(int row) { return (row >> 1) & 7; }
// 512-byte rows read with ds_read_b64_tr_b16 (4 consecutive k x 64 contiguous bytes)
__device__ __forceinline__ int swz512(int row) { return (row & 3) << 2; }

template <bool NN>
__global__ void __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_f16_kernel(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, _Float16 *__restrict__ C, int M, int N,
                int K) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  const int wm = wave >> 2, wn = wave & 3;

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
  const char *Ap = (const char *)(A + (int64_t)m0 * K);
  const char *Bp = NN ? (const char *)(B + n0) : (const char *)(B + (int64_t)n0 * K);

  // ---- global -> LDS copies, 16 B per lane, 1 KB per wave-wide copy
  // A (and B in TN): 8 rows of 128 B per copy; 32 copies per tile, 4 per wave.
  uint32_t goff_a[4], goff_b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = (i * NWAVES + wave) * 8 + (lane >> 3);
    const int cp = lane & 7;
    goff_a[i] = (uint32_t)row * (uint32_t)(K * 2) + (uint32_t)((cp ^ swz128(row)) * 16);
    if (!NN) {
      goff_b[i] = goff_a[i];
    } else {  // B tile is BK rows (k) of 512 B (256 n): 2 rows per copy
      const int krow = (i * NWAVES + wave) * 2 + (lane >> 5);
      const int cpb = lane & 31;
      goff_b[i] = (uint32_t)krow * (uint32_t)(N * 2) + (uint32_t)((cpb ^ swz512(krow)) * 16);
    }
  }
  auto load_stage = [&](int kt, int stage) {
    const char *ga = Ap + (size_t)kt * (BK * 2);
    const char *gb = NN ? Bp + (size_t)kt * BK * (size_t)(N * 2) : Bp + (size_t)kt * (BK * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_dma16(ga + goff_a[i], lds_base + stage * STAGE + (i * NWAVES + wave) * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_dma16(gb + goff_b[i], lds_base + stage * STAGE + A_TILE + (i * NWAVES + wave) * 1024);
  };

  // ---- LDS read addresses.  K-step s (16 deep): lane (r, g) needs k = 16s + 8g .. +8 of its row.
  int a_rd[4], b_rd[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    a_rd[s] = (wm * 128 + r) * 128 + (((2 * s + g) ^ swz128(r)) * 16);          // + 32*128 per m block
    b_rd[s] = A_TILE + (wn * 64 + r) * 128 + (((2 * s + g) ^ swz128(r)) * 16);  // + 32*128 per n block (TN)
  }
  // NN: B^T operand via ds_read_b64_tr_b16 from [k][n] rows (see the V operand of the attention kernel)
  const int li = lane & 15;
  const int bk_row = 8 * g + (li >> 2);                                // + 16 s + 4 h2: slot t of lane g is k = 16s + 8g + t, as in A
  const int bn_col = wn * 64 + 16 * ((lane >> 4) & 1) + 4 * (li & 3);  // + 32 nb
  int bt_rd[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int c = (bn_col + 32 * nb) >> 3;
    bt_rd[nb] = A_TILE + bk_row * 512 + ((c ^ swz512(bk_row)) * 16) + (bn_col & 7) * 2;
  }

  f32x16 acc[4][2];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mb][nb][v] = 0.f;

  const int k_tiles = K / BK;
  // operand fetch for K-step s of the tile in LDS stage `st`
  auto fetch = [&](const char *st, int s, half8 (&aop)[4], half8 (&bop)[2]) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      if (!NN) {
        bop[nb] = *(const half8 *)(st + b_rd[s] + nb * 32 * 128);
      } else {
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
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) aop[mb] = *(const half8 *)(st + a_rd[s] + mb * 32 * 128);
  };
  auto mma = [&](const half8 (&aop)[4], const half8 (&bop)[2]) {
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)  // transposed block: MFMA rows = n (B operand first), columns = m
        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bop[nb], aop[mb], acc[mb][nb], 0, 0, 0);
  };

  load_stage(0, 0);
  wait_lds_dma();
  __syncthreads();
  half8 a0[4], b0[2], a1[4], b1[2];  // two operand register sets: K-step s+1 is fetched while K-step s multiplies
  fetch(smem, 0, a0, b0);
  for (int kt = 0; kt < k_tiles; ++kt) {
    const int stage = kt & 1;
    load_stage(kt + 1 < k_tiles ? kt + 1 : kt, stage ^ 1);
    const char *st = smem + stage * STAGE;
    // sched_barrier(0): the compiler's scheduler would otherwise sink each fetch down to its first use and expose
    // the LDS latency in front of every multiply
    fetch(st, 1, a1, b1);
    __builtin_amdgcn_sched_barrier(0);
    mma(a0, b0);
    __builtin_amdgcn_sched_barrier(0);
    fetch(st, 2, a0, b0);
    __builtin_amdgcn_sched_barrier(0);
    mma(a1, b1);
    __builtin_amdgcn_sched_barrier(0);
    fetch(st, 3, a1, b1);
    __builtin_amdgcn_sched_barrier(0);
    mma(a0, b0);
    __builtin_amdgcn_sched_barrier(0);
    wait_lds_dma();
    __syncthreads();  // next stage has landed for everybody; this stage may be refilled after the last reads below
    // first K-step of the next tile is fetched before the last multiply of this one (the barrier above already
    // guarantees the data; the refill of THIS stage only starts after the next barrier)
    fetch(smem + (stage ^ 1) * STAGE, 0, a0, b0);
    __builtin_amdgcn_sched_barrier(0);
    mma(a1, b1);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- epilogue: lane (m = r, g) holds n = 8i + 4g + j of each block
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    _Float16 *crow = C + (int64_t)(m0 + wm * 128 + mb * 32 + r) * N + n0 + wn * 64;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        half4 o4;
#pragma unroll
        for (int j = 0; j < 4; ++j) o4[j] = (_Float16)acc[mb][nb][4 * i + j];
        *(half4 *)(crow + nb * 32 + 8 * i + 4 * g) = o4;
      }
  }
}

template <bool NN>
hipError_t launch(int M, int N, int K, const void *A, const void *B, void *C, hipStream_t s) {
  static bool attr_done = false;
  auto kern = gemm_f16_kernel<NN>;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, dim3((M / BM) * (N / BN)), dim3(T), LDS_BYTES, s, (const _Float16 *)A, (const _Float16 *)B,
                     (_Float16 *)C, M, N, K);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_f16(int M, int N, int K, const void *A, const void *B, void *C, int layout, hipStream_t s) {
  return layout == 0 ? launch<false>(M, N, K, A, B, C, s) : launch<true>(M, N, K, A, B, C, s);
}

}  // namespace cfk
