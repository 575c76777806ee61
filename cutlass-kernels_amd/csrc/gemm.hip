// Dense (batched) GEMM D = alpha * A.B + beta * C with fp32 accumulation and an fp32 epilogue, D row-major M x N, for
// fp16 operands (v_mfma_f32_16x16x32_f16) and fp32 operands (v_mfma_f32_32x32x2_f32) -- gfx950 only.
//
// Secondary bench beside the attention kernels, with their XOR-swizzled LDS rows and transpose reads.
// Takes the place of gemm_device/gemm of the reference's CuTe example (src/cute-gemm-tma-gma/gemm.cu:57-463: TMA load
// of one A and one B tile, one synchronous WGMMA batch per K-tile, no pipelining; its type 1 is float, type 3 half,
// :677-684; batch count L with packed strides, :519-521) and of the CUTLASS-API example with its alpha / beta
// epilogue (src/cutlass-gemm/gemm.cu:87-140, 318-324).  Layouts: TN = A is M x K and B is N x K, both K-contiguous
// (the reference's form, :362-380); NN (fp16 only) = B is K x N, N-contiguous (the literal C = A.B), whose B operand is
// read with ds_read_b64_tr_b16 exactly as V is in the attention kernel.  The reference writes C column-major
// (:386-389); C and D are row-major here.  gfx950 has no tf32/xf32 MFMA: fp32 operands multiply in full fp32.
//
// Workgroup = 4 waves (one per SIMD) on a 256 x 256 macro tile; wave (wm, wn) of a 2 x 2 grid owns 128 x 128 of C, its
// 256 accumulator registers in the AGPR half of the register file.  fp16 operands multiply on 16x16x32 MFMAs
// (gemm_kernel16, 8 x 8 blocks per wave: the power-efficient shape on this board), fp32 operands on 32x32x2
// (gemm_kernel_f32, 4 x 4 blocks).  K tiles are 128 bytes deep (64 halves / 32 floats) and go global -> registers -> LDS:
// 16-byte buffer loads a tile ahead (scalar resource + 32-bit lane offset, no vector address arithmetic), parked in
// one of two 64 KB LDS stages by ds_write_b128 while the other stage multiplies, one barrier per tile; every multiply
// is followed by at most one fragment read or one store/load pair, see the pipeline comments in the kernels.
// (Global -> LDS copy instructions instead of the register path, through a ring of four 32-deep stages and spread the
// same way, measured 1.57 against 1.94 PFLOP/s on constant operands: with one wave per SIMD an LDS-destination load
// holds up the issuing wave and with it the MFMA pipe.)  The MFMA computes the TRANSPOSED block (rows = n, columns =
// m); the epilogue stages each row of blocks through LDS and stores whole rows, 16 bytes per lane.
// Measured on MI355X, M=N=K=8192 fp16 TN: 1.34-1.40 PFLOP/s on U(-1,1) operands, where the board is power-limited
// (the vendor library's kernel for this shape, also on 16x16x32 MFMAs: 1.55); fp32: 152 TFLOP/s.
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
typedef int int4v __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256;

// K-contiguous rows of PITCH bytes (128: two rows per 256-byte bank period; 64: four): 16 consecutive rows at one
// 16-byte chunk index must spread over all banks -> rows at the same place in the period get distinct XOR values
template <int PITCH>
__device__ __forceinline__ int swz_k(int row) { return PITCH == 128 ? (row >> 1) & 7 : (row >> 2) & 3; }

// The fp32 kernel (TN only), on v_mfma_f32_32x32x2_f32: 4 x 4 blocks of 32 x 32 per wave.  BKB = bytes of a K-contiguous
// tile row (32 floats at 128).  blockIdx.y = problem of a batch.  4 waves of 128 x 128, one per SIMD.
template <int BKB>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
gemm_kernel_f32(const float *__restrict__ A, const float *__restrict__ B, const float *__restrict__ Cin, float *__restrict__ D,
                int M, int N, int K, float alpha, float beta) {
  using T = float;
  constexpr int ES = sizeof(T);
  constexpr int BK = BKB / ES;
  using Frag = f32x4;  // 16 bytes of a row: the operand of one K-step
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, g = lane >> 5;
  constexpr int WN = 2, NWAVES = 4;
  constexpr int NB = 4;                // 32-column blocks per wave
  constexpr int PITCH = BKB;           // bytes per K-contiguous LDS row
  constexpr int A_TILE = BM * PITCH;   // B tile likewise (n rows)
  constexpr int STAGE = 2 * A_TILE;
  constexpr int CPW = A_TILE / 1024 / NWAVES;  // 16-byte pieces per lane and operand tile
  constexpr int RPC = 1024 / PITCH;    // rows per wave-wide 1 KB piece
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

  const int64_t batch = blockIdx.y;  // packed strides M*K, N*K, M*N (reference: gemm.cu:519-521)
  A += batch * M * K;
  B += batch * N * K;
  D += batch * M * N;
  if (Cin) Cin += batch * M * N;
  const char *Ap = (const char *)(A + (int64_t)m0 * K);
  const char *Bp = (const char *)(B + (int64_t)n0 * K);

  // ---- global -> register -> LDS staging, 16 B per lane and piece.  Piece i of wave w covers tile rows
  // (i*NWAVES + w)*RPC .. +RPC; lane l owns LDS slot (row l / CPR, chunk position l % CPR) of the piece and fetches
  // chunk position ^ swz(row) of that row: the XOR swizzle is applied on the global side, LDS writes are linear.
  // The loads are ordinary loads into registers (compiler-tracked), issued a tile ahead of the ds_write that parks
  // them in LDS: unlike LDS-destination loads they do not hold up the issuing wave, which with one wave per SIMD
  // would hold up the MFMA pipe.
  uint32_t goff_a[CPW], goff_b[CPW];
#pragma unroll
  for (int i = 0; i < CPW; ++i) {
    const int row = (i * NWAVES + wave) * RPC + lane / (PITCH / 16);
    const int cp = lane % (PITCH / 16);
    goff_a[i] = (uint32_t)row * (uint32_t)(K * ES) + (uint32_t)((cp ^ swz_k<PITCH>(row)) * 16);
    goff_b[i] = goff_a[i];
  }
  const uint32_t st_off = wave * 1024 + lane * 16;  // + (piece * NWAVES) * 1024 (+ A_TILE for B) + stage * STAGE
  int4v stg[2 * CPW];                               // the tile in flight: A pieces, then B pieces
  // Buffer loads: a scalar resource per operand tile (rebuilt per tile by the scalar unit) plus the lane's 32-bit
  // offset, so that a load costs no vector address arithmetic.
  using Rsrc = __amdgpu_buffer_rsrc_t;
  auto tile_ptrs = [&](int kt, Rsrc &ga, Rsrc &gb) {
    const char *pa = Ap + (size_t)kt * PITCH;
    const char *pb = Bp + (size_t)kt * PITCH;
    ga = __builtin_amdgcn_make_buffer_rsrc((void *)pa, 0, -1, 0x00020000);
    gb = __builtin_amdgcn_make_buffer_rsrc((void *)pb, 0, -1, 0x00020000);
  };
  auto load_piece = [&](Rsrc ga, Rsrc gb, int c) {
    const u32x4 x = c < CPW ? __builtin_amdgcn_raw_buffer_load_b128(ga, (int)goff_a[c], 0, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(gb, (int)goff_b[c - CPW], 0, 0);
    stg[c] = __builtin_bit_cast(int4v, x);
  };
  auto store_piece = [&](int stage, int c) {
    char *dst = smem + stage * STAGE + st_off + (c < CPW ? c * NWAVES * 1024 : A_TILE + (c - CPW) * NWAVES * 1024);
    *(int4v *)dst = stg[c];
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
  f32x16 acc[4][NB];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mb][nb][v] = 0.f;

  const int k_tiles = K / BK;
  // One 16-byte operand fragment of K-step s of the tile in LDS stage `st`, in the order the multiplies first need
  // them: i = 0: B block 0, 1: A block 0, 2..4: B blocks 1..3, 5..7: A blocks 1..3
  auto fetch_one = [&](const char *st, int s, int i, Frag (&aop)[4], Frag (&bop)[NB]) {
    const bool is_a = i == 1 || i >= 5;
    const int blk = i == 0 ? 0 : i == 1 ? 0 : i <= 4 ? i - 1 : i - 4;
    if (is_a) {
      aop[blk] = *(const Frag *)(st + a_rd[s] + blk * 32 * PITCH);
    } else {
      bop[blk] = *(const Frag *)(st + b_rd[s] + blk * 32 * PITCH);
    }
  };
  // One block multiply (one MFMA, or 4 for fp32 operands).  Transposed block: MFMA rows = n (B operand first)
  auto mma_block = [&](const Frag (&aop)[4], const Frag (&bop)[NB], int mb, int nb) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(bop[nb][e], aop[mb][e], acc[mb][nb], 0, 0, 0);
  };

  // Pipeline: two LDS stages and one tile in registers.  While tile kt multiplies out of stage kt % 2, the registers
  // (tile kt+1, loaded a tile ago) are written to the other stage -- whose readers passed the barrier that opened
  // this tile -- and refilled with tile kt+2, all before the tile's one barrier.  With one wave per SIMD nothing but
  // this wave's own instruction stream keeps the MFMA pipe fed: a run of LDS and memory instructions between two
  // multiplies stalls it.  So every K-step is laid out as 16 slots of one block multiply plus at most a piece of the
  // other work, pinned in that order: the even slots carry the eight fragment reads of the next K-step (or, behind
  // the barrier, of the next tile's first); the odd slots of all K-steps but the last carry the staging, the
  // ds_write of a piece of tile kt+1 and, LD_LAG odd slots later, the load of the same piece of tile kt+2 (a load
  // issued right behind the store that frees its register waits for that store to have read it).
  // Measured (8192^3, constant operands): 1.64 PFLOP/s with reads and staging in runs of 8 and 3 instructions, 1.94
  // with one per slot, 2.04 with the lagged load.
  constexpr int CPT = 2 * CPW;
  constexpr int ST_STEPS = KS > 1 ? KS - 1 : 1;
  constexpr int ST_PER = (CPT + ST_STEPS - 1) / ST_STEPS;     // pieces per K-step
  constexpr int LD_LAG = 2;
  static_assert(ST_PER + LD_LAG <= 8, "stores and lagged loads of a K-step must fit its eight odd slots");
  auto st_slot = [](int c) { return (c / ST_PER) * 8 + c % ST_PER; };  // odd slot (of the tile) of piece c's store
  Rsrc ga, gb;
  tile_ptrs(0, ga, gb);
#pragma unroll
  for (int c = 0; c < CPT; ++c) load_piece(ga, gb, c);
#pragma unroll
  for (int c = 0; c < CPT; ++c) store_piece(0, c);
  tile_ptrs(k_tiles > 1 ? 1 : 0, ga, gb);
#pragma unroll
  for (int c = 0; c < CPT; ++c) load_piece(ga, gb, c);
  __syncthreads();
  Frag aop[2][4], bop[2][NB];  // two operand register sets: K-step s+1 is fetched while K-step s multiplies
#pragma unroll
  for (int i = 0; i < 8; ++i) fetch_one(smem, 0, i, aop[0], bop[0]);
  int stage = 0;
  for (int kt = 0; kt < k_tiles; ++kt) {
    const char *st = smem + stage * STAGE;
    const int nstage = stage ^ 1;
    tile_ptrs(kt + 2 < k_tiles ? kt + 2 : k_tiles - 1, ga, gb);  // clamped at the end: a surplus tile is loaded and dropped
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) {
      const bool last = s2 + 1 == KS;
      // tile kt+1 is in LDS for everybody; all reads of this tile's stage have completed
      if (last) __syncthreads();
      const char *src = last ? smem + nstage * STAGE : st;
      const int s_next = last ? 0 : s2 + 1;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        mma_block(aop[s2 & 1], bop[s2 & 1], i / 4, i % 4);
        if (i % 2 == 0) {
          fetch_one(src, s_next, i / 2, aop[(s2 + 1) & 1], bop[(s2 + 1) & 1]);
        } else {
          const int t = s2 * 8 + i / 2;  // odd slot number within the tile
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (st_slot(c) == t) store_piece(nstage, c);
#pragma unroll
          for (int c = 0; c < CPT; ++c)
            if (st_slot(c) + LD_LAG == t) load_piece(ga, gb, c);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    stage = nstage;
  }

  // ---- epilogue: D = alpha * acc + beta * C in fp32 (src/cutlass-gemm/gemm.cu:318-324).  Lane (m = r, g) holds
  // n = 8i + 4g + j of each block: stored directly, a wave-wide store would touch 32 rows with 16 or 32 bytes each.
  // Each 32 x 128 row of blocks goes through the wave's own LDS region (the stages are dead: every wave passed the last
  // tile's barrier after its last stage reads and writes) as raw fp32 accumulators and leaves as whole rows, 16 bytes
  // per lane; alpha, beta and the single rounding to T are applied on the way out.
  constexpr int E_PITCH = 128 * 4 + 16;          // bytes per staged row of 128 floats, padded
  constexpr int EPL = 16 / ES;                   // elements per lane and store (8 halves / 4 floats)
  constexpr int LPR = 128 / EPL, RPP = 64 / LPR; // lanes per row, rows per wave-wide store
  using OutV = f32x4;
  const bool with_c = Cin != nullptr && beta != 0.f;
  char *et = smem + wave * (32 * E_PITCH);
  const int e_row = lane / LPR, e_col = (lane % LPR) * EPL;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f32x4 v4;
#pragma unroll
        for (int j = 0; j < 4; ++j) v4[j] = acc[mb][nb][4 * i + j];
        *(f32x4 *)(et + r * E_PITCH + (nb * 32 + 8 * i + 4 * g) * 4) = v4;
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int pass = 0; pass < 32 / RPP; ++pass) {
      const int row = pass * RPP + e_row;
      const int64_t off = (int64_t)(m0 + wm * 128 + mb * 32 + row) * N + n0 + wn * NB * 32 + e_col;
      float v[EPL];
#pragma unroll
      for (int q = 0; q < EPL / 4; ++q) {
        const f32x4 x = *(const f32x4 *)(et + row * E_PITCH + (e_col + 4 * q) * 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[4 * q + j] = alpha * x[j];
      }
      if (with_c) {
        const OutV c = *(const OutV *)(Cin + off);
#pragma unroll
        for (int j = 0; j < EPL; ++j) v[j] += beta * (float)c[j];
      }
      OutV o;
#pragma unroll
      for (int j = 0; j < EPL; ++j) o[j] = (T)v[j];
      *(OutV *)(D + off) = o;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // the region is rewritten by the next row of blocks
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// 512-byte rows read with ds_read_b64_tr_b16 in the 16x16x32 lane map: a 32-lane half of the wave touches rows
// 8g .. 8g+3 of two k groups g x 32 contiguous bytes; bit 0 stays clear so the 32 bytes stay contiguous
__device__ __forceinline__ int swz512n(int row) { return ((row & 3) | (((row >> 3) & 1) << 2)) << 1; }

// The fp16 kernel on 16x16x32 MFMAs (v_mfma_f32_16x16x32_f16): the same workgroup tile, staging path and epilogue as
// gemm_kernel_f32, with the wave's 128 x 128 of C as 8 x 8 blocks (NWAVES = 4; NWAVES = 8 runs two waves per SIMD on
// 128 x 64 each and measured the same).  Measured, 8192^3 TN, same session: 1401 TFLOP/s on U(-1,1) operands against
// 1309 for the same kernel on 32x32x16 MFMAs (8 waves: 1390); on constant operands 1837 against 2048 (LDS writes between the
// short multiplies hold the MFMA pipe up for about 20 cycles each).  On U(-1,1) operands this board is
// power-limited and the deeper, narrower MFMA moves half the accumulator bits per FLOP: a register-only loop sustains
// 1.90 PFLOP/s with it against 1.69 with 32x32x16.  Lane (c = lane % 16, g = lane / 16) holds, of an operand fragment,
// row c and contraction slots 8g .. 8g+7 (16 bytes), and of an accumulator block column c, rows 4g .. 4g+3.  The MFMA
// computes the transposed block (rows = n, columns = m), so a lane owns 4 consecutive n of one row m of C.
template <bool NN, int NWAVES>
__global__ void __launch_bounds__(NWAVES * 64) __attribute__((amdgpu_waves_per_eu(NWAVES / 4, NWAVES / 4)))
gemm_kernel16(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, const _Float16 *__restrict__ Cin,
              _Float16 *__restrict__ D, int M, int N, int K, float alpha, float beta) {
  using T = _Float16;
  constexpr int ES = 2, PITCH = 128, BK = PITCH / ES;  // 64-deep K tiles: two K-steps of 32
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, g = lane >> 4;
  constexpr int WN = NWAVES / 2;       // waves along n: the wave tile is 128 x 256/WN
  constexpr int NB = 8;                // 16-row blocks per wave
  constexpr int NBN = BN / WN / 16;    // 16-column blocks per wave
  constexpr int A_TILE = BM * PITCH;   // TN: B tile likewise (n rows); NN: BK rows (k) of 512 B
  constexpr int STAGE = 2 * A_TILE;
  constexpr int CPW = A_TILE / 1024 / NWAVES;  // 16-byte pieces per lane and operand tile
  constexpr int RPC = 1024 / PITCH;    // rows per wave-wide 1 KB piece
  constexpr int KS = PITCH / 64;       // K-steps per tile: 64 bytes of a row (four 16-byte fragments, one per g) each
  const int wm = wave / WN, wn = wave % WN;

  // tile order and XCD remap as in gemm_kernel_f32
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

  const int64_t batch = blockIdx.y;
  A += batch * M * K;
  B += batch * N * K;
  D += batch * M * N;
  if (Cin) Cin += batch * M * N;
  const char *Ap = (const char *)(A + (int64_t)m0 * K);
  const char *Bp = NN ? (const char *)(B + n0) : (const char *)(B + (int64_t)n0 * K);

  // ---- global -> register -> LDS staging (see gemm_kernel_f32)
  uint32_t goff_a[CPW], goff_b[CPW];
#pragma unroll
  for (int i = 0; i < CPW; ++i) {
    const int row = (i * NWAVES + wave) * RPC + lane / (PITCH / 16);
    const int cp = lane % (PITCH / 16);
    goff_a[i] = (uint32_t)row * (uint32_t)(K * ES) + (uint32_t)((cp ^ swz_k<PITCH>(row)) * 16);
    if (!NN) {
      goff_b[i] = goff_a[i];
    } else {  // B tile is BK rows (k) of 512 B (256 n): 2 rows per piece
      const int krow = (i * NWAVES + wave) * 2 + (lane >> 5);
      const int cpb = lane & 31;
      goff_b[i] = (uint32_t)krow * (uint32_t)(N * 2) + (uint32_t)((cpb ^ swz512n(krow)) * 16);
    }
  }
  const uint32_t st_off = wave * 1024 + lane * 16;
  int4v stg[2 * CPW];
  using Rsrc = __amdgpu_buffer_rsrc_t;
  auto tile_ptrs = [&](int kt, Rsrc &ga, Rsrc &gb) {
    const char *pa = Ap + (size_t)kt * PITCH;
    const char *pb = NN ? Bp + (size_t)kt * BK * (size_t)(N * 2) : Bp + (size_t)kt * PITCH;
    ga = __builtin_amdgcn_make_buffer_rsrc((void *)pa, 0, -1, 0x00020000);
    gb = __builtin_amdgcn_make_buffer_rsrc((void *)pb, 0, -1, 0x00020000);
  };
  auto load_piece = [&](Rsrc ga, Rsrc gb, int p) {
    const u32x4 x = p < CPW ? __builtin_amdgcn_raw_buffer_load_b128(ga, (int)goff_a[p], 0, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(gb, (int)goff_b[p - CPW], 0, 0);
    stg[p] = __builtin_bit_cast(int4v, x);
  };
  auto store_piece = [&](int stage, int p) {
    char *dst = smem + stage * STAGE + st_off + (p < CPW ? p * NWAVES * 1024 : A_TILE + (p - CPW) * NWAVES * 1024);
    *(int4v *)dst = stg[p];
  };

  // ---- LDS read addresses.  K-step s: lane (c, g) needs bytes 64s + 16g .. +16 of its row (k = 32s + 8g .. +8).
  // swz_k<128> depends on the row within its group of 16 only, so blocks are immediates.
  int a_rd[KS], b_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    a_rd[s] = (wm * 128 + c) * PITCH + (((4 * s + g) ^ swz_k<PITCH>(c)) * 16);                // + 16 rows per m block
    b_rd[s] = A_TILE + (wn * NBN * 16 + c) * PITCH + (((4 * s + g) ^ swz_k<PITCH>(c)) * 16);       // + 16 rows per n block (TN)
  }
  // NN: the n-side operand via two ds_read_b64_tr_b16 from [k][n] rows: within its block of 16 lanes, lane L hands
  // the read the address of (k row L/4, columns 4(L%4) .. +3) and receives k rows 0..3 of column L; block g reads k
  // rows 8g .. 8g+3, the second read 4 further
  const int bk_row = 8 * g + (c >> 2);          // + 32 s (+ 4)
  const int cg = c & 3;
  int bt_rd[NBN];
#pragma unroll
  for (int nb = 0; nb < NBN; ++nb) {
    const int chunk = (wn * NBN * 16 + 16 * nb) / 8 + (cg >> 1);  // 16-byte chunk of the 512-byte row
    bt_rd[nb] = A_TILE + bk_row * 512 + ((chunk ^ swz512n(bk_row)) * 16) + (cg & 1) * 8;
  }

  f32x4 acc[NB][NBN];  // [m block][n block]
#pragma unroll
  for (int mb = 0; mb < NB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NBN; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int k_tiles = K / BK;
  // operand fragments of K-step s of the tile in LDS stage `st`: m block blk, n block blk
  auto fetch_a = [&](const char *st, int s, int blk) -> half8 { return *(const half8 *)(st + a_rd[s] + blk * 16 * PITCH); };
  auto fetch_b = [&](const char *st, int s, int blk) -> half8 {
    if constexpr (!NN) {
      return *(const half8 *)(st + b_rd[s] + blk * 16 * PITCH);
    } else {
      union {
        struct { short4v lo, hi; } p;
        half8 h;
      } u;
      const char *bp = st + bt_rd[blk] + s * 32 * 512;
      u.p.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, bp));
      u.p.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4v, bp + 4 * 512));
      return u.h;
    }
  };

  // Pipeline as in gemm_kernel_f32 (two LDS stages, one tile in registers, one barrier per tile), laid out as slots of
  // one multiply each (K-step major, then m block, then n block; SPM = NBN slots per m block) with at most one piece
  // of other work behind each multiply, pinned in that order.  Fragment registers: the n-side fragments of a K-step
  // are live throughout it and double-buffered (bop[K-step parity]); the m-side fragment of block mb is only needed
  // for its NBN multiplies and lives in a ring of four (aop[mb % 4]), read two blocks ahead.
  //   K-step 0:  first slot of m block mb: m fragment mb+2 (the last two: blocks 0, 1 of K-step 1);  slot SPM/2 of
  //              m blocks 0 .. NBN-1: n fragment mb of K-step 1;  the CPT slots i % (NB*NBN/CPT) == 1: ds_write of a
  //              staging piece of tile kt+1 and, LD_LAG pieces behind it, the load of the same piece of tile kt+2
  //   K-step 1:  first slot of m blocks 0..5: m fragment mb+2;  first slot of m block 6: the barrier (every read of
  //              this tile's stage and every write of the next tile's is in front of it), then one per slot the first
  //              fragments of the next tile (n 0 .. NBN-1 and m 0, 1 of its K-step 0) in the order they are needed
  constexpr int CPT = 2 * CPW;
  constexpr int LD_LAG = 2;
  constexpr int SPM = NBN;                    // slots per m block
  constexpr int ST_EVERY = NB * NBN / CPT;    // a staging piece every so many slots of K-step 0
  static_assert(KS == 2 && ST_EVERY >= 2 && NB * NBN % CPT == 0, "slot layout");
  // The multiplies are asm statements with "+a" accumulators: the compiler's hazard recognizer does not see the
  // matrix-pipe write -> accumulate-read dependency between two of them, so the distance between two multiplies into
  // one accumulator is this layout's business.  Every accumulator block is used once per K-step: NB * NBN multiplies
  // lie between two uses (64), each holding the pipe for the 4 passes of v_mfma_f32_16x16x32_f16; back-to-back
  // dependent MFMAs of this shape need 4 passes + 2 wait states.  Fewer blocks per wave than that (or a reordering that
  // revisits a block within one K-step) would need nops here.
  static_assert(NB * NBN >= 8, "distance between two multiplies into one accumulator: at least the MFMA's passes plus its wait states");
  Rsrc ga, gb;
  tile_ptrs(0, ga, gb);
#pragma unroll
  for (int p = 0; p < CPT; ++p) load_piece(ga, gb, p);
#pragma unroll
  for (int p = 0; p < CPT; ++p) store_piece(0, p);
  tile_ptrs(k_tiles > 1 ? 1 : 0, ga, gb);
#pragma unroll
  for (int p = 0; p < CPT; ++p) load_piece(ga, gb, p);
  __syncthreads();
  half8 aop[4], bop[2][NBN];
#pragma unroll
  for (int nb = 0; nb < NBN; ++nb) bop[0][nb] = fetch_b(smem, 0, nb);
  aop[0] = fetch_a(smem, 0, 0);
  aop[1] = fetch_a(smem, 0, 1);
  int stage = 0;
  for (int kt = 0; kt < k_tiles; ++kt) {
    const char *st = smem + stage * STAGE;
    const char *nx = smem + (stage ^ 1) * STAGE;
    const int nstage = stage ^ 1;
    tile_ptrs(kt + 2 < k_tiles ? kt + 2 : k_tiles - 1, ga, gb);  // clamped at the end: a surplus tile is loaded and dropped
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) {
#pragma unroll
      for (int i = 0; i < NB * NBN; ++i) {
        const int mb = i / SPM, nb = i % SPM;
        if (s2 == 1 && i == 6 * SPM) __syncthreads();
        // written out so that the accumulator is updated in place in the AGPR half: through the builtin the register
        // allocator moves the small accumulators between the two halves (280 copies per tile).  Nothing but these
        // multiplies touches the accumulators inside the loop, so no hazard is hidden from the compiler here.
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[mb][nb]) : "v"(bop[s2][nb]), "v"(aop[mb % 4]));
        if (nb == 0 && (s2 == 0 || mb <= 5)) {
          const int blk = mb + 2;
          aop[blk % 4] = blk < NB ? fetch_a(st, s2, blk) : fetch_a(st, 1, blk - NB);
        }
        if (s2 == 0 && nb == SPM / 2 && mb < NBN) bop[1][mb] = fetch_b(st, 1, mb);
        if (s2 == 1 && i >= 6 * SPM && i < 6 * SPM + NBN + 2) {
          // n 0, m 0, n 1, m 1, n 2 ...
          const int j = i - 6 * SPM;
          if (j == 1) aop[0] = fetch_a(nx, 0, 0);
          else if (j == 3) aop[1] = fetch_a(nx, 0, 1);
          else bop[0][j == 0 ? 0 : j == 2 ? 1 : j - 2] = fetch_b(nx, 0, j == 0 ? 0 : j == 2 ? 1 : j - 2);
        }
        if (i % ST_EVERY == 1) {
          const int q = (s2 * NB * NBN + i) / ST_EVERY;  // staging slot number within the tile
          if (q < CPT) store_piece(nstage, q);
          if (q >= LD_LAG && q - LD_LAG < CPT) load_piece(ga, gb, q - LD_LAG);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    stage = nstage;
  }

  // the last multiplies have left the pipe before the epilogue reads their accumulators (the compiler does not see
  // the dependency through the asm statements)
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // ---- epilogue: D = alpha * acc + beta * C in fp32, each 16 x 128 row of blocks staged through the wave's own LDS
  // region (see gemm_kernel_f32) and stored as whole rows, 16 bytes per lane
  constexpr int E_PITCH = 128 * 4 + 16;
  constexpr int EPL = 8;                          // halves per lane and store
  constexpr int WCOLS = NBN * 16;                   // columns of the wave tile
  constexpr int LPR = WCOLS / EPL, RPP = 64 / LPR;  // lanes per row, rows per wave-wide store
  const bool with_c = Cin != nullptr && beta != 0.f;
  char *et = smem + wave * (16 * E_PITCH);
  const int e_row = lane / LPR, e_col = (lane % LPR) * EPL;
#pragma unroll
  for (int mb = 0; mb < NB; ++mb) {
#pragma unroll
    for (int nb = 0; nb < NBN; ++nb) *(f32x4 *)(et + c * E_PITCH + (nb * 16 + 4 * g) * 4) = acc[mb][nb];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int pass = 0; pass < 16 / RPP; ++pass) {
      const int row = pass * RPP + e_row;
      const int64_t off = (int64_t)(m0 + wm * 128 + mb * 16 + row) * N + n0 + wn * WCOLS + e_col;
      float v[EPL];
#pragma unroll
      for (int q = 0; q < EPL / 4; ++q) {
        const f32x4 x = *(const f32x4 *)(et + row * E_PITCH + (e_col + 4 * q) * 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[4 * q + j] = alpha * x[j];
      }
      if (with_c) {
        const half8 cv = *(const half8 *)(Cin + off);
#pragma unroll
        for (int j = 0; j < EPL; ++j) v[j] += beta * (float)cv[j];
      }
      half8 o;
#pragma unroll
      for (int j = 0; j < EPL; ++j) o[j] = (T)v[j];
      *(half8 *)(D + off) = o;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // the region is rewritten by the next row of blocks
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

template <class T, bool NN>
struct GemmLaunch {
  static constexpr int BKB = 128;  // 64-deep K tiles for fp16, 32-deep for fp32
  static constexpr int LDS_BYTES = 2 * 2 * BM * BKB;
  static constexpr int WAVES16 = 4;  // waves of the fp16 kernel
  static constexpr auto kern = [] {
    if constexpr (sizeof(T) == 2) return gemm_kernel16<NN, WAVES16>;
    else return gemm_kernel_f32<BKB>;
  }();
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
    hipLaunchKernelGGL(kern, dim3((g.M / BM) * (g.N / BN), g.batch), dim3(sizeof(T) == 2 ? WAVES16 * 64 : 256), LDS_BYTES, s, (const T *)g.A,
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
