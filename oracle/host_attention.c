/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the fused multi-head-attention forward path and the
 * dense GEMM example.  Nothing in the product (the HIP library, its host driver, the Python binding)
 * may link, load or call this file; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg do, and only as the checker / the reported CPU baseline.
 *
 * It restates, in plain C with OpenMP, the host reference attention of the reference repository:
 *   TestAttention::compute            include/utils/fmha_cutlass.hpp:154-317
 *   (GEMM-I   P = alpha0 * Q.K^T      include/utils/fmha_cutlass.hpp:204-220, fp32 accumulate,
 *    softmax rows on the host         include/utils/fmha_cutlass.hpp:240-302, both exp and exp2 branches,
 *    GEMM-II  O = P.V                 include/utils/fmha_cutlass.hpp:305-314)
 * over the reference's [B, S, H, D] ("BMHK", D contiguous) tensors with leading dimension H*D
 * (include/utils/fmha_cutlass.hpp:146-150), on float up-casts of the operands exactly as the driver
 * feeds it (src/fmha-pipeline/fmha_forward.cu:613-631).
 *
 * The two GEMMs of the reference run as CUTLASS's naive reference::device::GemmComplex (an external,
 * un-vendored dependency): one thread per output element, k ascending, float accumulator,
 * result = alpha * acc.  That summation order is kept here (k ascending per output element).
 *
 * Parity pins (tests/test_oracle.py): float64 closed-form softmax(QK^T/sqrt(D))V on small inputs,
 * exp-branch == exp2-branch, rows of P sum to one, Q = 0 gives the mean of V, a dominant key selects
 * its V row, key-permutation invariance, integer-valued inputs give bit-exact scores.
 * The reference holds no golden vectors for this path; the literal curand input stream of its driver
 * is not reproducible here ("parity unpinned" for that stream only: the tests draw their own seeded inputs).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define CFK_ORACLE_LOG2E 1.4426950408889634074f /* fmha_cutlass.hpp:74 kLog2e */

int cfk_oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/*
 * One (batch, head) problem.  q/k/v/o point at element [b, 0, h, 0]; ld = H*D.
 * kt_scratch: D*Skv floats, K viewed column-major (k x n) as the reference's LayoutK does
 * (fmha_cutlass.hpp:37,147) so the n loop is unit-stride while k stays the ascending outer sum index.
 */
static void attention_one_head(const float *q, const float *k, const float *v, float *o, float *s_dbg,
                               float *norm, float *inv_sum_out, int Sq, int Skv, int D, int64_t ld,
                               float alpha0, int use_pow2, int use_prescaling, int row_start,
                               int row_step, float *kt_scratch) {
  const float alpha_mma0 = use_prescaling ? alpha0 : 1.0f; /* fmha_cutlass.hpp:206 */
  const float post_scaling = use_prescaling ? 1.0f : alpha0; /* fmha_cutlass.hpp:207 */

#pragma omp parallel for schedule(static)
  for (int n = 0; n < Skv; ++n)
    for (int d = 0; d < D; ++d) kt_scratch[(int64_t)d * Skv + n] = k[(int64_t)n * ld + d];

  const int n_rows = (Sq - row_start + row_step - 1) / row_step;
#pragma omp parallel
  {
    float *p = (float *)malloc(sizeof(float) * (size_t)Skv);
    float *acc_o = (float *)malloc(sizeof(float) * (size_t)D);
#pragma omp for schedule(dynamic, 8)
    for (int r = 0; r < n_rows; ++r) {
      const int m = row_start + r * row_step;
      const float *qm = q + (int64_t)m * ld;
      /* GEMM-I: acc over k ascending, then alpha * acc (GemmComplex semantics). */
      for (int n = 0; n < Skv; ++n) p[n] = 0.0f;
      for (int d = 0; d < D; ++d) {
        const float qv = qm[d];
        const float *ktd = kt_scratch + (int64_t)d * Skv;
#pragma omp simd
        for (int n = 0; n < Skv; ++n) p[n] += qv * ktd[n];
      }
      for (int n = 0; n < Skv; ++n) p[n] = alpha_mma0 * p[n];
      if (s_dbg) memcpy(s_dbg + (int64_t)m * Skv, p, sizeof(float) * (size_t)Skv); /* :230-236 */

      float mx, sum = 0.0f, inv;
      if (use_pow2) { /* fmha_cutlass.hpp:242-273 */
        for (int n = 0; n < Skv; ++n) p[n] = CFK_ORACLE_LOG2E * post_scaling * p[n];
        mx = p[0];
        for (int n = 1; n < Skv; ++n) mx = p[n] > mx ? p[n] : mx;
        for (int n = 0; n < Skv; ++n) sum += exp2f(p[n] - mx);
        inv = 1.0f / sum;
        for (int n = 0; n < Skv; ++n) p[n] = exp2f(p[n] - mx) * inv;
      } else { /* fmha_cutlass.hpp:274-302; post_scaling is not applied on this branch there either */
        mx = p[0];
        for (int n = 1; n < Skv; ++n) mx = p[n] > mx ? p[n] : mx;
        for (int n = 0; n < Skv; ++n) sum += expf(p[n] - mx);
        inv = 1.0f / sum;
        for (int n = 0; n < Skv; ++n) p[n] = expf(p[n] - mx) * inv;
      }
      if (norm) norm[m] = mx;
      if (inv_sum_out) inv_sum_out[m] = inv;

      /* GEMM-II: O[m, :] = sum_n P[m, n] * V[n, :], n ascending per output element. */
      for (int d = 0; d < D; ++d) acc_o[d] = 0.0f;
      for (int n = 0; n < Skv; ++n) {
        const float pn = p[n];
        const float *vn = v + (int64_t)n * ld;
#pragma omp simd
        for (int d = 0; d < D; ++d) acc_o[d] += pn * vn[d];
      }
      memcpy(o + (int64_t)m * ld, acc_o, sizeof(float) * (size_t)D);
    }
    free(p);
    free(acc_o);
  }
}

/*
 * fp32 reference attention.  Q: [B,Sq,H,D], K,V: [B,Skv,H,D], O: [B,Sq,H,D] (all float, D contiguous).
 * s_dbg (nullable): [B,H,Sq,Skv] pre-softmax scores as the reference stores them (alpha-scaled when
 * use_prescaling).  norm / inv_sum (nullable): [B,H,Sq] row max and 1/row-sum
 * (fmha_cutlass.hpp:185-188 offsets).
 * bh_pairs (nullable): n_pairs x {b,h} to restrict the (batch, head) problems computed; NULL = all.
 * Rows computed: row_start, row_start+row_step, ...; other rows of O are left untouched.
 * Returns 0, or -1 on bad arguments.
 */
int cfk_oracle_attention_f32(const float *Q, const float *K, const float *V, float *O, float *s_dbg,
                             float *norm, float *inv_sum, int B, int Sq, int Skv, int H, int D,
                             float alpha0, int use_pow2, int use_prescaling, const int *bh_pairs,
                             int n_pairs, int row_start, int row_step) {
  if (!Q || !K || !V || !O || B <= 0 || Sq <= 0 || Skv <= 0 || H <= 0 || D <= 0) return -1;
  if (row_step <= 0 || row_start < 0) return -1;
  const int64_t ld = (int64_t)H * D;
  float *kt = (float *)malloc(sizeof(float) * (size_t)D * (size_t)Skv);
  if (!kt) return -1;
  const int total = bh_pairs ? n_pairs : B * H;
  for (int i = 0; i < total; ++i) {
    const int b = bh_pairs ? bh_pairs[2 * i] : i / H;
    const int h = bh_pairs ? bh_pairs[2 * i + 1] : i % H;
    if (b < 0 || b >= B || h < 0 || h >= H) {
      free(kt);
      return -1;
    }
    const float *q = Q + (int64_t)b * Sq * ld + (int64_t)h * D;
    const float *k = K + (int64_t)b * Skv * ld + (int64_t)h * D;
    const float *v = V + (int64_t)b * Skv * ld + (int64_t)h * D;
    float *o = O + (int64_t)b * Sq * ld + (int64_t)h * D;
    const int64_t bh = (int64_t)b * H + h;
    attention_one_head(q, k, v, o, s_dbg ? s_dbg + bh * Sq * (int64_t)Skv : NULL,
                       norm ? norm + bh * Sq : NULL, inv_sum ? inv_sum + bh * Sq : NULL, Sq, Skv, D, ld,
                       alpha0, use_pow2, use_prescaling, row_start, row_step, kt);
  }
  free(kt);
  return 0;
}

/*
 * Dense GEMM oracle for the secondary bench: C[m, n] = sum_k A[m, k] * B[n, k]  ("TN": A is M x K and
 * B is N x K, both K-contiguous -- src/cute-gemm-tma-gma/gemm.cu:362-380), float accumulate, k
 * ascending, C written row-major float [n_rows x N] for the selected rows only.
 * b_is_kn != 0 reads B as K x N row-major instead (the literal C = A.B form).
 */
int cfk_oracle_gemm_f32(const float *A, const float *Bm, float *C, int M, int N, int K, int b_is_kn,
                        const int *rows, int n_rows) {
  if (!A || !Bm || !C || M <= 0 || N <= 0 || K <= 0) return -1;
  const int total = rows ? n_rows : M;
  float *bt = NULL; /* K x N view so that n is unit stride and k ascends in the outer loop */
  if (!b_is_kn) {
    bt = (float *)malloc(sizeof(float) * (size_t)K * (size_t)N);
    if (!bt) return -1;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
      for (int k = 0; k < K; ++k) bt[(int64_t)k * N + n] = Bm[(int64_t)n * K + k];
  }
  const float *bkn = b_is_kn ? Bm : bt;
  int bad = 0;
#pragma omp parallel for schedule(dynamic, 1)
  for (int r = 0; r < total; ++r) {
    const int m = rows ? rows[r] : r;
    if (m < 0 || m >= M) {
      bad = 1;
      continue;
    }
    float *c = C + (int64_t)r * N;
    for (int n = 0; n < N; ++n) c[n] = 0.0f;
    for (int k = 0; k < K; ++k) {
      const float a = A[(int64_t)m * K + k];
      const float *bk = bkn + (int64_t)k * N;
#pragma omp simd
      for (int n = 0; n < N; ++n) c[n] += a * bk[n];
    }
  }
  free(bt);
  return bad ? -1 : 0;
}
