// gemm -- bench/test driver for cfk_gemm_f16 with the command line and output line of the reference's CuTe GEMM
// example (src/cute-gemm-tma-gma/gemm.cu:469-691):   gemm <type> [M] [N] [K] [L] [check]
//   type 3 = fp16 (the only type built here; 1 = fp32/tf32 of the reference is reported unsupported)
//   M N K default 5120 5120 4096 (:668-678); L = batch count (problems run back to back); "check" verifies.
// A is M x K, B is N x K, both K-contiguous, values 2*rand()/RAND_MAX - 1 (:482-485), C preset to -1.  The
// reference compares bitwise with cuBLAS (:645-651); without cuBLAS here the check is a naive fp32 GPU GEMM of the
// same fp16 operands: |c - ref| <= 2e-3 * |ref| + 1e-2, plus a bit-exact run on integer-valued operands in [-8, 8]
// (the criterion of the reference's other GEMM example, src/cutlass-gemm/gemm.cu:277-294, 329-359).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/cfk_fmha.h"

#define HIP_CHECK(x)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (x);                                                                     \
    if (e_ != hipSuccess) {                                                                  \
      fprintf(stderr, "HIP error: %s (%s:%d)\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      return 2;                                                                              \
    }                                                                                        \
  } while (0)

// naive checker: one thread per C element, fp32 accumulate, k ascending
__global__ void naive_gemm_tn(const _Float16 *A, const _Float16 *B, float *C, int M, int N, int K) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)M * N) return;
  const int m = (int)(idx / N), n = (int)(idx % N);
  float acc = 0.f;
  for (int k = 0; k < K; ++k) acc += (float)A[(long long)m * K + k] * (float)B[(long long)n * K + k];
  C[idx] = acc;
}

static int run_check(int m, int n, int k, bool integers) {
  const size_t na = (size_t)m * k, nb = (size_t)n * k, nc = (size_t)m * n;
  std::vector<_Float16> ha(na), hb(nb), hc(nc);
  srand(integers ? 7 : 1);
  for (auto &x : ha) x = integers ? (_Float16)(float)(rand() % 17 - 8) : (_Float16)(2 * (rand() / double(RAND_MAX)) - 1);
  for (auto &x : hb) x = integers ? (_Float16)(float)(rand() % 17 - 8) : (_Float16)(2 * (rand() / double(RAND_MAX)) - 1);
  _Float16 *da, *db, *dc;
  float *dref;
  HIP_CHECK(hipMalloc(&da, na * 2));
  HIP_CHECK(hipMalloc(&db, nb * 2));
  HIP_CHECK(hipMalloc(&dc, nc * 2));
  HIP_CHECK(hipMalloc(&dref, nc * 4));
  HIP_CHECK(hipMemcpy(da, ha.data(), na * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(db, hb.data(), nb * 2, hipMemcpyHostToDevice));
  if (cfk_gemm_f16(m, n, k, da, db, dc, CFK_GEMM_TN, nullptr) != CFK_OK) {
    fprintf(stderr, "cfk_gemm_f16: %s\n", cfk_last_error());
    return 2;
  }
  hipLaunchKernelGGL(naive_gemm_tn, dim3((unsigned)((nc + 255) / 256)), dim3(256), 0, 0, da, db, dref, m, n, k);
  HIP_CHECK(hipDeviceSynchronize());
  std::vector<float> ref(nc);
  HIP_CHECK(hipMemcpy(hc.data(), dc, nc * 2, hipMemcpyDeviceToHost));
  HIP_CHECK(hipMemcpy(ref.data(), dref, nc * 4, hipMemcpyDeviceToHost));
  long long bad = 0;
  for (size_t i = 0; i < nc; ++i) {
    const float got = (float)hc[i];
    const bool ok = integers ? (hc[i] == (_Float16)ref[i]) : (std::fabs(got - ref[i]) <= 2e-3f * std::fabs(ref[i]) + 1e-2f);
    if (!ok && bad++ < 5) printf("failed [%zu] %f %f\n", i, got, ref[i]);
  }
  printf("gemm-check (%s): %s\n", integers ? "integer operands, bit-exact" : "uniform operands", bad ? "Failed" : "Passed");
  hipFree(da); hipFree(db); hipFree(dc); hipFree(dref);
  return bad ? 3 : 0;
}

int main(int argc, char **argv) {
  int type = 3, m = 5120, n = 5120, k = 4096, l = 1;
  bool check = false;
  int pos = 0;
  for (int i = 1; i < argc; ++i) {
    if (!strcmp(argv[i], "check")) { check = true; continue; }
    int v = atoi(argv[i]);
    switch (pos++) {
      case 0: type = v; break;
      case 1: m = v; break;
      case 2: n = v; break;
      case 3: k = v; break;
      case 4: l = v; break;
    }
  }
  if (type != 3) {
    printf("invalid type value (3 = fp16 is the only type built; 1 | 2 of the reference are not)\n");
    return 1;
  }
  if (l < 1) l = 1;
  printf("M = %d\nN = %d\nK = %d\nL = %d\n", m, n, k, l);
  const size_t na = (size_t)m * k, nb = (size_t)n * k, nc = (size_t)m * n;
  std::vector<_Float16> ha(na * l), hb(nb * l), hc(nc * l, (_Float16)-1.0f);
  for (auto &x : ha) x = (_Float16)(2 * (rand() / double(RAND_MAX)) - 1);
  for (auto &x : hb) x = (_Float16)(2 * (rand() / double(RAND_MAX)) - 1);
  _Float16 *da, *db, *dc;
  HIP_CHECK(hipMalloc(&da, na * l * 2));
  HIP_CHECK(hipMalloc(&db, nb * l * 2));
  HIP_CHECK(hipMalloc(&dc, nc * l * 2));
  HIP_CHECK(hipMemcpy(da, ha.data(), na * l * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(db, hb.data(), nb * l * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dc, hc.data(), nc * l * 2, hipMemcpyHostToDevice));
  auto run = [&]() -> int {
    for (int b = 0; b < l; ++b)
      if (cfk_gemm_f16(m, n, k, da + na * b, db + nb * b, dc + nc * b, CFK_GEMM_TN, nullptr) != CFK_OK) {
        fprintf(stderr, "cfk_gemm_f16: %s\n", cfk_last_error());
        return 2;
      }
    return 0;
  };
  if (run()) return 1;  // run once (:509-520)
  HIP_CHECK(hipDeviceSynchronize());
  const int timing_iterations = 1000;  // :499
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  HIP_CHECK(hipEventRecord(e0));
  for (int i = 0; i < timing_iterations; ++i)
    if (run()) return 1;
  HIP_CHECK(hipEventRecord(e1));
  HIP_CHECK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  const double t = ms / 1e3 / timing_iterations, gflops = 2.0 * m * n * k * l * 1e-9;  // :498
  printf("CUTE_GEMM:     [%6.1f]GFlop/s  (%6.4f)ms\n", gflops / t, t * 1000);            // line format of :600-601
  hipFree(da); hipFree(db); hipFree(dc);
  if (check) {
    const int cm = m < 1024 ? m : 1024, cn = n < 1024 ? n : 1024;
    int rc = run_check(cm, cn, k, false);
    if (rc == 0) rc = run_check(cm, cn, k < 512 ? k : 512, true);
    return rc;
  }
  return 0;
}
