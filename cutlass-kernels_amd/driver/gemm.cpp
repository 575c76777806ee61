// gemm -- bench/test driver for cfk_gemm with the command lines and output lines of the reference's two GEMM examples.
//
//   gemm <type> [M] [N] [K] [L] [check]        the CuTe example (src/cute-gemm-tma-gma/gemm.cu:469-691)
//     type 1 = float operands, 3 = half (:677-684; 2 is commented out there and rejected here); M N K default
//     5120 5120 4096 (:668-678); L = batch count, packed strides (:519-521); "check" verifies.
//     A is M x K, B is N x K, both K-contiguous, values 2*rand()/RAND_MAX - 1 (:482-485), C preset to -1, alpha = 1,
//     beta = 0 (:495-496).  The reference compares bitwise with cuBLAS (:645-651); without cuBLAS here the check is a
//     naive fp32 GPU GEMM of the same operands (|c - ref| <= 2e-3 |ref| + 1e-2 for half, 1e-4 |ref| + 2e-4 for float)
//     plus a bit-exact run on integer-valued operands.
//
//   gemm --m=<int> --n=<int> --k=<int> --alpha=<f32> --beta=<f32> --iterations=<int>
//                                               the CUTLASS-API example (src/cutlass-gemm/gemm.cu:182-236, 364-418)
//     half operands, uniform integers in [-8, 8] (:277-294), D = alpha * A.B + beta * C, checked for EQUALITY against
//     a reference GEMM (:329-359; here the naive GPU GEMM with the same fp32 epilogue), then timed; defaults
//     5120 x 4096 x 4096, alpha 1, beta 0, 1000 iterations (:190-194).
//
// C and D are row-major M x N here (column-major in the reference, gemm.cu:386-389 and cutlass-gemm/gemm.cu:96-98).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
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

// naive checker: one thread per element, fp32 accumulate with k ascending, fp32 epilogue
template <class T>
__global__ void naive_gemm_tn(const T *A, const T *B, const T *C, float *D, int M, int N, int K, float alpha, float beta) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)M * N) return;
  const int m = (int)(idx / N), n = (int)(idx % N);
  float acc = 0.f;
  for (int k = 0; k < K; ++k) acc += (float)A[(long long)m * K + k] * (float)B[(long long)n * K + k];
  D[idx] = alpha * acc + (C && beta != 0.f ? beta * (float)C[idx] : 0.f);
}

template <class T>
static int call_gemm(int m, int n, int k, int l, float alpha, float beta, const T *a, const T *b, const T *c, T *d) {
  cfk_gemm_params p{};
  p.dtype = sizeof(T) == 4 ? CFK_FP32 : CFK_FP16;
  p.layout = CFK_GEMM_TN;
  p.m = m;
  p.n = n;
  p.k = k;
  p.batch = l;
  p.alpha = alpha;
  p.beta = beta;
  p.a = a;
  p.b = b;
  p.c = c;
  p.d = d;
  if (cfk_gemm(&p, nullptr) != CFK_OK) {
    fprintf(stderr, "cfk_gemm: %s\n", cfk_last_error());
    return 2;
  }
  return 0;
}

// One problem against the naive GEMM.  integers: operands in [-8, 8] and an equality check (every partial sum is an
// integer below 2^24, so fp32 accumulation is exact in any order and the one rounding to T is the same on both sides).
template <class T>
static int run_check(int m, int n, int k, bool integers, float alpha, float beta, const char *label) {
  const size_t na = (size_t)m * k, nb = (size_t)n * k, nc = (size_t)m * n;
  std::vector<T> ha(na), hb(nb), hc(nc), hd(nc);
  srand(integers ? 7 : 1);
  auto val = [&]() { return integers ? (T)(float)(rand() % 17 - 8) : (T)(2 * (rand() / double(RAND_MAX)) - 1); };
  for (auto &x : ha) x = val();
  for (auto &x : hb) x = val();
  for (auto &x : hc) x = val();
  T *da, *db, *dc, *dd;
  float *dref;
  HIP_CHECK(hipMalloc(&da, na * sizeof(T)));
  HIP_CHECK(hipMalloc(&db, nb * sizeof(T)));
  HIP_CHECK(hipMalloc(&dc, nc * sizeof(T)));
  HIP_CHECK(hipMalloc(&dd, nc * sizeof(T)));
  HIP_CHECK(hipMalloc(&dref, nc * 4));
  HIP_CHECK(hipMemcpy(da, ha.data(), na * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(db, hb.data(), nb * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dc, hc.data(), nc * sizeof(T), hipMemcpyHostToDevice));
  if (call_gemm<T>(m, n, k, 1, alpha, beta, da, db, dc, dd)) return 2;
  hipLaunchKernelGGL(naive_gemm_tn<T>, dim3((unsigned)((nc + 255) / 256)), dim3(256), 0, 0, da, db, dc, dref, m, n, k,
                     alpha, beta);
  HIP_CHECK(hipDeviceSynchronize());
  std::vector<float> ref(nc);
  HIP_CHECK(hipMemcpy(hd.data(), dd, nc * sizeof(T), hipMemcpyDeviceToHost));
  HIP_CHECK(hipMemcpy(ref.data(), dref, nc * 4, hipMemcpyDeviceToHost));
  const float rtol = sizeof(T) == 4 ? 1e-4f : 2e-3f, atol = sizeof(T) == 4 ? 2e-4f : 1e-2f;
  long long bad = 0;
  for (size_t i = 0; i < nc; ++i) {
    const float got = (float)hd[i];
    const bool ok = integers ? (hd[i] == (T)ref[i]) : (std::fabs(got - ref[i]) <= rtol * std::fabs(ref[i]) + atol);
    if (!ok && bad++ < 5) printf("failed [%zu] %f %f\n", i, got, ref[i]);
  }
  if (label) printf("%s%s\n", label, bad ? "Failed" : "Passed");
  hipFree(da); hipFree(db); hipFree(dc); hipFree(dd); hipFree(dref);
  return bad ? 3 : 0;
}

// the CuTe example: time L packed problems, alpha = 1, beta = 0
template <class T>
static int cute_example(int m, int n, int k, int l, bool check) {
  printf("M = %d\nN = %d\nK = %d\nL = %d\n", m, n, k, l);
  const size_t na = (size_t)m * k * l, nb = (size_t)n * k * l, nc = (size_t)m * n * l;
  std::vector<T> ha(na), hb(nb), hc(nc, (T)-1.0f);
  for (auto &x : ha) x = (T)(2 * (rand() / double(RAND_MAX)) - 1);
  for (auto &x : hb) x = (T)(2 * (rand() / double(RAND_MAX)) - 1);
  T *da, *db, *dc;
  HIP_CHECK(hipMalloc(&da, na * sizeof(T)));
  HIP_CHECK(hipMalloc(&db, nb * sizeof(T)));
  HIP_CHECK(hipMalloc(&dc, nc * sizeof(T)));
  HIP_CHECK(hipMemcpy(da, ha.data(), na * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(db, hb.data(), nb * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dc, hc.data(), nc * sizeof(T), hipMemcpyHostToDevice));
  if (call_gemm<T>(m, n, k, l, 1.f, 0.f, da, db, nullptr, dc)) return 1;  // run once (:509-520)
  HIP_CHECK(hipDeviceSynchronize());
  const int timing_iterations = sizeof(T) == 4 ? 100 : 1000;  // :499 (fewer for the 16x slower fp32 MFMA)
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  HIP_CHECK(hipEventRecord(e0));
  for (int i = 0; i < timing_iterations; ++i)
    if (call_gemm<T>(m, n, k, l, 1.f, 0.f, da, db, nullptr, dc)) return 1;
  HIP_CHECK(hipEventRecord(e1));
  HIP_CHECK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  const double t = ms / 1e3 / timing_iterations, gflops = 2.0 * m * n * k * l * 1e-9;  // :498
  printf("CUTE_GEMM:     [%6.1f]GFlop/s  (%6.4f)ms\n", gflops / t, t * 1000);            // line format of :600-601
  hipFree(da); hipFree(db); hipFree(dc);
  if (check) {
    const int cm = m < 1024 ? m : 1024, cn = n < 1024 ? n : 1024;
    int rc = run_check<T>(cm, cn, k, false, 1.f, 0.f, "gemm-check (uniform operands): ");
    if (rc == 0) rc = run_check<T>(cm, cn, k < 512 ? k : 512, true, 1.f, 0.f, "gemm-check (integer operands, bit-exact): ");
    return rc;
  }
  return 0;
}

// the CUTLASS-API example: equality check of D = alpha A.B + beta C on integer operands, then the timing loop
static int cutlass_example(int m, int n, int k, float alpha, float beta, int iterations) {
  // the check runs on the problem itself when it is small, else on its leading 1024 x 1024 x min(k, 1024) corner
  const int cm = m < 1024 ? m : 1024, cn = n < 1024 ? n : 1024, ck = k < 1024 ? k : 1024;
  const int rc = run_check<_Float16>(cm, cn, ck, true, alpha, beta, nullptr);
  if (rc == 2) return 2;
  printf("  Disposition: %s\n", rc == 0 ? "Passed" : "Failed");
  if (iterations > 0) {
    const size_t na = (size_t)m * k, nb = (size_t)n * k, nc = (size_t)m * n;
    std::vector<_Float16> ha(na), hb(nb), hc(nc);
    srand(2023);
    for (auto &x : ha) x = (_Float16)(float)(rand() % 17 - 8);
    for (auto &x : hb) x = (_Float16)(float)(rand() % 17 - 8);
    for (auto &x : hc) x = (_Float16)(float)(rand() % 17 - 8);
    _Float16 *da, *db, *dc, *dd;
    HIP_CHECK(hipMalloc(&da, na * 2));
    HIP_CHECK(hipMalloc(&db, nb * 2));
    HIP_CHECK(hipMalloc(&dc, nc * 2));
    HIP_CHECK(hipMalloc(&dd, nc * 2));
    HIP_CHECK(hipMemcpy(da, ha.data(), na * 2, hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(db, hb.data(), nb * 2, hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dc, hc.data(), nc * 2, hipMemcpyHostToDevice));
    if (call_gemm<_Float16>(m, n, k, 1, alpha, beta, da, db, dc, dd)) return 1;  // warm-up (:385)
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    HIP_CHECK(hipEventRecord(e0));
    for (int i = 0; i < iterations; ++i)
      if (call_gemm<_Float16>(m, n, k, 1, alpha, beta, da, db, dc, dd)) return 1;
    HIP_CHECK(hipEventRecord(e1));
    HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double avg_ms = ms / iterations;
    printf("  Problem Size: %dx%dx%d\n", m, n, k);  // :411-413
    printf("  Avg runtime: %g ms\n", avg_ms);
    printf("  GFLOPS: %g\n", 2.0 * m * n * k / 1e9 / (avg_ms / 1e3));
    hipFree(da); hipFree(db); hipFree(dc); hipFree(dd);
  }
  return rc;
}

int main(int argc, char **argv) {
  if (argc >= 2 && !strncmp(argv[1], "--", 2)) {  // the CUTLASS-API example's options
    int m = 5120, n = 4096, k = 4096, iterations = 1000;
    float alpha = 1.f, beta = 0.f;
    for (int i = 1; i < argc; ++i) {
      const std::string a = argv[i];
      const size_t eq = a.find('=');
      const std::string key = a.substr(2, eq == std::string::npos ? std::string::npos : eq - 2);
      const char *val = eq == std::string::npos ? "" : argv[i] + eq + 1;
      if (key == "help") {
        printf("gemm --m=<int> --n=<int> --k=<int> --alpha=<f32> --beta=<f32> --iterations=<int>\n"
               "gemm <type: 1 float | 3 half> [M] [N] [K] [L] [check]\n");
        return 0;
      } else if (key == "m") m = atoi(val);
      else if (key == "n") n = atoi(val);
      else if (key == "k") k = atoi(val);
      else if (key == "alpha") alpha = (float)atof(val);
      else if (key == "beta") beta = (float)atof(val);
      else if (key == "iterations") iterations = atoi(val);
      else { printf("unknown option %s\n", argv[i]); return 1; }
    }
    return cutlass_example(m, n, k, alpha, beta, iterations);
  }
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
  if (l < 1) l = 1;
  if (type == 1) return cute_example<float>(m, n, k, l, check);
  if (type == 3) return cute_example<_Float16>(m, n, k, l, check);
  printf("invalid type value (1 | 3 are the only legal values)\n");  // :686-688
  return 1;
}
