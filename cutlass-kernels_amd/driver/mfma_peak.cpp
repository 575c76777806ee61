// mfma_peak -- measures what the MFMA pipe of THIS board sustains, so that "% of peak" figures of the attention
// and GEMM kernels can be read against something achievable: a register-only loop of independent
// v_mfma_f32_32x32x16_f16 (or 32x32x64 fp8) instructions, no memory, no VALU, two waves per SIMD, run once with
// constant operands and once with N(0,1) operands.  On a power-limited part the second number is the real
// ceiling for dense random data: operand bit toggling costs power and the clock governor lowers the core clock
// (the tool prints the clock it observed: shader-clock ticks of s_memtime per 100 MHz tick of s_memrealtime).
//
// A second set of lines prices the other work of a real kernel in that regime: the same fp16 loop with v_fma_f32,
// v_exp_f32 and 16-byte LDS reads (conflict-free, feeding the MFMA's A operand) added per MFMA.
//
//   mfma_peak [--ms=30] [--no-mix] [--waves-per-simd=2]
//       --ms: approximate run time per measurement; --no-mix skips the second set; --waves-per-simd=1|2: 4-wave
//       workgroups per CU (the GEMM kernel runs one wave per SIMD, the attention kernels two)
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef int int8v __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define HIP_CHECK(x)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (x);                                                                     \
    if (e_ != hipSuccess) {                                                                  \
      fprintf(stderr, "HIP error: %s (%s:%d)\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      return 2;                                                                              \
    }                                                                                        \
  } while (0)

// FP8 = false: fp16 32x32x16 (SMALL: 16x16x32); true: e4m3 32x32x64 (SMALL: 16x16x128).  The small shapes do half
// the FLOP per instruction in half the passes.  `data` holds 4096 operand dwords per variant.
template <bool FP8, bool SMALL>
__global__ void __launch_bounds__(256) mfma_loop(float *out, int iters, long long *clk, const int *data) {
  f32x16 c[4];
  f32x4 c4[8];  // eight independent chains: the 4-pass shapes have twice the issue rate per dependent chain
  for (int i = 0; i < 4; ++i)
    for (int v = 0; v < 16; ++v) c[i][v] = 0.f;
  for (int i = 0; i < 8; ++i)
    for (int v = 0; v < 4; ++v) c4[i][v] = 0.f;
  int8v a[4], b[4];
  for (int u = 0; u < 4; ++u)
    for (int t = 0; t < 8; ++t) {
      a[u][t] = data[(threadIdx.x * 131 + u * 17 + t * 7 + blockIdx.x) & 4095];
      b[u][t] = data[(threadIdx.x * 37 + u * 29 + t * 3 + 1000 + blockIdx.x) & 4095];
    }
  const long long t0 = clock64(), w0 = wall_clock64();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      if (FP8) {
        if (SMALL)
          c4[u % 8] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[u % 4], b[(u + 1) % 4], c4[u % 8], 0, 0, 0, 0, 0, 0);
        else
          c[u % 4] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[u % 4], b[(u + 1) % 4], c[u % 4], 0, 0, 0, 0, 0, 0);
      } else {
        half8 ha, hb;
        __builtin_memcpy(&ha, &a[u % 4], 16);
        __builtin_memcpy(&hb, &b[(u + 1) % 4], 16);
        // written out so that the accumulator is updated in place (through the builtin the register allocator
        // rotates the eight small accumulators through copies, 56 moves per 16 multiplies)
        if (SMALL) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c4[u % 8]) : "v"(ha), "v"(hb));
        else c[u % 4] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ha, hb, c[u % 4], 0, 0, 0);
      }
    }
  }
  const long long t1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int v = 0; v < 16; ++v) s += c[i][v];
  for (int i = 0; i < 8; ++i)
    for (int v = 0; v < 4; ++v) s += c4[i][v];
  if (s == 12345.678f) out[0] = s;  // keeps the loop alive
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    clk[0] = t1 - t0;
    clk[1] = w1 - w0;
  }
}

typedef int int4v __attribute__((ext_vector_type(4)));

// The fp16 32x32x16 loop plus, per MFMA: NV v_fma_f32, NE v_exp_f32 and NL ds_read_b128 (one wave-wide read of
// 1 KB, conflict-free).  The first read of each MFMA supplies its A operand, further ones are only waited for.
// The LDS base alternates with the outer iteration so that the reads stay in the loop; they are ordinary loads the
// compiler schedules and waits for.  One 4-wave workgroup holds 32 KB of LDS.
template <int NV, int NE, int NL>
__global__ void __launch_bounds__(256) mix_loop(float *out, int iters, long long *clk, const int *data) {
  __shared__ __attribute__((aligned(16))) int lds[8192];
  for (int i = threadIdx.x; i < 8192; i += 256) lds[i] = data[(i * 13 + blockIdx.x) & 4095];
  __syncthreads();
  f32x16 c[4];
  for (int i = 0; i < 4; ++i)
    for (int v = 0; v < 16; ++v) c[i][v] = 0.f;
  int8v a[4], b[4];
  for (int u = 0; u < 4; ++u)
    for (int t = 0; t < 8; ++t) {
      a[u][t] = data[(threadIdx.x * 131 + u * 17 + t * 7 + blockIdx.x) & 4095];
      b[u][t] = data[(threadIdx.x * 37 + u * 29 + t * 3 + 1000 + blockIdx.x) & 4095];
    }
  float x[8];
  for (int t = 0; t < 8; ++t) x[t] = (float)((data[(threadIdx.x * 8 + t) & 4095] >> 7) & 255) * (1.f / 256.f) - 0.5f;
  const int lane_dw = (threadIdx.x & 63) * 4;  // dword index of this lane's 16 bytes within a 1 KB row
  const long long t0 = clock64(), w0 = wall_clock64();
  for (int i = 0; i < iters; ++i) {
    const int4v *row = reinterpret_cast<const int4v *>(lds + (i & 1) * 4096 + lane_dw);  // 16 rows of 1 KB
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      half8 ha, hb;
      __builtin_memcpy(&ha, &a[u % 4], 16);
      __builtin_memcpy(&hb, &b[(u + 1) % 4], 16);
#pragma unroll
      for (int w = 0; w < NL; ++w) {
        const int4v d = row[((u * NL + w) % 16) * 64];
        if (w == 0) __builtin_memcpy(&ha, &d, 16);
        else asm volatile("" ::"v"(d));
      }
      c[u % 4] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ha, hb, c[u % 4], 0, 0, 0);
#pragma unroll
      for (int w = 0; w < NV; ++w) {
        const int k = (u * NV + w) % 8;
        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[k]) : "v"(x[(k + 3) % 8]), "v"(x[(k + 5) % 8]));
      }
#pragma unroll
      for (int w = 0; w < NE; ++w) {
        const int k = (u * NE + w + 1) % 8;
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[k]));
      }
    }
    if (NV + NE > 0) {  // keeps the VALU operands bounded and toggling
#pragma unroll
      for (int t = 0; t < 8; ++t) x[t] = __builtin_amdgcn_fractf(x[t]) - 0.5f;
    }
  }
  const long long t1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int v = 0; v < 16; ++v) s += c[i][v];
  for (int t = 0; t < 8; ++t) s += x[t];
  if (s == 12345.678f) out[0] = s;
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    clk[0] = t1 - t0;
    clk[1] = w1 - w0;
  }
}

static uint8_t e4m3_of(float x) {  // coarse encoder, good enough for operand statistics
  const uint8_t sign = x < 0 ? 0x80 : 0;
  float ax = std::fabs(x);
  if (ax < std::ldexp(1.f, -9)) return sign;
  if (ax > 448.f) ax = 448.f;
  int e;
  const float f = std::frexp(ax, &e);  // ax = f * 2^e, f in [0.5,1)
  int exp = e - 1 + 7;
  if (exp < 1) return sign | (uint8_t)std::lround(ax * 512.f);
  int mant = (int)std::lround((f * 2.f - 1.f) * 8.f);
  if (mant == 8) { mant = 0; ++exp; }
  if (exp > 15 || (exp == 15 && mant == 7)) { exp = 15; mant = 6; }
  return sign | (uint8_t)((exp << 3) | mant);
}

typedef void (*loop_kernel)(float *, int, long long *, const int *);

static int g_waves_per_simd = 2;

static int measure_kernel(loop_kernel kern, double flop_per_mfma, const char *label, const int *ddata, double target_ms, int cus) {
  float *dout;
  long long *dclk;
  HIP_CHECK(hipMalloc(&dout, 4));
  HIP_CHECK(hipMalloc(&dclk, 16));
  const int grid = cus * g_waves_per_simd;  // 4-wave workgroups: one per CU and wave per SIMD
  int iters = 2000;
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  float ms = 0.f;
  for (int pass = 0; pass < 3; ++pass) {  // pass 0 sizes the run, pass 1 settles the clock, pass 2 is reported
    HIP_CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), 0, 0, dout, iters, dclk, ddata);
    HIP_CHECK(hipEventRecord(e1));
    HIP_CHECK(hipEventSynchronize(e1));
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (pass == 0) iters = (int)(iters * target_ms / (ms > 1e-3f ? ms : 1e-3f)) + 1;
  }
  long long clk[2];
  HIP_CHECK(hipMemcpy(clk, dclk, 16, hipMemcpyDeviceToHost));
  const double tflops = flop_per_mfma * 16.0 * iters * grid * 4.0 / (ms * 1e-3) / 1e12;
  printf("%-44s %8.1f TFLOP/s   %7.3f ms   core clock %.3f GHz\n", label, tflops, ms, (double)clk[0] / (double)clk[1] * 0.1);
  (void)hipFree(dout);
  (void)hipFree(dclk);
  return 0;
}

template <bool FP8, bool SMALL = false>
static int measure(const char *label, const int *ddata, double target_ms, int cus) {
  return measure_kernel(mfma_loop<FP8, SMALL>, (FP8 ? 2.0 * 32 * 32 * 64 : 2.0 * 32 * 32 * 16) / (SMALL ? 2 : 1), label, ddata, target_ms, cus);
}

// one line with constant and one with N(0,1) operands
template <int NV, int NE, int NL>
static int measure_mix(const char *what, const int *d_const, const int *d_rand, double target_ms, int cus) {
  char label[96];
  snprintf(label, sizeof label, "%s, constant", what);
  if (measure_kernel(mix_loop<NV, NE, NL>, 2.0 * 32 * 32 * 16, label, d_const, target_ms, cus)) return 2;
  snprintf(label, sizeof label, "%s, N(0,1)", what);
  return measure_kernel(mix_loop<NV, NE, NL>, 2.0 * 32 * 32 * 16, label, d_rand, target_ms, cus);
}

int main(int argc, char **argv) {
  double target_ms = 30.0;
  bool mix = true;
  for (int i = 1; i < argc; ++i) {
    if (!strncmp(argv[i], "--ms=", 5)) target_ms = atof(argv[i] + 5);
    if (!strcmp(argv[i], "--no-mix")) mix = false;
    if (!strncmp(argv[i], "--waves-per-simd=", 17)) g_waves_per_simd = atoi(argv[i] + 17) < 1 ? 1 : atoi(argv[i] + 17) > 4 ? 4 : atoi(argv[i] + 17);
  }
  hipDeviceProp_t prop;
  HIP_CHECK(hipGetDeviceProperties(&prop, 0));
  printf("device: %s, %d CUs, nominal clock %.2f GHz, %d wave(s) per SIMD\n", prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1e6,
         g_waves_per_simd);
  std::mt19937 gen(3081);
  std::normal_distribution<float> nd(0.f, 1.f);
  std::vector<int> h_const16(4096), h_rand16(4096), h_const8(4096), h_rand8(4096);
  for (int i = 0; i < 4096; ++i) {
    _Float16 one = (_Float16)1.0f, pair[2] = {(_Float16)nd(gen), (_Float16)nd(gen)};
    uint16_t ob, pb[2];
    memcpy(&ob, &one, 2);
    memcpy(pb, pair, 4);
    h_const16[i] = ob | (ob << 16);
    h_rand16[i] = pb[0] | (pb[1] << 16);
    h_const8[i] = 0x38383838;  // 1.0 in e4m3
    uint32_t w = 0;
    for (int t = 0; t < 4; ++t) w |= (uint32_t)e4m3_of(nd(gen) * 64.f) << (8 * t);  // N(0,1) scaled as amax/448 would
    h_rand8[i] = (int)w;
  }
  int *d;
  HIP_CHECK(hipMalloc(&d, 4 * 4096 * 4));
  HIP_CHECK(hipMemcpy(d, h_const16.data(), 16384, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d + 4096, h_rand16.data(), 16384, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d + 8192, h_const8.data(), 16384, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d + 12288, h_rand8.data(), 16384, hipMemcpyHostToDevice));
  const int cus = prop.multiProcessorCount;
  if (measure<false>("fp16 32x32x16, constant operands", d, target_ms, cus)) return 2;
  if (measure<false>("fp16 32x32x16, N(0,1) operands", d + 4096, target_ms, cus)) return 2;
  if (measure<true>("fp8 e4m3 32x32x64, constant operands", d + 8192, target_ms, cus)) return 2;
  if (measure<true>("fp8 e4m3 32x32x64, N(0,1)*64 operands", d + 12288, target_ms, cus)) return 2;
  if (measure<false>("fp16 32x32x16, N(0,1) operands (repeat)", d + 4096, target_ms, cus)) return 2;
  if (measure<false, true>("fp16 16x16x32, constant operands", d, target_ms, cus)) return 2;
  if (measure<false, true>("fp16 16x16x32, N(0,1) operands", d + 4096, target_ms, cus)) return 2;
  if (measure<true, true>("fp8 e4m3 16x16x128, constant operands", d + 8192, target_ms, cus)) return 2;
  if (measure<true, true>("fp8 e4m3 16x16x128, N(0,1)*64 operands", d + 12288, target_ms, cus)) return 2;
  if (measure<false>("fp16 32x32x16, N(0,1) operands (repeat)", d + 4096, target_ms, cus)) return 2;
  if (!mix) return 0;
  printf("fp16 32x32x16 plus other work per MFMA:\n");
  const int *dc = d, *dr = d + 4096;
  if (measure_mix<0, 0, 0>("  nothing", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<2, 0, 0>("  2 v_fma", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<4, 0, 0>("  4 v_fma", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<2, 1, 0>("  2 v_fma + 1 v_exp", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<0, 0, 1>("  1 ds_read_b128 (as A)", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<0, 0, 2>("  2 ds_read_b128", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<2, 1, 1>("  2 v_fma + 1 v_exp + 1 ds_read_b128", dc, dr, target_ms, cus)) return 2;
  if (measure_mix<0, 0, 0>("  nothing (repeat)", dc, dr, target_ms, cus)) return 2;
  return 0;
}
