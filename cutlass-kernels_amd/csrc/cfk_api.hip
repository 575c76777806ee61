// C-ABI of libcfk_fmha.so (declared in include/cfk_fmha.h): argument validation, kernel selection, launch.
// Host-side counterpart of fmhaForwardDevice (src/fmha-pipeline/fmha_forward.cu:86-383): where the reference
// builds TMA descriptors and picks a kernel by compile-time macros, this layer checks the run-time shape
// against the tile plan and dispatches to a gfx950 instantiation.
#include "../../include/cfk_fmha.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "fmha_common.h"

namespace {

thread_local char g_err[512] = "";
std::atomic<int> g_predictable{0}, g_fast_e4m3{0};

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Shape / enum checks shared by the plan query and the launch.  Fills `plan`.
int check_fmha(const cfk_fmha_fwd_params *p, cfk::FmhaPlan *plan, bool need_pointers) {
  if (!p) return fail(CFK_ERR_INVALID_ARG, "params is NULL");
  if (p->dtype != CFK_FP16 && p->dtype != CFK_FP8_E4M3)
    return fail(CFK_ERR_INVALID_ARG, "Unsupported type: %d (1 = fp16, 2 = fp8 e4m3)", p->dtype);
  if (p->v_dtype != CFK_FP16 && p->v_dtype != CFK_FP8_E4M3)
    return fail(CFK_ERR_INVALID_ARG, "Unsupported V type: %d", p->v_dtype);
  if (p->batch <= 0 || p->heads <= 0 || p->seqlen_q <= 0 || p->seqlen_kv <= 0)
    return fail(CFK_ERR_INVALID_ARG, "batch, heads, seqlen_q, seqlen_kv must be positive (got %d, %d, %d, %d)",
                p->batch, p->heads, p->seqlen_q, p->seqlen_kv);
  if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256)
    return fail(CFK_ERR_UNSUPPORTED, "Unsupported head dim: %d", p->head_dim);
  if (p->v_layout != CFK_V_BSHD && p->v_layout != CFK_V_BDHS)
    return fail(CFK_ERR_INVALID_ARG, "unknown v_layout %d", p->v_layout);
  if (p->dtype == CFK_FP16 && p->v_dtype != CFK_FP16)
    return fail(CFK_ERR_UNSUPPORTED, "fp16 Q,K with fp8 V is not a mode of the reference; v_dtype must be fp16");
  if (p->v_dtype == CFK_FP16 && p->v_layout != CFK_V_BSHD)
    return fail(CFK_ERR_UNSUPPORTED, "pre-transposed V ([B,D,H,S]) is an fp8-V layout");
  if (!(p->softmax_scale > 0.f) || !std::isfinite(p->softmax_scale))
    return fail(CFK_ERR_INVALID_ARG, "softmax_scale must be positive and finite");
  if (p->dtype == CFK_FP8_E4M3) {
    const float d[3] = {p->q_descale, p->k_descale, p->v_dtype == CFK_FP8_E4M3 ? p->v_descale : 1.0f};
    for (float x : d)
      if (!(x > 0.f) || !std::isfinite(x)) return fail(CFK_ERR_INVALID_ARG, "fp8 descales must be positive and finite");
  }
  const long long bh = (long long)p->batch * p->heads;
  if (bh > (1 << 24)) return fail(CFK_ERR_UNSUPPORTED, "batch*heads too large");
  const bool tap = p->dbg_s != nullptr;
  bool ok = p->dtype == CFK_FP16     ? cfk::plan_fmha_f16(p->head_dim, p->seqlen_q, p->seqlen_kv, (int)bh, tap, plan)
            : p->v_dtype == CFK_FP16 ? cfk::plan_fmha_hybrid(p->head_dim, p->seqlen_q, p->seqlen_kv, (int)bh, tap, plan)
                                     : cfk::plan_fmha_fp8(p->head_dim, p->seqlen_q, p->seqlen_kv, (int)bh, p->v_layout, tap, plan);
  if (!ok) return fail(CFK_ERR_UNSUPPORTED, "no kernel for dtype %d head dim %d v_layout %d", p->dtype, p->head_dim, p->v_layout);
  // The kernels carry no masks, exactly like the reference (no bounds handling: fmha_forward.cu:361-372).
  if (p->seqlen_q % plan->q_multiple != 0)
    return fail(CFK_ERR_UNSUPPORTED, "seqlen_q %d is not a multiple of %d (query tile %d)", p->seqlen_q, plan->q_multiple, plan->block_m);
  if (p->seqlen_kv % plan->kv_multiple != 0)
    return fail(CFK_ERR_UNSUPPORTED, "seqlen_kv %d is not a multiple of the key tile %d", p->seqlen_kv, plan->kv_multiple);
  const long long elems = bh * (long long)(p->seqlen_q > p->seqlen_kv ? p->seqlen_q : p->seqlen_kv) * p->head_dim;
  if (elems >= (1LL << 40)) return fail(CFK_ERR_UNSUPPORTED, "tensor too large");
  // the kernels address one batch slice with 32-bit byte offsets
  if ((long long)(p->seqlen_q > p->seqlen_kv ? p->seqlen_q : p->seqlen_kv) * p->heads * p->head_dim * 2 >= (1LL << 31))
    return fail(CFK_ERR_UNSUPPORTED, "seqlen * heads * head_dim * 2 bytes must stay below 2 GiB per batch entry");
  if (need_pointers && (!p->q || !p->k || !p->v || !p->o))
    return fail(CFK_ERR_INVALID_ARG, "q, k, v, o must be non-NULL device pointers");
  return CFK_OK;
}

int check_device() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(CFK_ERR_NO_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  static thread_local int checked_dev = -1;
  if (checked_dev == dev) return CFK_OK;
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail(CFK_ERR_HIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(CFK_ERR_NO_DEVICE, "device %d is %s; this library is built for gfx950 only", dev, prop.gcnArchName);
  checked_dev = dev;
  return CFK_OK;
}

}  // namespace

namespace cfk {
bool predictable_latency() { return g_predictable.load(std::memory_order_relaxed) != 0; }
bool fast_e4m3_weights() { return g_fast_e4m3.load(std::memory_order_relaxed) != 0; }
}  // namespace cfk

extern "C" {

int cfk_fmha_forward_plan(const cfk_fmha_fwd_params *params, int32_t *block_m, int32_t *block_n, int32_t *lds_bytes,
                          int32_t *threads) {
  cfk::FmhaPlan plan{};
  int rc = check_fmha(params, &plan, false);
  if (rc != CFK_OK) return rc;
  if (block_m) *block_m = plan.block_m;
  if (block_n) *block_n = plan.block_n;
  if (lds_bytes) *lds_bytes = plan.lds_bytes;
  if (threads) *threads = plan.threads;
  return CFK_OK;
}

int cfk_fmha_forward_mfma(const cfk_fmha_fwd_params *params, int32_t *mfma_rows) {
  cfk::FmhaPlan plan{};
  int rc = check_fmha(params, &plan, false);
  if (rc != CFK_OK) return rc;
  if (mfma_rows) *mfma_rows = plan.mfma;
  return CFK_OK;
}

int cfk_fmha_forward_kernel(const cfk_fmha_fwd_params *params, char *name, int32_t capacity) {
  cfk::FmhaPlan plan{};
  int rc = check_fmha(params, &plan, false);
  if (rc != CFK_OK) return rc;
  if (!name || capacity <= (int32_t)strlen(plan.kernel)) return fail(CFK_ERR_INVALID_ARG, "name buffer of %d bytes is too small", capacity);
  memcpy(name, plan.kernel, strlen(plan.kernel) + 1);
  return CFK_OK;
}

int cfk_fmha_forward(const cfk_fmha_fwd_params *p, void *stream) {
  cfk::FmhaPlan plan{};
  int rc = check_fmha(p, &plan, true);
  if (rc != CFK_OK) return rc;
  rc = check_device();
  if (rc != CFK_OK) return rc;
  constexpr float kLog2e = 1.4426950408889634074f;  // fmha_forward.cu:452
  cfk::FmhaArgs a{};
  a.q = p->q;
  a.k = p->k;
  a.v = p->v;
  a.o = p->o;
  a.s_tap = p->dbg_s;
  a.row_max = p->dbg_row_max;
  a.row_sum = p->dbg_row_sum;
  a.B = p->batch;
  a.H = p->heads;
  a.Sq = p->seqlen_q;
  a.Skv = p->seqlen_kv;
  a.v_layout = p->v_layout;
  // Deferred rescale: O and l are only rescaled when a tile's max exceeds the max the reference point was set from by
  // more than tau (log2 domain).  fp16 P: 2^8 of head-room.  e4m3 P already sits 2^7 above the reference point, which
  // leaves 1.  With e4m3 P the row's largest weight is an exact power of two only while the reference point follows
  // the running max (as the reference's does on every tile, online_softmax.h:144-165); the rounding error of that
  // weight (<= 6 %) averages out over long key sequences but shows in the reference's error-percentage measure on short
  // ones, so those run with tau = 0.
  a.tau = p->v_dtype != CFK_FP8_E4M3 ? 8.0f : p->seqlen_kv < 2048 ? 0.0f : 1.0f;
  // e4m3 P: in the pass without a row max per tile the reference point comes from the first tile, so a row's largest
  // weight is not the exact power of two it is under a running max, and over few keys the rounding of that weight shows in
  // the reference's error-percentage gate (fmha_forward.cu:638-639, limit 0.001 %): 0.0000 % over the 4096 keys of the
  // reference's own problem, 0.00001..0.00006 % at 3072 and 3584 keys, 0.0001..0.0003 % at 2560, 0.0005..0.0013 % at 2048
  // (head dims 128, 256, 64).  Key lengths below 3072 take the max-tracking pass only.
  a.direct_p = g_fast_e4m3.load(std::memory_order_relaxed);
  a.track_only = cfk::predictable_latency() || (p->v_dtype == CFK_FP8_E4M3 && p->seqlen_kv < 3072) ? 1 : 0;
  hipError_t e;
  a.s_scale = p->dtype == CFK_FP16 ? p->softmax_scale : p->softmax_scale * p->q_descale * p->k_descale;
  if (p->dtype == CFK_FP16) {
    a.scale_log2 = p->softmax_scale * kLog2e;
    a.out_scale = 1.0f;
    e = cfk::launch_fmha_f16(a, p->head_dim, (hipStream_t)stream);
  } else if (p->v_dtype == CFK_FP16) {  // hybrid: fp16 V carries no scale
    a.scale_log2 = p->softmax_scale * kLog2e * p->q_descale * p->k_descale;
    a.out_scale = 1.0f;
    e = cfk::launch_fmha_hybrid(a, p->head_dim, (hipStream_t)stream);
  } else {
    a.scale_log2 = p->softmax_scale * kLog2e * p->q_descale * p->k_descale;
    a.out_scale = p->v_descale;
    e = cfk::launch_fmha_fp8(a, p->head_dim, (hipStream_t)stream);
  }
  if (e != hipSuccess) return fail(CFK_ERR_HIP, "FMHA launch failed: %s", hipGetErrorString(e));
  return CFK_OK;
}

int cfk_set_option(int32_t option, int32_t value) {
  if (option == CFK_OPT_PREDICTABLE_LATENCY) g_predictable.store(value != 0, std::memory_order_relaxed);
  else if (option == CFK_OPT_FAST_E4M3_WEIGHTS) g_fast_e4m3.store(value != 0, std::memory_order_relaxed);
  else return fail(CFK_ERR_INVALID_ARG, "unknown option %d", option);
  return CFK_OK;
}

int cfk_gemm(const cfk_gemm_params *p, void *stream) {
  if (!p) return fail(CFK_ERR_INVALID_ARG, "params is NULL");
  if (p->dtype != CFK_FP16 && p->dtype != CFK_FP32)
    return fail(CFK_ERR_INVALID_ARG, "GEMM dtype must be CFK_FP16 or CFK_FP32 (got %d)", p->dtype);
  if (p->m <= 0 || p->n <= 0 || p->k <= 0 || p->batch <= 0)
    return fail(CFK_ERR_INVALID_ARG, "M, N, K, batch must be positive (got %d, %d, %d, %d)", p->m, p->n, p->k, p->batch);
  if (!p->a || !p->b || !p->d) return fail(CFK_ERR_INVALID_ARG, "A, B, D must be non-NULL device pointers");
  if (p->layout != CFK_GEMM_TN && p->layout != CFK_GEMM_NN)
    return fail(CFK_ERR_INVALID_ARG, "unknown GEMM layout %d", p->layout);
  if (p->dtype == CFK_FP32 && p->layout != CFK_GEMM_TN)
    return fail(CFK_ERR_UNSUPPORTED, "fp32 GEMM is built for the TN layout only");
  if (p->m % 256 || p->n % 256 || p->k % 64)
    return fail(CFK_ERR_UNSUPPORTED, "M and N must be multiples of 256 and K of 64 (got %d, %d, %d)", p->m, p->n, p->k);
  if (p->batch > 65535) return fail(CFK_ERR_UNSUPPORTED, "batch must be <= 65535 (got %d)", p->batch);
  // the kernel addresses a 256-row tile of A / B (TN) and a 64-row K-slab of B (NN) with 32-bit byte offsets
  const long long esz = p->dtype == CFK_FP32 ? 4 : 2;
  if (256LL * p->k * esz >= (1LL << 32))
    return fail(CFK_ERR_UNSUPPORTED, "K too large: 256 * K * element size must stay below 4 GiB (K = %d)", p->k);
  if (p->layout == CFK_GEMM_NN && 64LL * p->n * 2 >= (1LL << 32))
    return fail(CFK_ERR_UNSUPPORTED, "N too large for the NN layout: 64 * N * 2 must stay below 4 GiB (N = %d)", p->n);
  int rc = check_device();
  if (rc != CFK_OK) return rc;
  cfk::GemmArgs g{};
  g.A = p->a;
  g.B = p->b;
  g.C = p->c;
  g.D = p->d;
  g.M = p->m;
  g.N = p->n;
  g.K = p->k;
  g.batch = p->batch;
  g.layout = p->layout;
  g.f32 = p->dtype == CFK_FP32;
  g.alpha = p->alpha;
  g.beta = p->beta;
  hipError_t e = cfk::launch_gemm(g, (hipStream_t)stream);
  if (e == hipErrorNotSupported) return fail(CFK_ERR_UNSUPPORTED, "GEMM dtype %d / layout %d is not built", p->dtype, p->layout);
  if (e != hipSuccess) return fail(CFK_ERR_HIP, "GEMM launch failed: %s", hipGetErrorString(e));
  return CFK_OK;
}

int cfk_gemm_f16(int32_t M, int32_t N, int32_t K, const void *A, const void *B, void *C, int32_t layout, void *stream) {
  if (!C) return fail(CFK_ERR_INVALID_ARG, "A, B, C must be non-NULL device pointers");
  cfk_gemm_params p{};
  p.dtype = CFK_FP16;
  p.layout = layout;
  p.m = M;
  p.n = N;
  p.k = K;
  p.batch = 1;
  p.alpha = 1.0f;
  p.beta = 0.0f;
  p.a = A;
  p.b = B;
  p.c = nullptr;
  p.d = C;
  return cfk_gemm(&p, stream);
}

int cfk_init(void) {
  int rc = check_device();
  if (rc != CFK_OK) return rc;
  hipError_t e = cfk::prepare_fmha_f16();
  if (e == hipSuccess) e = cfk::prepare_fmha_fp8();
  if (e == hipSuccess) e = cfk::prepare_fmha_hybrid();
  if (e == hipSuccess) e = cfk::prepare_gemm();
  if (e != hipSuccess) return fail(CFK_ERR_HIP, "kernel set-up failed: %s", hipGetErrorString(e));
  return CFK_OK;
}

const char *cfk_last_error(void) { return g_err; }

const char *cfk_version(void) { return "cfk-mi355x 0.2 gfx950"; }

}  // extern "C"
