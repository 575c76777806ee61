/*
 * cfk_fmha.h -- C-ABI of libcfk_fmha.so: fused multi-head-attention forward (fp16 and fp8 e4m3) and the
 * dense GEMM examples (fp16 / fp32 operands) for AMD Instinct MI355X (gfx950).
 *
 * The reference repository (ColfaxResearch/cutlass-kernels) has no FFI: its hot path sits behind the C++
 * template fmhaForwardDevice<PrecType, Gemm2Type, SoftType, OutputType, HEADDIM>
 * (src/fmha-pipeline/fmha_forward.cu:86-93), called by its driver through fmhaForwardDeviceLoop
 * (src/fmha-pipeline/fmha_forward.cu:387-419, call sites :578-592).  The entry points below carry that same
 * contract over plain pointers and sizes so that a driver written against the reference's host function can
 * call HIP where it called CUDA.
 *
 * All pointers are DEVICE pointers owned by the caller; nothing is allocated, freed or retained by the
 * library; every call is asynchronous on `stream` (a hipStream_t passed as void*, NULL = default stream).
 * Functions return CFK_OK (0) or a negative cfk_status; cfk_last_error() holds a message for the calling
 * thread's last failure.  The library never calls exit() (the reference does, :758-760).
 */
#ifndef CFK_FMHA_H_
#define CFK_FMHA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum cfk_status {
  CFK_OK = 0,
  CFK_ERR_INVALID_ARG = -1, /* null pointer, non-positive size, unknown enum value            */
  CFK_ERR_UNSUPPORTED = -2, /* head dim / precision / layout / tile divisibility not supported */
  CFK_ERR_HIP = -3,         /* a HIP runtime call failed (message names it)                    */
  CFK_ERR_NO_DEVICE = -4    /* no gfx950 device is current                                     */
} cfk_status;

/* Operand precision; values mirror the driver flag --prec-type (src/fmha-pipeline/fmha_forward.cu:694,733). */
typedef enum cfk_dtype { CFK_FP16 = 1, CFK_FP8_E4M3 = 2, CFK_FP32 = 3 /* GEMM only */ } cfk_dtype;

/* Layout of V in memory.  Not accepted: the reference's third convention, -DFP8NOSHFL (fmha_forward.cu:534-558), which
 * additionally permutes V's sequence index inside every block of 16 on the host so that its kernel needs no register
 * shuffles.  The kernels here need neither the shuffles nor the permutation (the key order of P is applied where V is
 * read from the LDS): a caller that keeps that host permutation must drop it, or O comes out wrong. */
typedef enum cfk_v_layout {
  CFK_V_BSHD = 0, /* [B, S_kv, H, D], D contiguous -- the reference's default (fmha_forward.cu:189-190)       */
  CFK_V_BDHS = 1  /* [B, D, H, S_kv], S contiguous -- the reference's offline pre-transposed fp8 V (GEMM2FP8,
                     fmha_forward.cu:231-232, 514-532); accepted for fp8 only                                   */
} cfk_v_layout;

/*
 * Arguments of one forward call.  Replaces the argument list of fmhaForwardDevice
 * (src/fmha-pipeline/fmha_forward.cu:88-93): SEQLEN, KEYLEN, NUMHEADS, BATCH, tensorQ/K/V, tensorS, tensorO,
 * miOut, sPrimeOut, scale, stream; HEADDIM and the precisions are run-time fields here instead of template
 * parameters.  The reference's `iterations` argument (a launch loop inside the entry) is the caller's loop here.
 */
typedef struct cfk_fmha_fwd_params {
  int32_t dtype;     /* cfk_dtype of Q and K                                                                  */
  int32_t v_dtype;   /* cfk_dtype of V (and of P).  Equal to dtype, or CFK_FP16 with dtype = CFK_FP8_E4M3: the
                        reference's hybrid mode, fp8 Q,K with fp16 P,V -- what its --prec-type=2 computes when built
                        without -DGEMM2FP8 (fmha_forward.cu:446-450)                                            */
  int32_t batch;     /* BATCH                                                                                 */
  int32_t heads;     /* NUMHEADS                                                                              */
  int32_t seqlen_q;  /* SEQLEN: multiple of 32; a last query tile (128 or 256 rows) may be filled to a whole number
                        of 32-row waves (the reference: whole tiles of its compile-time 64 or 128 rows,
                        shared_storage.h:4-15)                                                                */
  int32_t seqlen_kv; /* KEYLEN: multiple of 64 (32 for fp16 V at head_dim 256); cfk_fmha_forward_plan reports the
                        key tile actually chosen                                                              */
  int32_t head_dim;  /* HEADDIM: 64, 128 or 256 (fmha_forward.cu:746-761)                                     */
  int32_t v_layout;  /* cfk_v_layout                                                                          */
  const void *q;     /* [B, S_q,  H, D] dtype, D contiguous (fmha_forward.cu:151-152)                         */
  const void *k;     /* [B, S_kv, H, D] dtype               (fmha_forward.cu:162-163)                         */
  const void *v;     /* v_layout, v_dtype                                                                     */
  void *o;           /* [B, S_q, H, D] fp16, always (fmha_forward.cu:245-246, 471)                            */
  float softmax_scale; /* natural-domain scale, normally 1/sqrt(D); the library multiplies by log2(e) itself.
                          (The reference passes scale*log2e, fmha_forward.cu:452-454.)                        */
  float q_descale;   /* fp8 per-tensor scales: real value = code value * descale.  1.0f reproduces the        */
  float k_descale;   /* reference, which applies no scaling (fmha_forward.cu:498-500).  Ignored for fp16.     */
  float v_descale;   /* ignored when v_dtype is CFK_FP16                                                      */
  float *dbg_s;       /* optional tap, [B, H, S_q, S_kv] fp32: pre-softmax scores softmax_scale * Q K^T (natural
                         domain, fp8 descales applied) -- the reference's tensorS under COPYOUTMM0
                         (fmha_consumer.h:31-42), which it scales on the host before gemm-check-1
                         (fmha_forward.cu:640-653).  Selects a debug build of the kernel (128-row tile); NULL = off */
  float *dbg_row_max; /* optional tap, [B, H, S_q] fp32: running row max in the log2 domain (score*scale*log2e),
                         the reference's miOut under COPYOUTMI (fmha_epilogue.h:7-46); NULL = off              */
  float *dbg_row_sum; /* optional tap, [B, H, S_q] fp32: row sum of exp2(t - max), not its reciprocal, the
                         reference's sPrimeOut (fmha_forward.cu:668-672); NULL = off.  The sum is taken over the
                         weights AS ROUNDED to the precision of P (fp16, or e4m3 for v_dtype = CFK_FP8_E4M3) -- the
                         weights the second GEMM applies, so that rows of O are exactly normalised -- where the
                         reference sums the fp32 values before the cast (online_softmax.h:173-206).  The rounding
                         is unbiased: the two sums agree to ~1e-4 relative (fp16) / < 1 % (e4m3).  One exception:
                         e4m3 with head_dim 256 sums the fp32 values, as the reference does                    */
} cfk_fmha_fwd_params;

/* FMHA forward: O = softmax(softmax_scale * Q K^T) V per (batch, head); no mask, no dropout.
 * Replaces fmhaForwardDevice (src/fmha-pipeline/fmha_forward.cu:86-383), one launch per call. */
int cfk_fmha_forward(const cfk_fmha_fwd_params *params, void *stream);

/* Bytes of LDS and the tile shape the library would pick for `params` (query rows per workgroup, keys per
 * tile); the reference fixes these at compile time (src/fmha-pipeline/shared_storage.h:4-22).  Any of the
 * out-pointers may be NULL.  Does not touch the GPU. */
int cfk_fmha_forward_plan(const cfk_fmha_fwd_params *params, int32_t *block_m, int32_t *block_n,
                          int32_t *lds_bytes, int32_t *threads);

/* The MFMA shape of the kernel build the library would pick for `params`: 32 (32x32x16 / 32x32x64 MFMAs) or 16
 * (16x16x32; fp16 operands: problems with more work items than half the CUs -- the more power-efficient shape on this
 * board -- and small ones at head dims 64 and 128, whose 32-row workgroups split the keys over their waves).  No
 * counterpart in the reference, whose MMA atom is fixed at compile time (src/fmha-pipeline/ss_helper.h:3-94).  The
 * environment variable CFK_FMHA_TILE=<query rows>x<keys>[/16|/16h|/32] overrides the automatic choice of tile and shape
 * (16h / 32h: the builds with the hand-scheduled main loop and persistent workgroups, fp16 / e4m3 at head dim 128; 32x64:
 * the small-grid build).
 * Does not touch the GPU. */
int cfk_fmha_forward_mfma(const cfk_fmha_fwd_params *params, int32_t *mfma_rows);

/* The name of the kernel instantiation the library would launch for `params`, as a profiler's kernel trace prints it
 * without its namespaces and with the booleans as 0/1, e.g. "fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>" (template
 * arguments: head dim, keys per tile, waves, waves per SIMD, e4m3 QK, e4m3 PV, V pre-transposed, score tap, tiles per
 * barrier, K fragment prefetch, 16x16x32 MFMAs, hand-scheduled loop): ties a measurement to the code that was measured.
 * `name` receives a NUL-terminated string of fewer than 80 bytes; CFK_ERR_INVALID_ARG if `capacity` is too small.  No
 * counterpart in the reference (one kernel per executable: src/fmha-pipeline/fmha_forward.cu:321-331).  Does not touch
 * the GPU. */
int cfk_fmha_forward_kernel(const cfk_fmha_fwd_params *params, char *name, int32_t capacity);

/* GEMM layouts for cfk_gemm_f16. */
typedef enum cfk_gemm_layout {
  CFK_GEMM_TN = 0, /* A: M x K (K contiguous), B: N x K (K contiguous) -- the reference's form
                      (src/cute-gemm-tma-gma/gemm.cu:362-380)                                                  */
  CFK_GEMM_NN = 1  /* A: M x K (K contiguous), B: K x N (N contiguous) -- the literal C = A.B                  */
} cfk_gemm_layout;

/* Dense GEMM C = A.B (fp16 operands, fp32 accumulate, fp16 C row-major M x N, N contiguous).
 * Replaces gemm(...) of the CuTe example (src/cute-gemm-tma-gma/gemm.cu:336-463) with alpha = 1, beta = 0.
 * M, N multiples of 256; K a multiple of 64. */
int cfk_gemm_f16(int32_t M, int32_t N, int32_t K, const void *A, const void *B, void *C, int32_t layout,
                 void *stream);

/* General form: D = alpha * A.B + beta * C for `batch` problems stored back to back (strides M*K, N*K, M*N elements).
 * Replaces
 *   - gemm(m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC, ..., L) of the CuTe example
 *     (src/cute-gemm-tma-gma/gemm.cu:336-463; type 1 = float operands, type 3 = half, :677-684; batch L, :519-521), and
 *   - Gemm::Arguments{{m,n,k}, {A, B}, {{alpha, beta}, C, D}} of the CUTLASS-API example
 *     (src/cutlass-gemm/gemm.cu:318-324).
 * dtype = CFK_FP16 or CFK_FP32 is the element type of A, B, C and D; accumulation and the epilogue are fp32 (the
 * reference accumulates in the C type).  gfx950 has no tf32 MFMA: CFK_FP32 multiplies in full fp32.  C and D are
 * row-major M x N; c may be NULL (beta is then ignored) and may alias d.  CFK_GEMM_NN exists for CFK_FP16 only.
 * M, N multiples of 256; K a multiple of 64; batch >= 1. */
typedef struct cfk_gemm_params {
  int32_t dtype;  /* cfk_dtype */
  int32_t layout; /* cfk_gemm_layout */
  int32_t m, n, k, batch;
  float alpha, beta;
  const void *a, *b, *c;
  void *d;
} cfk_gemm_params;
int cfk_gemm(const cfk_gemm_params *p, void *stream);

/* Process-wide options (read by every later call; set them before launching from several threads).  No counterpart in the
 * reference, whose choices of this kind are compile-time macros (src/fmha-pipeline/README.md:11-28). */
typedef enum cfk_option {
  /* 1: no optimistic first pass.  Two kernels first walk the keys with a softmax reference point fixed by the first key
   * tile (no row max per tile) and, only if some weight left the range of P's type, walk them again tracking the running
   * max as the reference does on every tile (online_softmax.h:123-165): e4m3 P from 3072 keys on, and fp16 problems
   * with more work items than half the CUs.  On scores that climb along the key axis that costs up to twice the time.  With this option
   * every call takes the max-tracking path from the start: the same results to rounding, a run time that does not
   * depend on the data (a few per cent slower on ordinary data).  0 (default): two passes where they pay. */
  CFK_OPT_PREDICTABLE_LATENCY = 1,
  /* 1: e4m3 weights without an exponential.  In the first of the two passes above, kernels with e4m3 P (head dims 64
   * and 128) then build the e4m3 code of a weight directly: read as an integer, the code of a positive e4m3 number is
   * 8 (log2 of it + 7) with the mantissa interpolated linearly, so sat_u8(round(8 (c s - m) + 55.54)) is exp2(c s - m)
   * rounded to e4m3 up to that interpolation -- one multiply-add and one conversion per score in place of multiply-add,
   * exponential and conversion: +11 % on B=4 H=16 S=4096 D=128, +27 % at head dim 64.  A fifth of the weights then
   * differ from the correctly rounded code by one step: on N(0,1) data the rms error of O against the fp32 reference
   * grows from 6.8e-4 to 8.1e-4 and the share of elements that fail the reference's own check (|d| > 5e-3 and more
   * than 10 % relative, src/fmha-pipeline/fmha_forward.cu:638-639) from 0-1e-4 % to 1e-4-6e-4 % with excursions above
   * its limit of 1e-3 % -- which is why this is an option.  The max-tracking pass always takes the exponential.
   * 0 (default): exponential and conversion everywhere. */
  CFK_OPT_FAST_E4M3_WEIGHTS = 2
} cfk_option;
int cfk_set_option(int32_t option, int32_t value);

/* Optional: performs the one-time per-process set-up of every kernel (raising their dynamic-LDS limits) on the
 * current device.  Launch calls do the same on first use of a kernel, thread-safely; calling this first keeps that
 * set-up out of latency-critical first calls and out of stream captures.  No counterpart in the reference, whose
 * entry sets the attribute on every call (include/utils/cuda_launch.hpp:7-20).  Needs a gfx950 device. */
int cfk_init(void);

/* Message for the calling thread's most recent non-zero return ("" if none). */
const char *cfk_last_error(void);

/* "cfk-mi355x <version> gfx950" */
const char *cfk_version(void);

#ifdef __cplusplus
}
#endif
#endif /* CFK_FMHA_H_ */
