"""ctypes binding of the C-ABI in ``include/cfk_fmha.h``.

Mirrors the reference's host entry ``fmhaForwardDevice`` (src/fmha-pipeline/fmha_forward.cu:86-93): device
pointers for Q/K/V/O in [B,S,H,D], sizes, softmax scale, precision.  torch is used only to own device memory
and streams; all compute happens in ``libcfk_fmha.so``.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcfk_fmha.so")
_lib = None

CFK_FP16 = 1
CFK_FP8_E4M3 = 2
CFK_FP32 = 3  # GEMM only
CFK_V_BSHD = 0
CFK_V_BDHS = 1
CFK_GEMM_TN = 0
CFK_GEMM_NN = 1
CFK_OPT_PREDICTABLE_LATENCY = 1
CFK_OPT_FAST_E4M3_WEIGHTS = 2


class CfkError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"cfk error {code}: {msg}")
        self.code = code


class FmhaFwdParams(ctypes.Structure):
    """``cfk_fmha_fwd_params`` (include/cfk_fmha.h)."""
    _fields_ = [
        ("dtype", ctypes.c_int32), ("v_dtype", ctypes.c_int32),
        ("batch", ctypes.c_int32), ("heads", ctypes.c_int32),
        ("seqlen_q", ctypes.c_int32), ("seqlen_kv", ctypes.c_int32),
        ("head_dim", ctypes.c_int32), ("v_layout", ctypes.c_int32),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("o", ctypes.c_void_p),
        ("softmax_scale", ctypes.c_float),
        ("q_descale", ctypes.c_float), ("k_descale", ctypes.c_float), ("v_descale", ctypes.c_float),
        ("dbg_s", ctypes.c_void_p), ("dbg_row_max", ctypes.c_void_p), ("dbg_row_sum", ctypes.c_void_p),
    ]


class GemmParams(ctypes.Structure):
    """``cfk_gemm_params`` (include/cfk_fmha.h)."""
    _fields_ = [
        ("dtype", ctypes.c_int32), ("layout", ctypes.c_int32),
        ("m", ctypes.c_int32), ("n", ctypes.c_int32), ("k", ctypes.c_int32), ("batch", ctypes.c_int32),
        ("alpha", ctypes.c_float), ("beta", ctypes.c_float),
        ("a", ctypes.c_void_p), ("b", ctypes.c_void_p), ("c", ctypes.c_void_p), ("d", ctypes.c_void_p),
    ]


def lib_path() -> str:
    return _LIB_PATH


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 (``make -C csrc``; always recompiles what changed)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    res = subprocess.run(cmd, capture_output=not verbose, text=True)
    if res.returncode != 0:
        raise RuntimeError("building libcfk_fmha.so failed:\n" + (res.stdout or "") + (res.stderr or ""))
    return _LIB_PATH


def lib():
    """The loaded C-ABI library.  Raises if it has not been built -- there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
                f"or make -C {os.path.join(_HERE, 'csrc')}). There is no CPU fallback.")
        l = ctypes.CDLL(_LIB_PATH)
        l.cfk_fmha_forward.restype = ctypes.c_int
        l.cfk_fmha_forward.argtypes = [ctypes.POINTER(FmhaFwdParams), ctypes.c_void_p]
        l.cfk_fmha_forward_plan.restype = ctypes.c_int
        l.cfk_fmha_forward_plan.argtypes = [ctypes.POINTER(FmhaFwdParams)] + [ctypes.POINTER(ctypes.c_int32)] * 4
        l.cfk_fmha_forward_mfma.restype = ctypes.c_int
        l.cfk_fmha_forward_mfma.argtypes = [ctypes.POINTER(FmhaFwdParams), ctypes.POINTER(ctypes.c_int32)]
        l.cfk_fmha_forward_kernel.restype = ctypes.c_int
        l.cfk_fmha_forward_kernel.argtypes = [ctypes.POINTER(FmhaFwdParams), ctypes.c_char_p, ctypes.c_int32]
        l.cfk_gemm_f16.restype = ctypes.c_int
        l.cfk_gemm_f16.argtypes = [ctypes.c_int32] * 3 + [ctypes.c_void_p] * 3 + [ctypes.c_int32, ctypes.c_void_p]
        l.cfk_gemm.restype = ctypes.c_int
        l.cfk_gemm.argtypes = [ctypes.POINTER(GemmParams), ctypes.c_void_p]
        l.cfk_init.restype = ctypes.c_int
        l.cfk_init.argtypes = []
        l.cfk_set_option.restype = ctypes.c_int
        l.cfk_set_option.argtypes = [ctypes.c_int32, ctypes.c_int32]
        l.cfk_last_error.restype = ctypes.c_char_p
        l.cfk_version.restype = ctypes.c_char_p
        _lib = l
    return _lib


def init() -> None:
    """``cfk_init``: one-time set-up of every kernel on the current device (optional; launches do it on demand)."""
    _check(lib().cfk_init())


def set_option(option: int, value: int) -> None:
    """``cfk_set_option``: process-wide options (``CFK_OPT_PREDICTABLE_LATENCY``, ``CFK_OPT_FAST_E4M3_WEIGHTS``)."""
    _check(lib().cfk_set_option(option, value))


def last_error() -> str:
    return lib().cfk_last_error().decode()


def version() -> str:
    return lib().cfk_version().decode()


def _check(rc):
    if rc != 0:
        raise CfkError(rc, last_error())


def make_params(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, q=0, k=0, v=0, o=0, softmax_scale=None,
                q_descale=1.0, k_descale=1.0, v_descale=1.0, v_layout=CFK_V_BSHD, v_dtype=None,
                dbg_row_max=0, dbg_row_sum=0, dbg_s=0) -> FmhaFwdParams:
    p = FmhaFwdParams()
    p.dtype = dtype
    p.v_dtype = dtype if v_dtype is None else v_dtype
    p.batch, p.heads, p.seqlen_q, p.seqlen_kv, p.head_dim = batch, heads, seqlen_q, seqlen_kv, head_dim
    p.v_layout = v_layout
    p.q, p.k, p.v, p.o = q or None, k or None, v or None, o or None
    p.softmax_scale = (1.0 / math.sqrt(head_dim)) if softmax_scale is None else softmax_scale
    p.q_descale, p.k_descale, p.v_descale = q_descale, k_descale, v_descale
    p.dbg_s = dbg_s or None
    p.dbg_row_max = dbg_row_max or None
    p.dbg_row_sum = dbg_row_sum or None
    return p


def fmha_forward_plan(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, v_layout=CFK_V_BSHD, v_dtype=None):
    """(block_m, block_n, lds_bytes, threads) the library picks; raises CfkError for unsupported shapes.  No GPU needed."""
    p = make_params(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, v_layout=v_layout, v_dtype=v_dtype)
    out = [ctypes.c_int32() for _ in range(4)]
    _check(lib().cfk_fmha_forward_plan(ctypes.byref(p), *[ctypes.byref(x) for x in out]))
    return tuple(x.value for x in out)


def fmha_forward_mfma(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, v_layout=CFK_V_BSHD, v_dtype=None):
    """``cfk_fmha_forward_mfma``: 32 or 16, the MFMA shape of the kernel build the library picks.  No GPU needed."""
    p = make_params(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, v_layout=v_layout, v_dtype=v_dtype)
    out = ctypes.c_int32()
    _check(lib().cfk_fmha_forward_mfma(ctypes.byref(p), ctypes.byref(out)))
    return out.value


def fmha_forward_kernel(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, v_layout=CFK_V_BSHD, v_dtype=None):
    """``cfk_fmha_forward_kernel``: the name of the instantiation the library launches for this call, as a kernel trace
    prints it (``fmha_fwd_kernel16p<128,64,8,2,0,0,0,0,2,0,1,1>``).  No GPU needed."""
    p = make_params(dtype, batch, heads, seqlen_q, seqlen_kv, head_dim, v_layout=v_layout, v_dtype=v_dtype)
    buf = ctypes.create_string_buffer(80)
    _check(lib().cfk_fmha_forward_kernel(ctypes.byref(p), buf, len(buf)))
    return buf.value.decode()


def _stream_ptr(stream):
    if stream is None:
        import torch
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(stream if isinstance(stream, int) else stream.cuda_stream)


def fmha_forward(q, k, v, o=None, softmax_scale=None, q_descale=1.0, k_descale=1.0, v_descale=1.0,
                 v_layout=CFK_V_BSHD, row_max=None, row_sum=None, scores=None, stream=None, prepare=False):
    """O = softmax(scale * Q K^T) V on device tensors in [B,S,H,D] (D contiguous).
    ``prepare=True`` launches nothing and returns a ``PreparedForward``: a callable that repeats this exact call.

    q,k,v: torch CUDA tensors, float16, or float8_e4m3fn / uint8 holding e4m3 codes (v may be float16 with e4m3
    q,k: hybrid mode).  ``v`` is [B,D,H,S] when
    ``v_layout == CFK_V_BDHS``.  ``row_max`` / ``row_sum`` / ``scores`` are the optional debug taps.  Returns ``o`` (float16 [B,Sq,H,D]); launches asynchronously on ``stream``
    (default: torch's current stream)."""
    import torch
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise ValueError("q, k, v must be device tensors (there is no CPU path)")
    if not (q.is_contiguous() and k.is_contiguous() and v.is_contiguous()):
        raise ValueError("q, k, v must be contiguous [B,S,H,D]")
    if q.dtype == torch.float16:
        dtype = CFK_FP16
    elif q.dtype in (torch.float8_e4m3fn, torch.uint8):
        dtype = CFK_FP8_E4M3
    else:
        raise ValueError(f"unsupported dtype {q.dtype}")
    if k.dtype != q.dtype:
        raise ValueError("q and k must share one dtype")
    if v.dtype == q.dtype:
        v_dtype = dtype
    elif dtype == CFK_FP8_E4M3 and v.dtype == torch.float16:
        v_dtype = CFK_FP16  # hybrid mode: e4m3 Q,K with fp16 P,V (the reference's fp8 build without GEMM2FP8)
    else:
        raise ValueError("v must have the dtype of q, or float16 with fp8 q/k")
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    if tuple(k.shape) != (B, Skv, H, D):
        raise ValueError("k shape mismatch")
    want_v = (B, Skv, H, D) if v_layout == CFK_V_BSHD else (B, D, H, Skv)
    if tuple(v.shape) != want_v:
        raise ValueError(f"v shape {tuple(v.shape)} does not match layout {v_layout}: expected {want_v}")
    if o is None:
        o = torch.empty((B, Sq, H, D), dtype=torch.float16, device=q.device)
    elif o.dtype != torch.float16 or tuple(o.shape) != (B, Sq, H, D) or not o.is_contiguous() or not o.is_cuda:
        raise ValueError("o must be a contiguous float16 device tensor [B,Sq,H,D]")
    for t in (row_max, row_sum):
        if t is not None and (t.dtype != torch.float32 or tuple(t.shape) != (B, H, Sq) or not t.is_contiguous()):
            raise ValueError("row_max/row_sum must be contiguous float32 [B,H,Sq]")
    if scores is not None and (scores.dtype != torch.float32 or tuple(scores.shape) != (B, H, Sq, Skv)
                               or not scores.is_contiguous()):
        raise ValueError("scores must be contiguous float32 [B,H,Sq,Skv]")
    p = make_params(dtype, B, H, Sq, Skv, D, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), softmax_scale,
                    q_descale, k_descale, v_descale, v_layout, v_dtype=v_dtype,
                    dbg_row_max=row_max.data_ptr() if row_max is not None else 0,
                    dbg_row_sum=row_sum.data_ptr() if row_sum is not None else 0,
                    dbg_s=scores.data_ptr() if scores is not None else 0)
    if prepare:
        return PreparedForward(p, (q, k, v, o, row_max, row_sum, scores), stream)
    _check(lib().cfk_fmha_forward(ctypes.byref(p), _stream_ptr(stream)))
    return o


class PreparedForward:
    """One ``cfk_fmha_forward`` call with its parameter block filled in once (``fmha_forward(..., prepare=True)``): calling
    the object launches it again on the stream given at preparation (torch's current stream then, if none was given).
    What a C++ caller's launch loop does (src/fmha-pipeline/fmha_forward.cu:578-592): the checks and the ctypes
    marshalling of ``fmha_forward`` cost several microseconds per call, as much as a small problem's kernel."""

    def __init__(self, params, tensors, stream):
        self.params, self.tensors = params, tensors   # (the tensors are held so that their memory stays alive)
        self.o = tensors[3]
        self._ref = ctypes.byref(params)
        self._stream = _stream_ptr(stream)
        self._fn = lib().cfk_fmha_forward

    def __call__(self):
        rc = self._fn(self._ref, self._stream)
        if rc != 0:
            _check(rc)
        return self.o


def gemm_f16(a, b, c=None, layout=CFK_GEMM_TN, stream=None):
    """C[M,N] = A[M,K] . B  with B as [N,K] (TN, the reference's form) or [K,N] (NN); fp16 in, fp32 accumulate, fp16 out."""
    import torch
    if a.dtype != torch.float16 or b.dtype != torch.float16 or not (a.is_cuda and b.is_cuda):
        raise ValueError("a, b must be float16 device tensors")
    if not (a.is_contiguous() and b.is_contiguous()):
        raise ValueError("a, b must be contiguous")
    M, K = a.shape
    N = b.shape[0] if layout == CFK_GEMM_TN else b.shape[1]
    if tuple(b.shape) != ((N, K) if layout == CFK_GEMM_TN else (K, N)):
        raise ValueError("b shape mismatch")
    if c is None:
        c = torch.empty((M, N), dtype=torch.float16, device=a.device)
    _check(lib().cfk_gemm_f16(M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), layout, _stream_ptr(stream)))
    return c


def gemm(a, b, c=None, alpha=1.0, beta=0.0, out=None, layout=CFK_GEMM_TN, stream=None):
    """D = alpha * A.B + beta * C, fp32 accumulate and epilogue (``cfk_gemm``).

    ``a`` is [M,K] or [L,M,K]; ``b`` is [N,K] (TN, the reference's form, src/cute-gemm-tma-gma/gemm.cu:362-380) or
    [K,N] (NN, fp16 only), with the same leading batch dimension; ``c`` / ``out`` are [M,N] or [L,M,N].  float16 or
    float32 device tensors, all of one dtype (the reference's types 3 and 1, gemm.cu:677-684).
    """
    import torch
    if a.dtype not in (torch.float16, torch.float32) or b.dtype != a.dtype or not (a.is_cuda and b.is_cuda):
        raise ValueError("a, b must be float16 or float32 device tensors of one dtype")
    if a.dim() not in (2, 3) or b.dim() != a.dim():
        raise ValueError("a, b must both be 2-D or both 3-D (leading batch dimension)")
    if not (a.is_contiguous() and b.is_contiguous()):
        raise ValueError("a, b must be contiguous")
    L = a.shape[0] if a.dim() == 3 else 1
    M, K = a.shape[-2:]
    N = b.shape[-2] if layout == CFK_GEMM_TN else b.shape[-1]
    if tuple(b.shape[-2:]) != ((N, K) if layout == CFK_GEMM_TN else (K, N)) or (b.dim() == 3 and b.shape[0] != L):
        raise ValueError("b shape mismatch")
    shape = (L, M, N) if a.dim() == 3 else (M, N)
    if out is None:
        out = torch.empty(shape, dtype=a.dtype, device=a.device)
    for t in (c, out):
        if t is not None and (t.dtype != a.dtype or tuple(t.shape) != shape or not t.is_contiguous() or not t.is_cuda):
            raise ValueError("c / out must be contiguous device tensors of a's dtype and shape " + str(shape))
    p = GemmParams()
    p.dtype = CFK_FP16 if a.dtype == torch.float16 else CFK_FP32
    p.layout = layout
    p.m, p.n, p.k, p.batch = M, N, K, L
    p.alpha, p.beta = float(alpha), float(beta)
    p.a, p.b, p.d = a.data_ptr(), b.data_ptr(), out.data_ptr()
    p.c = c.data_ptr() if c is not None else None
    _check(lib().cfk_gemm(ctypes.byref(p), _stream_ptr(stream)))
    return out
