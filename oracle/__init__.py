"""CPU oracle for the FMHA-forward hot path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this
package, and only as the checker / reported CPU baseline.  The product (``cutlass-kernels_amd``) never does.

Contents (each function cites the reference lines it restates):

* :func:`attention_f32`, :func:`gemm_f32` -- ctypes front-ends of ``host_attention.c``
  (``include/utils/fmha_cutlass.hpp:154-317`` and ``src/cute-gemm-tma-gma/gemm.cu:362-380``).
* :func:`verify_tensor` -- the reference checker (``include/utils/random.hpp:54-90``).
* :func:`e4m3_decode`, :func:`e4m3_encode` -- OCP e4m3fn codec (what ``cutlass::float_e4m3_t`` is,
  ``src/fmha-pipeline/fmha_forward.cu:425-439``); round-to-nearest-even, saturating.
* :func:`online_softmax_tiled` -- numpy emulation of the kernel-side algorithm
  (``src/fmha-pipeline/online_softmax.h:87-207``, ``fmha_consumer.h:25-72``) for small cases.
* :func:`transpose_v_bdhs`, :func:`permute_keys16` -- the fp8 V layouts
  (``src/fmha-pipeline/fmha_forward.cu:514-532`` and ``:534-558``).

Pins: see ``tests/test_oracle.py``.  The reference ships no golden vectors for this path and its own
inputs come from an unreproducible curand stream, so the literal reference outputs are "parity
unpinned"; everything above is pinned by closed forms, invariants and exhaustive codec tables.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcfk_oracle.so")
_lib = None

LOG2E = np.float32(1.4426950408889634074)  # include/utils/fmha_cutlass.hpp:74


def build(force: bool = False) -> str:
    """Compile ``host_attention.c`` with gcc (plain ``make``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int)
        lib.cfk_oracle_attention_f32.restype = ctypes.c_int
        lib.cfk_oracle_attention_f32.argtypes = [fp, fp, fp, fp, fp, fp, fp] + [ctypes.c_int] * 5 + [
            ctypes.c_float, ctypes.c_int, ctypes.c_int, ip, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.cfk_oracle_gemm_f32.restype = ctypes.c_int
        lib.cfk_oracle_gemm_f32.argtypes = [fp, fp, fp] + [ctypes.c_int] * 4 + [ip, ctypes.c_int]
        lib.cfk_oracle_num_threads.restype = ctypes.c_int
        _lib = lib
    return _lib


def num_threads() -> int:
    return int(_load().cfk_oracle_num_threads())


def _fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)) if a is not None else None


def attention_f32(q, k, v, alpha0=None, use_pow2=False, use_prescaling=True, bh_pairs=None,
                  row_start=0, row_step=1, want_scores=False, want_stats=False, out=None):
    """fp32 ``softmax(alpha0 * Q K^T) V`` over ``[B,S,H,D]`` float32 arrays.

    Restates ``TestAttention::compute`` (include/utils/fmha_cutlass.hpp:154-317); ``alpha0`` defaults to
    ``1/sqrt(D)`` (:125).  Returns a dict with ``O`` ``[B,Sq,H,D]`` and, on request, ``S`` ``[B,H,Sq,Skv]``
    (pre-softmax scaled scores), ``row_max`` and ``inv_sum`` ``[B,H,Sq]``.  Rows/heads outside the
    selected subset keep the value NaN in ``O`` (so that an accidental comparison fails).
    """
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    B, Sq, H, D = q.shape
    Skv = k.shape[1]
    assert k.shape == (B, Skv, H, D) and v.shape == (B, Skv, H, D)
    if alpha0 is None:
        alpha0 = 1.0 / np.sqrt(np.float32(D))
    o = out if out is not None else np.full((B, Sq, H, D), np.nan, dtype=np.float32)
    s = np.full((B, H, Sq, Skv), np.nan, dtype=np.float32) if want_scores else None
    mx = np.full((B, H, Sq), np.nan, dtype=np.float32) if want_stats else None
    inv = np.full((B, H, Sq), np.nan, dtype=np.float32) if want_stats else None
    pairs = None
    n_pairs = 0
    if bh_pairs is not None:
        pairs = np.ascontiguousarray(np.asarray(bh_pairs, dtype=np.int32).reshape(-1, 2))
        n_pairs = pairs.shape[0]
    rc = _load().cfk_oracle_attention_f32(
        _fptr(q), _fptr(k), _fptr(v), _fptr(o), _fptr(s), _fptr(mx), _fptr(inv), B, Sq, Skv, H, D,
        ctypes.c_float(float(alpha0)), int(bool(use_pow2)), int(bool(use_prescaling)),
        pairs.ctypes.data_as(ctypes.POINTER(ctypes.c_int)) if pairs is not None else None, n_pairs,
        int(row_start), int(row_step))
    if rc != 0:
        raise ValueError("cfk_oracle_attention_f32 rejected its arguments")
    res = {"O": o}
    if want_scores:
        res["S"] = s
    if want_stats:
        res["row_max"] = mx
        res["inv_sum"] = inv
    return res


def gemm_f32(a, b, rows=None, b_is_kn=False):
    """``C[m,n] = sum_k A[m,k] B[n,k]`` (or ``B[k,n]`` when ``b_is_kn``), float accumulate, for the
    selected rows of A.  Restates the cute-gemm problem (src/cute-gemm-tma-gma/gemm.cu:362-380, 498)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    M, K = a.shape
    N = b.shape[1] if b_is_kn else b.shape[0]
    assert b.shape == ((K, N) if b_is_kn else (N, K))
    r = None if rows is None else np.ascontiguousarray(rows, dtype=np.int32)
    nr = M if r is None else r.shape[0]
    c = np.empty((nr, N), dtype=np.float32)
    rc = _load().cfk_oracle_gemm_f32(
        _fptr(a), _fptr(b), _fptr(c), M, N, K, int(bool(b_is_kn)),
        r.ctypes.data_as(ctypes.POINTER(ctypes.c_int)) if r is not None else None, nr)
    if rc != 0:
        raise ValueError("cfk_oracle_gemm_f32 rejected its arguments")
    return c


# ----------------------------------------------------------------------------------------------------
# checker (include/utils/random.hpp:54-90)
# ----------------------------------------------------------------------------------------------------
def verify_tensor(x, ref, err_count_expected=0.0):
    """Reference pass criterion: an element is an error iff NaN/Inf or (|d| > 5e-3 and |d|/|ref+1e-5| > 1e-1);
    pass iff 100*errors/size <= err_count_expected (a percentage: 1e-4 for fp16, 1e-3 for fp8,
    src/fmha-pipeline/fmha_forward.cu:638-639).  Returns (passed, error_percentage)."""
    x = np.asarray(x, dtype=np.float32).ravel()
    ref = np.asarray(ref, dtype=np.float32).ravel()
    size = min(x.size, ref.size)
    x, ref = x[:size], ref[:size]
    abs_diff = np.abs(x - ref)
    rel = abs_diff / np.abs(ref + np.float32(1e-5))
    bad = np.isnan(ref) | np.isnan(abs_diff) | np.isinf(abs_diff) | ((abs_diff > np.float32(5e-3)) & (rel > np.float32(1e-1)))
    pct = float(np.float32(bad.sum()) / np.float32(size) * 100)
    return pct <= err_count_expected, pct


# ----------------------------------------------------------------------------------------------------
# OCP e4m3fn codec (cutlass::float_e4m3_t; bias 7, max 448, no Inf, NaN = 0x7F / 0xFF)
# ----------------------------------------------------------------------------------------------------
def e4m3_decode_table() -> np.ndarray:
    """Closed-form value of each of the 256 codes (float32; NaN for 0x7F and 0xFF)."""
    codes = np.arange(256, dtype=np.int64)
    sign = np.where(codes & 0x80, -1.0, 1.0)
    e = (codes >> 3) & 0xF
    m = codes & 0x7
    val = np.where(e == 0, (m / 8.0) * 2.0 ** -6, (1.0 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))
    val = sign * val
    val[(codes & 0x7F) == 0x7F] = np.nan
    return val.astype(np.float32)


_E4M3_TABLE = e4m3_decode_table()
_E4M3_POS = _E4M3_TABLE[:0x7F].astype(np.float64)            # codes 0..0x7E, ascending values
_E4M3_MID = (_E4M3_POS[:-1] + _E4M3_POS[1:]) / 2.0             # exact in float64


def e4m3_decode(codes) -> np.ndarray:
    return _E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(x) -> np.ndarray:
    """float -> e4m3fn code, round-to-nearest-even, saturating to +-448 (NaN -> 0x7F)."""
    x = np.asarray(x, dtype=np.float32)
    ax = np.minimum(np.abs(x).astype(np.float64), 448.0)
    lo = np.searchsorted(_E4M3_MID, ax, side="left")
    hi = np.searchsorted(_E4M3_MID, ax, side="right")
    code = np.where(lo == hi, lo, np.where(lo % 2 == 0, lo, hi)).astype(np.uint8)
    code = np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)
    return np.where(np.isnan(x), np.uint8(0x7F), code).astype(np.uint8)


def quantize_e4m3_per_tensor(x):
    """Per-tensor amax scaling: scale = amax/448, codes = e4m3(x/scale).  Returns (codes, scale)."""
    x = np.asarray(x, dtype=np.float32)
    amax = float(np.max(np.abs(x)))
    scale = np.float32(amax / 448.0) if amax > 0 else np.float32(1.0)
    return e4m3_encode(x / scale), scale


# ----------------------------------------------------------------------------------------------------
# fp8 V layouts of the reference driver
# ----------------------------------------------------------------------------------------------------
def transpose_v_bdhs(v):
    """[B,S,H,D] -> [B,D,H,S] (src/fmha-pipeline/fmha_forward.cu:514-532)."""
    return np.ascontiguousarray(np.transpose(v, (0, 3, 2, 1)))


def permute_keys16(vt):
    """Permute the (last, sequence) index inside every block of 16:
    dst[p + 2r + 8q] = src[p + 2q + 4r], p,q in {0,1}, r in 0..3 (fmha_forward.cu:540-551)."""
    src_of_dst = np.empty(16, dtype=np.int64)
    for r in range(4):
        for q in range(2):
            for p in range(2):
                src_of_dst[p + 2 * r + 8 * q] = p + 2 * q + 4 * r
    s = vt.shape[-1]
    assert s % 16 == 0
    blk = vt.reshape(vt.shape[:-1] + (s // 16, 16))
    return np.ascontiguousarray(blk[..., src_of_dst].reshape(vt.shape))


# ----------------------------------------------------------------------------------------------------
# kernel-side algorithm, emulated (small cases only)
# ----------------------------------------------------------------------------------------------------
def online_softmax_tiled(q, k, v, bN, scale_log2, p_cast="f16", v_scale=1.0):
    """Numpy emulation of the per-tile loop of the device kernels for one head:
    q [Sq,D], k,v [Skv,D] float32 (already the up-cast operands).  ``scale_log2`` = softmax_scale*log2e
    (fmha_forward.cu:452-454).  Per tile j (fmha_consumer.h:25-72, online_softmax.h:87-207):
    S=QK_j^T; t=scale*S; m'=max(m,rowmax t); if j>0: a=exp2(m-m'), l*=a, O*=a; P=exp2(t-m');
    l+=rowsum(P) (fp32, before the down-cast); O += cast(P) V_j.  End: O *= 1/l (online_softmax.h:59-85).
    Returns (O, m_log2, l)."""
    q = np.asarray(q, np.float32)
    k = np.asarray(k, np.float32)
    v = np.asarray(v, np.float32)
    Sq, D = q.shape
    Skv = k.shape[0]
    assert Skv % bN == 0
    m = np.full((Sq,), -np.inf, np.float32)
    l = np.zeros((Sq,), np.float32)
    o = np.zeros((Sq, D), np.float32)
    for j in range(Skv // bN):
        kj, vj = k[j * bN:(j + 1) * bN], v[j * bN:(j + 1) * bN]
        t = np.float32(scale_log2) * (q @ kj.T).astype(np.float32)
        m_new = np.maximum(m, t.max(axis=1))
        if j > 0:
            a = np.exp2(m - m_new).astype(np.float32)
            l = l * a
            o = o * a[:, None]
        p = np.exp2(t - m_new[:, None]).astype(np.float32)
        l = l + p.sum(axis=1, dtype=np.float32)
        if p_cast == "f16":
            pc = p.astype(np.float16).astype(np.float32)
        elif p_cast == "e4m3":
            pc = e4m3_decode(e4m3_encode(p))
        else:
            pc = p
        o = o + (pc @ vj).astype(np.float32)
        m = m_new
    o = o * (np.float32(1.0) / l)[:, None] * np.float32(v_scale)
    return o, m, l
