"""CPU checker for the gfx950 kernels -- TEST INFRASTRUCTURE, never shipped.

Two independent statements of the reference's arithmetic live here:

* ``tyr_oracle.c`` (bound below through ctypes): plain scalar C following the
  reference's DSL kernels step by step (tiled online softmax, split-KV merge,
  f32-accumulate GEMM with bf16 epilogue, OCP E4M3 codec).
* ``libtorch_path.py``: the exact LibTorch calls the reference's FFI makes
  (cc/src/tyr.cpp:2563-2589, 4100-4133, 1602-1607), issued through the
  third-party ``torch`` package on CPU tensors.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The product (``tyr_amd``) must never do so.

All array arguments are numpy arrays; bf16 tensors travel as ``uint16`` bit
patterns, e4m3 tensors as ``uint8``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtyr_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile tyr_oracle.c with gcc (a few seconds)."""
    src = os.path.join(_HERE, "tyr_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libtyr_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        i64, f32, f64, vp, ci = (ctypes.c_int64, ctypes.c_float, ctypes.c_double,
                                 ctypes.c_void_p, ctypes.c_int)
        L.oracle_attn_fwd_f64.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, ci, f64]
        L.oracle_attn_fwd_f64.restype = None
        L.oracle_attn_fwd_f64_ex.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, ci, i64, vp, f64]
        L.oracle_attn_fwd_f64_ex.restype = None
        L.oracle_attn_bwd_f64_ex.argtypes = [vp] * 7 + [i64] * 5 + [ci, i64, vp, f64]
        L.oracle_attn_bwd_f64_ex.restype = None
        L.oracle_attn_fwd_f64_mask.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, ci, i64, vp, vp, f64]
        L.oracle_attn_fwd_f64_mask.restype = None
        L.oracle_attn_bwd_f64_mask.argtypes = [vp] * 7 + [i64] * 5 + [ci, i64, vp, vp, f64]
        L.oracle_attn_bwd_f64_mask.restype = None
        L.oracle_attn_bwd_f64.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, ci, f64]
        L.oracle_attn_bwd_f64.restype = None
        L.oracle_attn_fwd_tiled.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, ci, f32, i64]
        L.oracle_attn_fwd_tiled.restype = None
        L.oracle_gqa_decode.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, f32, i64]
        L.oracle_gqa_decode.restype = None
        L.oracle_gemm_bf16.argtypes = [vp, vp, vp, i64, i64, i64, ci]
        L.oracle_gemm_bf16.restype = None
        L.oracle_gemm_fp8.argtypes = [vp, vp, vp, vp, i64, i64, i64, f32, f32, ci]
        L.oracle_gemm_fp8.restype = None
        L.oracle_rope.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, ci]
        L.oracle_rope.restype = None
        L.oracle_layernorm_residual.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, f64]
        L.oracle_layernorm_residual.restype = None
        L.oracle_e4m3_decode.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3_decode.restype = f32
        L.oracle_e4m3_encode.argtypes = [f32]
        L.oracle_e4m3_encode.restype = ctypes.c_uint8
        L.oracle_f32_to_bf16.argtypes = [f32]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = f32
        L.oracle_num_threads.restype = ci
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _chk(a: np.ndarray, dtype, name: str) -> np.ndarray:
    if a.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {a.dtype}")
    return np.ascontiguousarray(a)


# ---- bf16 / e4m3 helpers (numpy, vectorised; same rules as the C code) -------------

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def e4m3_table() -> np.ndarray:
    """The 256 decoded values of OCP E4M3 (NaN at 0x7f / 0xff)."""
    L = lib()
    return np.array([L.oracle_e4m3_decode(i) for i in range(256)], dtype=np.float32)


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    L = lib()
    flat = np.ascontiguousarray(x, dtype=np.float32).ravel()
    return np.array([L.oracle_e4m3_encode(float(v)) for v in flat], dtype=np.uint8).reshape(x.shape)


# ---- the four operations --------------------------------------------------------------

def attn_fwd_f64(q, k, v, causal: bool, scale: float):
    """Textbook double-precision attention.  q,k,v uint16 [B,H,N,D] -> (O f32, LSE f32)."""
    q, k, v = (_chk(t, np.uint16, n) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    B, H, N, D = q.shape
    o = np.empty((B, H, N, D), np.float32)
    lse = np.empty((B, H, N), np.float32)
    lib().oracle_attn_fwd_f64(_p(q), _p(k), _p(v), _p(o), _p(lse), B, H, N, D, int(causal), float(scale))
    return o, lse


def attn_fwd_f64_ex(q, k, v, causal: bool, scale: float, window: int = 0, kv_lens=None, key_mask=None):
    """Double-precision attention with grouped queries (k, v may have fewer heads), a sliding window,
    per-sequence key lengths (int32 [B]) and a per-sequence key mask (uint8 / bool [B,N], nonzero = visible).
    -> (O f32 [B,Hq,N,D], LSE f32 [B,Hq,N])."""
    q, k, v = (_chk(t, np.uint16, n) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    o = np.empty((B, Hq, N, D), np.float32)
    lse = np.empty((B, Hq, N), np.float32)
    lens = None if kv_lens is None else _chk(np.asarray(kv_lens, dtype=np.int32), np.int32, "kv_lens")
    km = None if key_mask is None else _chk(np.asarray(key_mask).astype(np.uint8), np.uint8, "key_mask")
    assert km is None or km.shape == (B, N)
    lib().oracle_attn_fwd_f64_mask(_p(q), _p(k), _p(v), _p(o), _p(lse), B, Hq, Hkv, N, D, int(causal), int(window),
                                   None if lens is None else _p(lens), None if km is None else _p(km), float(scale))
    return o, lse


def attn_bwd_f64(q, k, v, d_o, causal: bool, scale: float):
    """Double-precision attention backward.  q,k,v,d_o uint16 [B,H,N,D] -> (dQ, dK, dV) f32."""
    q, k, v, d_o = (_chk(t, np.uint16, n) for t, n in ((q, "q"), (k, "k"), (v, "v"), (d_o, "d_o")))
    B, H, N, D = q.shape
    dq, dk, dv = (np.empty((B, H, N, D), np.float32) for _ in range(3))
    lib().oracle_attn_bwd_f64(_p(q), _p(k), _p(v), _p(d_o), _p(dq), _p(dk), _p(dv), B, H, N, D,
                              int(causal), float(scale))
    return dq, dk, dv


def attn_bwd_f64_ex(q, k, v, d_o, causal: bool, scale: float, window: int = 0, kv_lens=None, key_mask=None):
    """Double-precision attention backward with grouped queries, window, key lengths and key mask.
    q, d_o uint16 [B,Hq,N,D]; k, v uint16 [B,Hkv,N,D] -> (dQ [B,Hq,N,D], dK, dV [B,Hkv,N,D]) f32."""
    q, k, v, d_o = (_chk(t, np.uint16, n) for t, n in ((q, "q"), (k, "k"), (v, "v"), (d_o, "d_o")))
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    dq = np.empty((B, Hq, N, D), np.float32)
    dk, dv = np.empty((B, Hkv, N, D), np.float32), np.empty((B, Hkv, N, D), np.float32)
    lens = None if kv_lens is None else _chk(np.asarray(kv_lens, dtype=np.int32), np.int32, "kv_lens")
    km = None if key_mask is None else _chk(np.asarray(key_mask).astype(np.uint8), np.uint8, "key_mask")
    assert km is None or km.shape == (B, N)
    lib().oracle_attn_bwd_f64_mask(_p(q), _p(k), _p(v), _p(d_o), _p(dq), _p(dk), _p(dv), B, Hq, Hkv, N, D, int(causal),
                                   int(window), None if lens is None else _p(lens), None if km is None else _p(km),
                                   float(scale))
    return dq, dk, dv


def attn_fwd_tiled(q, k, v, causal: bool, scale: float, tile_kv: int = 64):
    """The reference kernel's tiled online softmax.  -> (O bf16 bits uint16, LSE f32)."""
    q, k, v = (_chk(t, np.uint16, n) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    B, H, N, D = q.shape
    o = np.empty((B, H, N, D), np.uint16)
    lse = np.empty((B, H, N), np.float32)
    lib().oracle_attn_fwd_tiled(_p(q), _p(k), _p(v), _p(o), _p(lse), B, H, N, D, int(causal),
                                float(scale), int(tile_kv))
    return o, lse


def gqa_decode(q, k, v, scale: float, num_splits: int = 1, kv_len: int | None = None):
    """q uint16 [B,Hq,1,D]; k,v uint16 [B,Hkv,Lmax,D]; attends to the first kv_len rows."""
    q, k, v = (_chk(t, np.uint16, n) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    B, Hq, one, D = q.shape
    assert one == 1
    _, Hkv, Lmax, _ = k.shape
    L = Lmax if kv_len is None else int(kv_len)
    o = np.empty((B, Hq, 1, D), np.uint16)
    lse = np.empty((B, Hq), np.float32)
    lib().oracle_gqa_decode(_p(q), _p(k), _p(v), _p(o), _p(lse), B, Hq, Hkv, L, D, Lmax,
                            float(scale), int(num_splits))
    return o, lse


def gemm_bf16(a, b, trans_b: bool = False):
    a, b = _chk(a, np.uint16, "a"), _chk(b, np.uint16, "b")
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == K
    c = np.empty((M, N), np.uint16)
    lib().oracle_gemm_bf16(_p(a), _p(b), _p(c), M, N, K, int(trans_b))
    return c


def gemm_fp8(aq, bq, scale_a: float, scale_b: float, trans_b: bool = False):
    """-> (C bf16 bits uint16, C f32 before the bf16 rounding)."""
    aq, bq = _chk(aq, np.uint8, "aq"), _chk(bq, np.uint8, "bq")
    M, K = aq.shape
    N = bq.shape[0] if trans_b else bq.shape[1]
    assert (bq.shape[1] if trans_b else bq.shape[0]) == K
    c = np.empty((M, N), np.uint16)
    cf = np.empty((M, N), np.float32)
    lib().oracle_gemm_fp8(_p(aq), _p(bq), _p(c), _p(cf), M, N, K, float(scale_a), float(scale_b),
                          int(trans_b))
    return c, cf


def rope(x, cos, sin):
    """Rotary embedding.  x float32 or uint16 (bf16 bits) [B,S,H,D]; cos, sin float32 [S,D/2] -> same dtype as x."""
    is_bf16 = x.dtype == np.uint16
    x = _chk(x, np.uint16 if is_bf16 else np.float32, "x")
    cos, sin = _chk(cos, np.float32, "cos"), _chk(sin, np.float32, "sin")
    B, S, H, D = x.shape
    y = np.empty_like(x)
    lib().oracle_rope(_p(x), _p(cos), _p(sin), _p(y), B, S, H, D, int(is_bf16))
    return y


def layernorm_residual(x, residual, weight, bias, eps: float = 1e-5):
    """Fused residual + LayerNorm.  uint16 (bf16 bits): x, residual [rows,d]; weight, bias [d] -> (out, out_resid)."""
    x, residual = _chk(x, np.uint16, "x"), _chk(residual, np.uint16, "residual")
    weight, bias = _chk(weight, np.uint16, "weight"), _chk(bias, np.uint16, "bias")
    rows, d = x.shape
    out, out_resid = np.empty_like(x), np.empty_like(x)
    lib().oracle_layernorm_residual(_p(x), _p(residual), _p(weight), _p(bias), _p(out), _p(out_resid), rows, d,
                                    float(eps))
    return out, out_resid


def num_threads() -> int:
    return int(lib().oracle_num_threads())
