"""Host-side mirror of the Lean entry points ``Tyr.GPU.GFX950.*`` for torch tensors.

Same names, argument meaning and error behaviour as the Lean declarations in
``tyr_amd/lean/Tyr/GPU/GFX950.lean`` (which bind ``lean_tyr_gpu_*`` in
``csrc/lean_shim.cpp``): outputs are freshly allocated and returned, every tensor argument
is checked the way the reference's generated launcher checks it
(Tyr/GPU/Codegen/Attribute.lean:334-336: device, contiguity, rank <= 4) and a failed
check or a negative status from the C ABI raises ``TyrGpuError`` -- the analogue of the
``IO.userError`` the Lean wrappers return.  torch is used for device memory and the
current stream only; all arithmetic happens in ``libtyr_hip.so``.
"""
from __future__ import annotations

import ctypes
import functools
import math

import torch

from . import _lib


class TyrGpuError(RuntimeError):
    """Raised where the Lean wrapper would return ``IO.userError msg``."""


def library_path() -> str:
    return _lib.LIB_PATH


def _check(t: torch.Tensor, name: str, dtype, ndim: int | None = None) -> None:
    if not isinstance(t, torch.Tensor):
        raise TyrGpuError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise TyrGpuError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise TyrGpuError(f"{name} must be contiguous")
    if t.dim() > 4:
        raise TyrGpuError(f"{name} must have dim <= 4")
    if ndim is not None and t.dim() != ndim:
        raise TyrGpuError(f"{name} must have dim == {ndim}")
    if t.dtype != dtype:
        raise TyrGpuError(f"{name} must have dtype {dtype}")


def _raise(rc: int, what: str) -> None:
    if rc != 0:
        msg = _lib.load().tyr_hip_strerror(rc).decode()
        raise TyrGpuError(f"{what}: {msg} (status {rc})")


def _stream(stream) -> int:
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def _on_launch_stream(fn):
    """Outputs and scratch come from torch's caching allocator, which ties a block to the stream that was
    current when it was allocated and may hand a freed block to the next allocation on that stream.  The kernels
    run on the caller's ``stream``; when that is not torch's current stream it is made current for the call, so the
    blocks belong to it and a scratch tensor dropped on return (its kernels still queued) can only be reused by
    work queued behind them.  ``stream`` may be a ``torch.cuda.Stream`` or a raw ``hipStream_t`` handle."""
    @functools.wraps(fn)
    def wrapper(*args, stream=None, **kwargs):
        if stream is None:
            return fn(*args, stream=None, **kwargs)
        if isinstance(stream, torch.cuda.Stream):
            s = stream
        else:
            s = torch.cuda.ExternalStream(int(stream)) if int(stream) else torch.cuda.default_stream()
        with torch.cuda.stream(s):
            return fn(*args, stream=s.cuda_stream, **kwargs)
    return wrapper


def device_info(device: int = 0) -> dict:
    L = _lib.load()
    name = ctypes.create_string_buffer(64)
    cu, lds, clk = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    hbm = ctypes.c_size_t()
    _raise(L.tyr_hip_device_info(device, name, 64, ctypes.byref(cu), ctypes.byref(lds), ctypes.byref(clk),
                                 ctypes.byref(hbm)), "device_info")
    return {"arch": name.value.decode(), "compute_units": cu.value, "lds_bytes_per_cu": lds.value,
            "clock_mhz": clk.value, "hbm_bytes": hbm.value}


def _key_mask_ptr(key_mask, B, N, window, kv_lens):
    """Device pointer of a [B, N] key mask (bool or uint8, nonzero = visible)."""
    if window or kv_lens is not None:
        raise TyrGpuError("a key mask cannot be combined with a window or key lengths")
    if not isinstance(key_mask, torch.Tensor):
        raise TyrGpuError("keyMask must be a tensor")
    if key_mask.dtype not in (torch.bool, torch.uint8):
        raise TyrGpuError("keyMask must have dtype torch.bool or torch.uint8")
    _check(key_mask, "keyMask", key_mask.dtype, 2)
    if tuple(key_mask.shape) != (B, N):
        raise TyrGpuError("keyMask must have shape [B, N]")
    return key_mask.data_ptr()


@_on_launch_stream
def flash_attn_fwd(q, k, v, causal: bool = True, scale: float | None = None, window: int = 0, kv_lens=None,
                   key_mask=None, stream=None):
    """O, LSE = flashAttnFwd q k v causal scale.

    q bf16 [B,Hq,N,D]; k, v bf16 [B,Hkv,N,D] with Hq % Hkv == 0 (query head h reads kv head h / (Hq/Hkv));
    ``window`` > 0 (causal only) lets query i see keys (i - window, i]; ``kv_lens`` (int32 [B] on the device)
    masks the keys at or beyond each sequence's length; ``key_mask`` (bool / uint8 [B,N] on the device, nonzero =
    visible) hides any set of keys per sequence instead.  -> (bf16 [B,Hq,N,D], f32 [B,Hq,N])."""
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _check(t, n, torch.bfloat16, 4)
    B, Hq, N, D = q.shape
    if k.shape != v.shape or k.shape[0] != B or k.shape[2] != N or k.shape[3] != D:
        raise TyrGpuError("k, v must have shape [B, Hkv, N, D] matching q's B, N, D")
    Hkv = k.shape[1]
    if Hkv == 0 or Hq % Hkv != 0:
        raise TyrGpuError("the number of query heads must be a multiple of the number of kv heads")
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lens_ptr = None
    if kv_lens is not None:
        _check(kv_lens, "kvLens", torch.int32, 1)
        if kv_lens.numel() != B:
            raise TyrGpuError("kvLens must hold one length per sequence")
        lens_ptr = kv_lens.data_ptr()
    o = torch.empty_like(q)
    lse = torch.empty((B, Hq, N), dtype=torch.float32, device=q.device)
    if key_mask is not None:
        rc = _lib.load().tyr_hip_flash_attn_fwd_mask(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                     lse.data_ptr(), B, Hq, Hkv, N, D, int(bool(causal)),
                                                     _key_mask_ptr(key_mask, B, N, window, kv_lens), float(scale),
                                                     _stream(stream))
        _raise(rc, "flashAttnFwd")
        return o, lse
    rc = _lib.load().tyr_hip_flash_attn_fwd_gqa(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                lse.data_ptr(), B, Hq, Hkv, N, D, int(bool(causal)), int(window),
                                                lens_ptr, float(scale), _stream(stream))
    _raise(rc, "flashAttnFwd")
    return o, lse


@_on_launch_stream
def flash_attn_bwd(q, k, v, o, lse, d_o, causal: bool = True, scale: float | None = None, window: int = 0,
                   kv_lens=None, key_mask=None, stream=None):
    """dQ, dK, dV = flashAttnBwd q k v o lse dO causal scale.

    q, o, d_o bf16 [B,Hq,N,D]; k, v bf16 [B,Hkv,N,D]; lse f32 [B,Hq,N]; o and lse as returned by
    flash_attn_fwd for the same q, k, v, causal, scale, window, kv_lens and key_mask.  Returns dQ [B,Hq,N,D] and
    dK, dV [B,Hkv,N,D] (summed over the query heads of each kv head), bf16."""
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (o, "o"), (d_o, "dO")):
        _check(t, n, torch.bfloat16, 4)
    if o.shape != q.shape or d_o.shape != q.shape or k.shape != v.shape:
        raise TyrGpuError("q, o, dO must have the same shape [B, Hq, N, D] and k, v the same shape [B, Hkv, N, D]")
    _check(lse, "lse", torch.float32, 3)
    B, Hq, N, D = q.shape
    if k.shape[0] != B or k.shape[2] != N or k.shape[3] != D:
        raise TyrGpuError("q, k, v, o, dO must have the same shape [B, H, N, D] (k, v may have fewer heads)")
    Hkv = k.shape[1]
    if Hkv == 0 or Hq % Hkv != 0:
        raise TyrGpuError("the number of query heads must be a multiple of the number of kv heads")
    if tuple(lse.shape) != (B, Hq, N):
        raise TyrGpuError("lse must have shape [B, H, N]")
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lens_ptr = None
    if kv_lens is not None:
        _check(kv_lens, "kvLens", torch.int32, 1)
        if kv_lens.numel() != B:
            raise TyrGpuError("kvLens must hold one length per sequence")
        lens_ptr = kv_lens.data_ptr()
    lib = _lib.load()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(k)
    nbytes = lib.tyr_hip_flash_attn_bwd_workspace_bytes(B, Hq, N, D)
    ws = torch.empty((max(int(nbytes), 16),), dtype=torch.uint8, device=q.device)
    if key_mask is not None:
        rc = lib.tyr_hip_flash_attn_bwd_mask(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                                             lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, Hq, Hkv, N,
                                             D, int(bool(causal)), _key_mask_ptr(key_mask, B, N, window, kv_lens),
                                             float(scale), ws.data_ptr(), ws.numel(), _stream(stream))
        _raise(rc, "flashAttnBwd")
        return dq, dk, dv
    rc = lib.tyr_hip_flash_attn_bwd_gqa(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                                        lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, Hq, Hkv, N, D,
                                        int(bool(causal)), int(window), lens_ptr, float(scale), ws.data_ptr(),
                                        ws.numel(), _stream(stream))
    _raise(rc, "flashAttnBwd")
    return dq, dk, dv


@_on_launch_stream
def gqa_decode(q, k, v, scale: float | None = None, num_splits: int = 0, kv_len: int | None = None,
               kv_lens=None, window: int = 0, stream=None):
    """O, LSE = gqaDecode q k v scale numSplits.

    q bf16 [B,Hq,1,D]; k, v bf16 [B,Hkv,Lmax,D] (the preallocated cache); the first ``kv_len``
    rows (default all) of every (batch, kv head) are attended to.  ``kv_lens`` (int32 [B] on the device)
    gives every sequence its own length in [0, kv_len] (a length of 0 yields O = 0, LSE = -inf); ``window`` > 0 restricts each sequence to its last
    ``window`` rows.  -> (bf16 [B,Hq,1,D], f32 [B,Hq]).
    """
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _check(t, n, torch.bfloat16, 4)
    B, Hq, one, D = q.shape
    if one != 1:
        raise TyrGpuError("q must have shape [B, Hq, 1, D]")
    if k.shape != v.shape or k.shape[0] != B or k.shape[3] != D:
        raise TyrGpuError("k, v must have shape [B, Hkv, L, D]")
    Hkv, Lmax = k.shape[1], k.shape[2]
    L = Lmax if kv_len is None else int(kv_len)
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    o = torch.empty_like(q)
    lse = torch.empty((B, Hq), dtype=torch.float32, device=q.device)
    nbytes = lib.tyr_hip_gqa_decode_workspace_bytes(B, Hq, max(Hkv, 1), max(L, 1), D, int(num_splits))
    ws = torch.empty((max(int(nbytes), 16),), dtype=torch.uint8, device=q.device)
    lens_ptr = None
    if kv_lens is not None:
        _check(kv_lens, "kvLens", torch.int32, 1)
        if kv_lens.numel() != B:
            raise TyrGpuError("kvLens must hold one length per sequence")
        lens_ptr = kv_lens.data_ptr()
    rc = lib.tyr_hip_gqa_decode_varlen(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                       B, Hq, Hkv, L, D, Lmax, lens_ptr, int(window), float(scale),
                                       int(num_splits), ws.data_ptr(), ws.numel(), _stream(stream))
    _raise(rc, "gqaDecode")
    return o, lse


@_on_launch_stream
def decode_rope_append(q, k_new, v_new, cos, sin, k_cache, v_cache, pos: int, stream=None):
    """qRot = decodeRopeAppend q kNew vNew cos sin kCache vCache pos.

    q bf16 [B,Hq,1,D] (or [B,1,Hq,D]); k_new, v_new bf16 [B,Hkv,1,D]; cos, sin f32 [1,D/2] (or [D/2]) for
    position ``pos``; caches bf16 [B,Hkv,maxLen,D], row ``pos`` of each is overwritten in place.  Returns the
    rotated q with q's shape."""
    for t, n in ((q, "q"), (k_new, "kNew"), (v_new, "vNew"), (k_cache, "kCache"), (v_cache, "vCache")):
        _check(t, n, torch.bfloat16, 4)
    _check(cos, "cos", torch.float32)
    _check(sin, "sin", torch.float32)
    B, Hkv, Lmax, D = k_cache.shape
    if v_cache.shape != k_cache.shape:
        raise TyrGpuError("k and v caches must have the same shape")
    if q.shape[0] != B or q.shape[-1] != D or q.shape[1] * q.shape[2] * B * D != q.numel() or 1 not in q.shape[1:3]:
        raise TyrGpuError("q must be [B, Hq, 1, D] or [B, 1, Hq, D]")
    Hq = q.shape[1] * q.shape[2]
    for t in (k_new, v_new):
        if t.numel() != B * Hkv * D or t.shape[-1] != D:
            raise TyrGpuError("kNew and vNew must hold B*Hkv rows of D elements")
    if cos.numel() != D // 2 or sin.numel() != D // 2:
        raise TyrGpuError("cos and sin must hold D/2 elements (the table row of this position)")
    if not 0 <= pos < Lmax:
        raise TyrGpuError("pos is outside the cache")
    q_out = torch.empty_like(q)
    rc = _lib.load().tyr_hip_decode_rope_append(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), cos.data_ptr(),
                                                sin.data_ptr(), q_out.data_ptr(), k_cache.data_ptr(),
                                                v_cache.data_ptr(), B, Hq, Hkv, D, Lmax, int(pos), _stream(stream))
    _raise(rc, "decodeRopeAppend")
    return q_out


@_on_launch_stream
def rope_fwd(x, cos, sin, stream=None):
    """y = applyRotaryEmb x cos sin.  x f32 or bf16 [B,S,H,D]; cos, sin f32 [S,D/2]."""
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise TyrGpuError("x must have dtype float32 or bfloat16")
    _check(x, "x", x.dtype, 4)
    _check(cos, "cos", torch.float32, 2)
    _check(sin, "sin", torch.float32, 2)
    B, S, H, D = x.shape
    if tuple(cos.shape) != (S, D // 2) or tuple(sin.shape) != (S, D // 2):
        raise TyrGpuError("cos and sin must have shape [S, D/2]")
    y = torch.empty_like(x)
    rc = _lib.load().tyr_hip_rope_fwd(x.data_ptr(), cos.data_ptr(), sin.data_ptr(), y.data_ptr(), B, S, H, D,
                                      1 if x.dtype == torch.bfloat16 else 0, _stream(stream))
    _raise(rc, "applyRotaryEmb")
    return y


@_on_launch_stream
def layernorm_residual(x, residual, weight, bias, eps: float = 1e-5, stream=None):
    """(out, outResid) = fusedLayerNormResidual x residual weight bias.  bf16; x, residual [..., d]; weight, bias [d]."""
    for t, n in ((x, "x"), (residual, "residual"), (weight, "weight"), (bias, "bias")):
        _check(t, n, torch.bfloat16)
    d = x.shape[-1]
    if residual.shape != x.shape or tuple(weight.shape) != (d,) or tuple(bias.shape) != (d,):
        raise TyrGpuError("residual must match x, weight and bias must be [d_model]")
    out, out_resid = torch.empty_like(x), torch.empty_like(x)
    rc = _lib.load().tyr_hip_layernorm_residual(x.data_ptr(), residual.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                                out.data_ptr(), out_resid.data_ptr(), x.numel() // d, d, float(eps),
                                                _stream(stream))
    _raise(rc, "fusedLayerNormResidual")
    return out, out_resid


@_on_launch_stream
def copy(src, stream=None):
    """out = copy src (any dtype, contiguous)."""
    _check(src, "input", src.dtype)
    dst = torch.empty_like(src)
    rc = _lib.load().tyr_hip_copy(src.data_ptr(), dst.data_ptr(), src.numel() * src.element_size(), _stream(stream))
    _raise(rc, "copy")
    return dst


@_on_launch_stream
def matmul_bf16(a, b, trans_b: bool = False, stream=None):
    """C = matmul a b for operands of rank > 2 (`lean_torch_matmul`): a bf16 [..., M, K]; b bf16 [..., K, N] with
    the same leading extents, or a plain [K, N] matrix used for every batch entry (b is [..., N, K] / [N, K] with
    trans_b) -> bf16 [..., M, N]."""
    _check(a, "a", torch.bfloat16)
    _check(b, "b", torch.bfloat16)
    if a.dim() < 2 or b.dim() < 2:
        raise TyrGpuError("a and b must have dim >= 2")
    if a.dim() == 2 and b.dim() == 2:
        return gemm_bf16(a, b, trans_b, stream=stream)
    if b.dim() != 2 and (b.dim() != a.dim() or b.shape[:-2] != a.shape[:-2]):
        raise TyrGpuError("b must be a matrix or share a's leading extents")
    if a.dim() == 2:
        raise TyrGpuError("a must carry the batch extents")
    M, K = a.shape[-2:]
    N, Kb = (b.shape[-2], b.shape[-1]) if trans_b else (b.shape[-1], b.shape[-2])
    if Kb != K:
        raise TyrGpuError("a and b have mismatched inner dimensions")
    batch = a.numel() // (M * K) if M * K else 0
    c = torch.empty(tuple(a.shape[:-2]) + (M, N), dtype=torch.bfloat16, device=a.device)
    rc = _lib.load().tyr_hip_gemm_bf16_batched(a.data_ptr(), b.data_ptr(), c.data_ptr(), batch, M, N, K, M * K,
                                               0 if b.dim() == 2 else K * N, M * N, int(bool(trans_b)),
                                               _stream(stream))
    _raise(rc, "matmul")
    return c


@_on_launch_stream
def gemm_bf16(a, b, trans_b: bool = False, stream=None):
    """C = gemmBf16 a b.  a bf16 [M,K]; b bf16 [K,N] (or [N,K] with trans_b) -> bf16 [M,N]."""
    _check(a, "a", torch.bfloat16, 2)
    _check(b, "b", torch.bfloat16, 2)
    M, K = a.shape
    N, Kb = (b.shape[0], b.shape[1]) if trans_b else (b.shape[1], b.shape[0])
    if Kb != K:
        raise TyrGpuError("a and b have mismatched inner dimensions")
    c = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    rc = _lib.load().tyr_hip_gemm_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, int(bool(trans_b)),
                                       _stream(stream))
    _raise(rc, "gemmBf16")
    return c


@_on_launch_stream
def gemm_fp8(aq, bq, scale_a: float, scale_b: float, trans_b: bool = False, stream=None):
    """C = gemmFp8 aq bq scaleA scaleB.  aq e4m3 [M,K]; bq e4m3 [K,N] (or [N,K]) -> bf16 [M,N]."""
    _check(aq, "a", torch.float8_e4m3fn, 2)
    _check(bq, "b", torch.float8_e4m3fn, 2)
    M, K = aq.shape
    N, Kb = (bq.shape[0], bq.shape[1]) if trans_b else (bq.shape[1], bq.shape[0])
    if Kb != K:
        raise TyrGpuError("a and b have mismatched inner dimensions")
    c = torch.empty((M, N), dtype=torch.bfloat16, device=aq.device)
    rc = _lib.load().tyr_hip_gemm_fp8(aq.data_ptr(), bq.data_ptr(), c.data_ptr(), M, N, K, float(scale_a),
                                      float(scale_b), int(bool(trans_b)), _stream(stream))
    _raise(rc, "gemmFp8")
    return c


@_on_launch_stream
def gemm_fp8_scaled(aq, bq, row_scale=None, col_scale=None, scale: float = 1.0, out_dtype=torch.float32,
                    trans_b: bool = False, stream=None):
    """C = gemmFp8Scaled aq bq rowScale colScale: out_dtype(scale * rowScale[m] * colScale[n] * (aq bq)[m, n]).

    The per-row / per-column dequantisation epilogue of `tkH100Fp8ScaledGemmFwd` (f32 out) and, with no scales and
    out_dtype = torch.float8_e4m3fn, the E4M3 epilogue of `tkH100Fp8E4M3GemmFwd`.  aq e4m3 [M,K]; bq e4m3 [K,N] (or
    [N,K] with trans_b); row_scale f32 [M], col_scale f32 [N] or None."""
    _check(aq, "a", torch.float8_e4m3fn, 2)
    _check(bq, "b", torch.float8_e4m3fn, 2)
    M, K = aq.shape
    N, Kb = (bq.shape[0], bq.shape[1]) if trans_b else (bq.shape[1], bq.shape[0])
    if Kb != K:
        raise TyrGpuError("a and b have mismatched inner dimensions")
    kinds = {torch.bfloat16: 0, torch.float32: 1, torch.float8_e4m3fn: 2}
    if out_dtype not in kinds:
        raise TyrGpuError("out_dtype must be bfloat16, float32 or float8_e4m3fn")
    ptrs = []
    for t, n, ln in ((row_scale, "rowScale", M), (col_scale, "colScale", N)):
        if t is None:
            ptrs.append(None)
            continue
        _check(t, n, torch.float32, 1)
        if t.numel() != ln:
            raise TyrGpuError(f"{n} must hold one scale per {'row' if ln == M else 'column'}")
        ptrs.append(t.data_ptr())
    c = torch.empty((M, N), dtype=out_dtype, device=aq.device)
    rc = _lib.load().tyr_hip_gemm_fp8_ex(aq.data_ptr(), bq.data_ptr(), c.data_ptr(), M, N, K, float(scale), ptrs[0], ptrs[1],
                                         kinds[out_dtype], int(bool(trans_b)), _stream(stream))
    _raise(rc, "gemmFp8Scaled")
    return c


@_on_launch_stream
def mse_loss_grad(out, target, stream=None):
    """(loss, dO) = lossAndGradOut out target: loss = 0.5 mean((out - target)^2) as an f32 scalar tensor,
    dO = bf16((out - target) / numel).  out, target bf16, same shape, numel % 8 == 0."""
    _check(out, "out", torch.bfloat16)
    _check(target, "target", torch.bfloat16)
    if out.shape != target.shape:
        raise TyrGpuError("out and target must have the same shape")
    lib = _lib.load()
    n = out.numel()
    d_out = torch.empty_like(out)
    loss = torch.empty((), dtype=torch.float32, device=out.device)
    ws = torch.empty((max(int(lib.tyr_hip_mse_loss_grad_workspace_bytes(n)), 16),), dtype=torch.uint8, device=out.device)
    rc = lib.tyr_hip_mse_loss_grad(out.data_ptr(), target.data_ptr(), d_out.data_ptr(), loss.data_ptr(), n, ws.data_ptr(),
                                   ws.numel(), _stream(stream))
    _raise(rc, "lossAndGradOut")
    return loss, d_out


@_on_launch_stream
def sgd_step(param, grad, lr: float, in_place: bool = False, stream=None):
    """(param', bf16 param') = sgdUpdate param grad lr: param' = param - f32(grad) * lr for an f32 master and a bf16
    gradient of the same shape, together with the bf16 cast the next step's kernels take.  ``in_place`` overwrites
    ``param`` instead of allocating."""
    _check(param, "param", torch.float32)
    _check(grad, "grad", torch.bfloat16)
    if param.shape != grad.shape:
        raise TyrGpuError("param and grad must have the same shape")
    out = param if in_place else torch.empty_like(param)
    out_bf16 = torch.empty_like(grad)
    rc = _lib.load().tyr_hip_sgd_step(param.data_ptr(), grad.data_ptr(), float(lr), out.data_ptr(), out_bf16.data_ptr(),
                                      param.numel(), _stream(stream))
    _raise(rc, "sgdUpdate")
    return out, out_bf16


def quantize_e4m3(x: torch.Tensor):
    """Per-tensor absmax quantisation used by the harness: s = absmax/448, xq = e4m3fn(x / s)."""
    s = float(x.abs().max()) / 448.0
    if s == 0.0:
        s = 1.0
    xq = (x.float() / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return xq, s
