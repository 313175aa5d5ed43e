"""ctypes binding of libtyr_hip.so.  There is no fallback: a missing library is an error."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TYR_HIP_LIBRARY overrides the location (e.g. to try an experimental build); there is still no fallback.
LIB_PATH = os.environ.get("TYR_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libtyr_hip.so")

# every symbol include/tyr_hip.h declares
SYMBOLS = (
    "tyr_hip_strerror", "tyr_hip_version", "tyr_hip_device_info", "tyr_hip_check_device_pointer",
    "tyr_hip_flash_attn_fwd", "tyr_hip_flash_attn_fwd_gqa", "tyr_hip_flash_attn_bwd_workspace_bytes", "tyr_hip_flash_attn_bwd",
    "tyr_hip_flash_attn_bwd_gqa", "tyr_hip_flash_attn_fwd_mask", "tyr_hip_flash_attn_bwd_mask",
    "tyr_hip_gqa_decode_workspace_bytes", "tyr_hip_gqa_decode_auto_splits",
    "tyr_hip_gqa_decode", "tyr_hip_gqa_decode_varlen", "tyr_hip_gqa_decode_static", "tyr_hip_gemm_bf16", "tyr_hip_gemm_bf16_batched", "tyr_hip_gemm_force_general", "tyr_hip_flash_attn_fwd_persistent", "tyr_hip_gemm_fp8", "tyr_hip_gemm_fp8_ex",
    "tyr_hip_decode_rope_append", "tyr_hip_rope_fwd", "tyr_hip_layernorm_residual", "tyr_hip_copy", "tyr_hip_mfma_sustain", "tyr_hip_mse_loss_grad_workspace_bytes", "tyr_hip_mse_loss_grad", "tyr_hip_sgd_step",
)

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C tyr_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "tyr_amd has no CPU or PyTorch fallback.")
    L = ctypes.CDLL(LIB_PATH)
    u64, vp, ci, f32, sz = ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    L.tyr_hip_strerror.argtypes = [ci]
    L.tyr_hip_strerror.restype = ctypes.c_char_p
    L.tyr_hip_version.argtypes = []
    L.tyr_hip_version.restype = ci
    L.tyr_hip_device_info.argtypes = [ci, ctypes.c_char_p, sz, ctypes.POINTER(ci), ctypes.POINTER(ci),
                                      ctypes.POINTER(ci), ctypes.POINTER(sz)]
    L.tyr_hip_device_info.restype = ci
    L.tyr_hip_check_device_pointer.argtypes = [vp]
    L.tyr_hip_check_device_pointer.restype = ci
    L.tyr_hip_flash_attn_fwd.argtypes = [vp, vp, vp, vp, vp, u64, u64, u64, u64, ci, f32, vp]
    L.tyr_hip_flash_attn_fwd.restype = ci
    L.tyr_hip_flash_attn_fwd_gqa.argtypes = [vp, vp, vp, vp, vp, u64, u64, u64, u64, u64, ci, u64, vp, f32, vp]
    L.tyr_hip_flash_attn_fwd_gqa.restype = ci
    L.tyr_hip_flash_attn_bwd_workspace_bytes.argtypes = [u64] * 4
    L.tyr_hip_flash_attn_bwd_workspace_bytes.restype = sz
    L.tyr_hip_flash_attn_bwd.argtypes = [vp] * 9 + [u64] * 4 + [ci, f32, vp, sz, vp]
    L.tyr_hip_flash_attn_bwd.restype = ci
    L.tyr_hip_flash_attn_bwd_gqa.argtypes = [vp] * 9 + [u64] * 5 + [ci, u64, vp, f32, vp, sz, vp]
    L.tyr_hip_flash_attn_bwd_gqa.restype = ci
    L.tyr_hip_flash_attn_fwd_mask.argtypes = [vp, vp, vp, vp, vp, u64, u64, u64, u64, u64, ci, vp, f32, vp]
    L.tyr_hip_flash_attn_fwd_mask.restype = ci
    L.tyr_hip_flash_attn_bwd_mask.argtypes = [vp] * 9 + [u64] * 5 + [ci, vp, f32, vp, sz, vp]
    L.tyr_hip_flash_attn_bwd_mask.restype = ci
    L.tyr_hip_gqa_decode_workspace_bytes.argtypes = [u64] * 6
    L.tyr_hip_gqa_decode_workspace_bytes.restype = sz
    L.tyr_hip_gqa_decode_auto_splits.argtypes = [u64] * 3
    L.tyr_hip_gqa_decode_auto_splits.restype = u64
    L.tyr_hip_gqa_decode.argtypes = [vp, vp, vp, vp, vp, u64, u64, u64, u64, u64, u64, f32, u64, vp, sz, vp]
    L.tyr_hip_gqa_decode.restype = ci
    L.tyr_hip_gqa_decode_varlen.argtypes = [vp, vp, vp, vp, vp, u64, u64, u64, u64, u64, u64, vp, u64, f32, u64, vp, sz, vp]
    L.tyr_hip_gqa_decode_varlen.restype = ci
    L.tyr_hip_gqa_decode_static.argtypes = [vp, vp, vp, vp, vp, u64, u64, u64, u64, u64, u64, f32, u64, vp]
    L.tyr_hip_gqa_decode_static.restype = ci
    L.tyr_hip_gemm_bf16.argtypes = [vp, vp, vp, u64, u64, u64, ci, vp]
    L.tyr_hip_gemm_bf16.restype = ci
    L.tyr_hip_gemm_bf16_batched.argtypes = [vp, vp, vp, u64, u64, u64, u64, u64, u64, u64, ci, vp]
    L.tyr_hip_gemm_bf16_batched.restype = ci
    L.tyr_hip_gemm_force_general.argtypes = [ci]
    L.tyr_hip_gemm_force_general.restype = ci
    L.tyr_hip_flash_attn_fwd_persistent.argtypes = [ci]
    L.tyr_hip_flash_attn_fwd_persistent.restype = ci
    L.tyr_hip_gemm_fp8.argtypes = [vp, vp, vp, u64, u64, u64, f32, f32, ci, vp]
    L.tyr_hip_gemm_fp8.restype = ci
    L.tyr_hip_gemm_fp8_ex.argtypes = [vp, vp, vp, u64, u64, u64, f32, vp, vp, ci, ci, vp]
    L.tyr_hip_gemm_fp8_ex.restype = ci
    L.tyr_hip_decode_rope_append.argtypes = [vp] * 8 + [u64] * 6 + [vp]
    L.tyr_hip_decode_rope_append.restype = ci
    L.tyr_hip_rope_fwd.argtypes = [vp, vp, vp, vp, u64, u64, u64, u64, ci, vp]
    L.tyr_hip_rope_fwd.restype = ci
    L.tyr_hip_layernorm_residual.argtypes = [vp] * 6 + [u64, u64, f32, vp]
    L.tyr_hip_layernorm_residual.restype = ci
    L.tyr_hip_copy.argtypes = [vp, vp, sz, vp]
    L.tyr_hip_copy.restype = ci
    L.tyr_hip_mfma_sustain.argtypes = [vp, sz, ci, u64, u64, vp, sz, ctypes.POINTER(ctypes.c_double), vp]
    L.tyr_hip_mfma_sustain.restype = ci
    L.tyr_hip_mse_loss_grad_workspace_bytes.argtypes = [u64]
    L.tyr_hip_mse_loss_grad_workspace_bytes.restype = sz
    L.tyr_hip_mse_loss_grad.argtypes = [vp, vp, vp, vp, u64, vp, sz, vp]
    L.tyr_hip_mse_loss_grad.restype = ci
    L.tyr_hip_sgd_step.argtypes = [vp, vp, f32, vp, vp, u64, vp]
    L.tyr_hip_sgd_step.restype = ci
    _lib = L
    return L
