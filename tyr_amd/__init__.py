"""tyr_amd -- MI355X (gfx950) kernels behind Tyr's GPU surface.

The product is ``lib/libtyr_hip.so`` (hand-written HIP kernels + C ABI, declared in
``include/tyr_hip.h``).  ``tyr_amd.gpu`` is the host-side mirror of the Lean entry points
(``lean/Tyr/GPU/GFX950.lean``) for callers that hold torch tensors; it only moves pointers.
"""
from .gpu import (TyrGpuError, flash_attn_fwd, flash_attn_bwd, gqa_decode, gemm_bf16, matmul_bf16, gemm_fp8, gemm_fp8_scaled, mse_loss_grad, sgd_step,
                  decode_rope_append, rope_fwd, layernorm_residual, copy, quantize_e4m3, device_info, library_path)

__all__ = ["TyrGpuError", "flash_attn_fwd", "flash_attn_bwd", "gqa_decode", "gemm_bf16", "matmul_bf16", "gemm_fp8", "gemm_fp8_scaled", "mse_loss_grad", "sgd_step",
           "decode_rope_append", "rope_fwd", "layernorm_residual", "copy", "quantize_e4m3", "device_info", "library_path"]
