"""The C-ABI library: it loads, exports every symbol include/tyr_hip.h declares, and its host-side
validation rejects bad arguments before touching a GPU (so these run without one)."""
import ctypes
import os
import re

import pytest

from tyr_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tyr_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tyr_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.SYMBOLS)


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name


def test_strerror_and_version():
    L = _lib.load()
    assert L.tyr_hip_version() >= 100
    assert L.tyr_hip_strerror(0) == b"ok"
    for code in range(-8, 0):
        assert L.tyr_hip_strerror(code) not in (b"", b"unknown tyr_hip status")
    assert b"CUDA tensor" in L.tyr_hip_strerror(-8)      # the reference launcher's wording
    assert L.tyr_hip_strerror(-99) == b"unknown tyr_hip status"


def test_host_validation_needs_no_gpu():
    L = _lib.load()
    p = 0x1000  # never dereferenced: every call below must fail validation first
    OK, NULL, SHAPE, UNSUP, MISAL, WS = 0, -1, -2, -3, -4, -5
    assert L.tyr_hip_gemm_bf16(None, p, p, 8, 8, 8, 0, None) == NULL
    assert L.tyr_hip_gemm_bf16(p, p, p, 0, 8, 8, 0, None) == SHAPE
    assert L.tyr_hip_gemm_bf16(p, p, p, 8, 8, 12, 0, None) == UNSUP
    assert L.tyr_hip_gemm_bf16(p + 2, p, p, 8, 8, 8, 0, None) == MISAL
    assert L.tyr_hip_gemm_bf16(p, p, p, 2 ** 40, 8, 8, 0, None) == SHAPE
    assert L.tyr_hip_gemm_bf16_batched(p, p, p, 0, 8, 8, 8, 64, 64, 64, 0, None) == SHAPE
    assert L.tyr_hip_gemm_bf16_batched(p, p, p, 2, 8, 8, 8, 64, 64, 32, 0, None) == SHAPE      # outputs would overlap
    assert L.tyr_hip_gemm_bf16_batched(p, p, p, 2, 8, 8, 8, 68, 64, 64, 0, None) == MISAL
    assert L.tyr_hip_gemm_bf16_batched(p, p, p, 70000, 8, 8, 8, 64, 64, 64, 0, None) == SHAPE
    prev = L.tyr_hip_gemm_force_general(1)
    assert L.tyr_hip_gemm_force_general(prev) == 1 and L.tyr_hip_gemm_force_general(prev) == prev
    prev = L.tyr_hip_flash_attn_fwd_persistent(1)
    assert L.tyr_hip_flash_attn_fwd_persistent(prev) == 1 and L.tyr_hip_flash_attn_fwd_persistent(prev) == prev
    # the calibration loop writes 256 floats per workgroup: a smaller sink is refused before any launch
    assert L.tyr_hip_mfma_sustain(p, 1 << 20, 0, 256, 10, p, 256 * 256 * 4 - 1, None, None) == WS
    assert L.tyr_hip_gemm_fp8(p, p, None, 16, 16, 16, 1.0, 1.0, 0, None) == NULL
    assert L.tyr_hip_gemm_fp8(p, p, p, 16, 8, 16, 1.0, 1.0, 0, None) == UNSUP
    assert L.tyr_hip_gemm_fp8_ex(p, p, p, 16, 16, 16, 1.0, None, None, 7, 0, None) == UNSUP           # unknown output type
    assert L.tyr_hip_gemm_fp8_ex(p, p, p, 16, 16, 16, 1.0, None, p + 4, 1, 0, None) == MISAL          # column scales: 16-byte rows
    assert L.tyr_hip_flash_attn_fwd(p, p, None, p, None, 1, 1, 16, 128, 1, 0.1, None) == NULL
    assert L.tyr_hip_flash_attn_fwd(p, p, p, p, None, 1, 1, 0, 128, 1, 0.1, None) == SHAPE
    assert L.tyr_hip_flash_attn_fwd(p, p, p, p, None, 1, 1, 16, 96, 1, 0.1, None) == UNSUP
    assert L.tyr_hip_flash_attn_fwd(p, p, p, p, None, 1, 1, 16, 128, 1, -1.0, None) == UNSUP
    assert L.tyr_hip_flash_attn_fwd(p, p, p + 8, p, None, 1, 1, 16, 128, 1, 0.1, None) == MISAL
    assert L.tyr_hip_gqa_decode(p, p, p, p, None, 1, 6, 4, 16, 128, 16, 0.1, 1, p, 1 << 20, None) == SHAPE   # Hq % Hkv
    assert L.tyr_hip_gqa_decode(p, p, p, p, None, 1, 8, 2, 16, 128, 8, 0.1, 1, p, 1 << 20, None) == SHAPE   # stride < L
    assert L.tyr_hip_gqa_decode(p, p, p, p, None, 1, 8, 2, 16, 96, 16, 0.1, 1, p, 1 << 20, None) == UNSUP
    assert L.tyr_hip_gqa_decode(p, p, p, p, None, 1, 8, 2, 16, 128, 16, 0.1, 1, None, 0, None) == WS
    assert L.tyr_hip_gqa_decode(p, p, p, p, None, 1, 8, 2, 16, 128, 16, 0.1, 1, p, 64, None) == WS
    assert L.tyr_hip_gqa_decode_workspace_bytes(2, 8, 2, 1000, 128, 4) == 2 * 8 * 4 * 130 * 4
    assert 1 <= L.tyr_hip_gqa_decode_auto_splits(32, 8, 8192) <= 64
    assert L.tyr_hip_gqa_decode_auto_splits(1, 1, 10) == 1
    assert OK == 0


def test_python_mirror_refuses_cpu_tensors_without_a_gpu():
    import torch
    import tyr_amd
    a = torch.zeros(16, 16, dtype=torch.bfloat16)
    with pytest.raises(tyr_amd.TyrGpuError, match="a must be a CUDA tensor"):
        tyr_amd.gemm_bf16(a, a)
    with pytest.raises(tyr_amd.TyrGpuError, match="q must be a CUDA tensor"):
        tyr_amd.flash_attn_fwd(a.view(1, 1, 16, 16), a.view(1, 1, 16, 16), a.view(1, 1, 16, 16))
