"""Launches emitted tile programs through their C-ABI launchers (`tyr_launch_<kernel>` in
libtyr_dsl.so).  Mirrors `<kernel>.launch tensors… scalars… grid block sharedMem stream` of the
reference (Tyr/GPU/Codegen/Attribute.lean:388-437) including its argument checks and messages
(Attribute.lean:334-336).  There is no fallback: a missing library is an error."""
from __future__ import annotations

import ctypes
import os

from .build import LIB_PATH
from .ir import Kernel

_libs = {}
_CT = {"UInt8": ctypes.c_uint8, "UInt16": ctypes.c_uint16, "UInt32": ctypes.c_uint32, "UInt64": ctypes.c_uint64,
       "USize": ctypes.c_size_t, "Float": ctypes.c_double, "Float32": ctypes.c_float, "Bool": ctypes.c_uint8}
_TORCH_DTYPE = {"Float32": "float32", "BFloat16": "bfloat16", "Float16": "float16", "FP8E4M3": "float8_e4m3fn"}


def load(path: str = LIB_PATH) -> ctypes.CDLL:
    if path not in _libs:
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python -m tyr_amd.dsl.build`. "
                               "Emitted kernels have no CPU fallback.")
        _libs[path] = ctypes.CDLL(path)
    return _libs[path]


def launch(kernel: Kernel, args, grid=(1, 1, 1), block=(128, 1, 1), shared_mem: int = 0, stream=None,
           library: ctypes.CDLL = None) -> None:
    """args: one entry per kernel parameter, in order -- a CUDA tensor for a pointer, a number for a scalar."""
    import torch
    if len(args) != len(kernel.params):
        raise TypeError(f"{kernel.name} takes {len(kernel.params)} arguments, got {len(args)}")
    fn = getattr(library if library is not None else load(), f"tyr_launch_{kernel.name}")
    cargs, ctypes_sig, keep = [], [], []
    for p, a in zip(kernel.params, args):
        if p.isPointer:
            if not isinstance(a, torch.Tensor) or not a.is_cuda:
                raise RuntimeError(f"{p.name} must be a CUDA tensor")
            if not a.is_contiguous():
                raise RuntimeError(f"{p.name} must be contiguous")
            if a.dim() > 4:
                raise RuntimeError(f"{p.name} must have dim <= 4")
            if a.dtype != getattr(torch, _TORCH_DTYPE[p.dtype]):
                raise RuntimeError(f"{p.name} must be {_TORCH_DTYPE[p.dtype]}")
            shape = (ctypes.c_int64 * 4)(*a.shape)
            keep.append(shape)
            cargs += [ctypes.c_void_p(a.data_ptr()), shape, ctypes.c_int(a.dim())]
            ctypes_sig += [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
        else:
            cargs.append(_CT[p.scalarTy](a))
            ctypes_sig.append(_CT[p.scalarTy])
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    cargs += [ctypes.c_uint64(int(x)) for x in (*grid, *block, shared_mem)] + [ctypes.c_void_p(stream)]
    ctypes_sig += [ctypes.c_uint64] * 7 + [ctypes.c_void_p]
    fn.argtypes, fn.restype = ctypes_sig, ctypes.c_int
    rc = fn(*cargs)
    if rc == -2:
        raise RuntimeError(f"invalid launch arguments for {kernel.name}")
    if rc != 0:
        raise RuntimeError(f"launch of {kernel.name} failed")
