"""Emits the tile programs of `tyr_amd.dsl.kernels` as one HIP translation unit and compiles it for
gfx950 into `tyr_amd/lib/libtyr_dsl.so` (the counterpart of the reference's generate-then-`make -C cc`
step, scripts/gpu/run_e2e_kernel.sh:54-64).  hipcc cross-compiles without a GPU."""
from __future__ import annotations

import os
import subprocess

from . import kernels
from .emit import emit_header, emit_translation_unit

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")
GEN_DIR = os.path.join(CSRC, "build", "dsl")
SRC_PATH = os.path.join(GEN_DIR, "tyr_dsl_kernels.hip")
LIB_PATH = os.path.join(_PKG, "lib", "libtyr_dsl.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
            "-packed-fp32-ops"]


def emit_sources(path: str = SRC_PATH, programs=kernels.ALL) -> str:
    os.makedirs(os.path.dirname(path), exist_ok=True)
    src = emit_translation_unit([f() for f in programs])
    with open(path, "w") as f:
        f.write(src)
    return path


HEADER_PATH = os.path.join(os.path.dirname(_PKG), "include", "tyr_dsl_kernels.h")


def header_text() -> str:
    return emit_header([f() for f in kernels.ALL], kernels.CITES)


def _compile(src: str, lib_path: str) -> str:
    os.makedirs(os.path.dirname(lib_path), exist_ok=True)
    cmd = [HIPCC] + HIPFLAGS + ["-I", CSRC, "-shared", src, "-o", lib_path]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on the emitted kernels:\n" + r.stderr[-4000:])
    return lib_path


def build(lib_path: str = LIB_PATH) -> str:
    return _compile(emit_sources(), lib_path)


def compile_programs(programs, src_path: str, lib_path: str) -> str:
    """Emits any list of tile programs (functions returning a Kernel) to `src_path` and compiles it to `lib_path`."""
    return _compile(emit_sources(src_path, programs), lib_path)


if __name__ == "__main__":
    with open(HEADER_PATH, "w") as f:
        f.write(header_text())
    print(HEADER_PATH)
    print(build())
