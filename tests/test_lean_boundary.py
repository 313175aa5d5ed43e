"""The Lean-facing half of the boundary, checked without a Lean toolchain (CPU only):
  * tyr_amd/csrc/lean_shim.cpp and the `lean_launch_*` wrappers the emitter prints type-check against
    the LibTorch headers of this image and a declarations-only <lean/lean.h> (tests/lean_stub/);
  * every `@[extern]` of GFX950.lean has a definition in the shim with the matching argument count;
  * the generated weak stubs (reference: cc/tools/generate_gpu_kernel_stubs.py:24-47) link, return the
    "unavailable in this build" IO.userError when called, and give way to a strong definition.
"""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STUB = os.path.join(ROOT, "tests", "lean_stub")
SHIM = os.path.join(ROOT, "tyr_amd", "csrc", "lean_shim.cpp")
LEAN = os.path.join(ROOT, "tyr_amd", "lean", "Tyr", "GPU", "GFX950.lean")
pytestmark = pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not installed")


def _torch_includes():
    from torch.utils import cpp_extension
    return [f"-I{p}" for p in cpp_extension.include_paths()]


def _syntax_only(path, extra=()):
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror=return-type", f"-I{STUB}", *_torch_includes(), "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__", *extra, path]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_lean_shim_type_checks_against_libtorch_and_the_lean_c_api():
    text = open(SHIM).read()
    assert "#ifdef TYR_HAVE_LEAN" in text
    _syntax_only(SHIM)
    # the check is not vacuous: the guarded half of the file is what got compiled
    r = subprocess.run(["g++", "-std=c++17", "-E", "-dM", f"-I{STUB}", *_torch_includes(), "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__", SHIM],
                       capture_output=True, text=True)
    assert "#define TYR_HAVE_LEAN 1" in r.stdout


def test_every_lean_extern_is_defined_by_the_shim_with_matching_arity():
    lean = open(LEAN).read()
    shim = open(SHIM).read()
    decls = re.findall(r'@\[extern\s+"(lean_tyr_gpu_\w+)"\]\s*opaque\s+\w+(.*?):\s*IO\b', lean, flags=re.S)
    assert len(decls) >= 15
    for sym, binders in decls:
        # Lean passes every binder (implicit ones first, in order) and a trailing world token
        n_lean = 0
        for grp in re.findall(r"[({]([^(){}]*?):[^(){}]*[)}]", binders):
            n_lean += len(grp.replace("@&", " ").split())
        m = re.search(r"lean_object\*\s+" + sym + r"\s*\((.*?)\)\s*\{", shim, flags=re.S)
        assert m, f"{sym} is declared in GFX950.lean but not defined in lean_shim.cpp"
        params = [p for p in re.sub(r"/\*.*?\*/", "", m.group(1), flags=re.S).split(",") if p.strip()]
        assert len(params) == n_lean + 1, (sym, n_lean, len(params))


def test_emitted_lean_launchers_type_check(tmp_path):
    from tyr_amd.dsl import kernels
    from tyr_amd.dsl.emit import LEAN_PREAMBLE, _Emitter
    ems = [_Emitter(f()) for f in kernels.ALL]
    # the launchers' own C-ABI twins are declared instead of defined: device code needs hipcc, this is a host check
    text = ("#include <stdint.h>\n#include <exception>\nextern \"C\" {\n" +
            "".join(e.launcher_signature() + ";\n" for e in ems) +
            "}\ntypedef int hipError_t;\nhipError_t hipGetLastError();\nconst char* hipGetErrorString(hipError_t);\n" +
            LEAN_PREAMBLE + "".join(e.lean_launcher_text() + "\n" for e in ems) + "#endif\n")
    assert text.count('extern "C" lean_object* lean_launch_') == len(ems)
    src = tmp_path / "lean_launchers.cpp"
    src.write_text(text)
    _syntax_only(str(src))


def test_weak_stubs_report_unavailable_and_yield_to_real_definitions(tmp_path):
    from tyr_amd.dsl import stubs
    syms = stubs.collect_symbols()
    assert "lean_tyr_gpu_flash_attn_fwd" in syms and "lean_launch_simpleGemm" in syms
    assert set(stubs.extern_symbols()) == set(re.findall(r"lean_object\*\s+(lean_tyr_gpu_\w+)\s*\(", open(SHIM).read()))
    gen = tmp_path / "gfx950_kernel_stubs.cpp"
    gen.write_text(stubs.render(syms))
    rt = os.path.join(STUB, "lean_runtime_for_tests.c")
    lib = tmp_path / "libstubs.so"
    subprocess.check_call(["gcc", "-c", "-fPIC", f"-I{STUB}", rt, "-o", str(tmp_path / "rt.o")])
    subprocess.check_call(["g++", "-std=c++17", "-shared", "-fPIC", f"-I{STUB}", str(gen), str(tmp_path / "rt.o"), "-o", str(lib)])
    L = ctypes.CDLL(str(lib))
    L.tyr_test_error_message.restype = ctypes.c_char_p
    L.tyr_test_error_message.argtypes = [ctypes.c_void_p]
    L.tyr_test_is_io_error.argtypes = [ctypes.c_void_p]
    for sym in ("lean_tyr_gpu_gemm_bf16", "lean_launch_tkFlashAttnFwd2BlockLse"):
        fn = getattr(L, sym)
        fn.restype = ctypes.c_void_p
        res = fn(ctypes.c_uint64(1), ctypes.c_uint64(2), None)          # any arguments: the stub is variadic
        assert L.tyr_test_is_io_error(res)
        msg = L.tyr_test_error_message(res).decode()
        assert msg == stubs.MESSAGE + sym and "unavailable in this build" in msg
    # a strong definition in the same link replaces the weak one
    strong = tmp_path / "strong.cpp"
    strong.write_text('#include <lean/lean.h>\nextern "C" lean_object* lean_tyr_gpu_copy(...) { return lean_io_result_mk_ok(lean_box(0)); }\n')
    lib2 = tmp_path / "libstubs2.so"
    subprocess.check_call(["g++", "-std=c++17", "-shared", "-fPIC", f"-I{STUB}", str(gen), str(strong), str(tmp_path / "rt.o"),
                           "-o", str(lib2)])
    L2 = ctypes.CDLL(str(lib2))
    L2.lean_tyr_gpu_copy.restype = ctypes.c_void_p
    L2.tyr_test_is_io_error.argtypes = [ctypes.c_void_p]
    assert not L2.tyr_test_is_io_error(L2.lean_tyr_gpu_copy(None))
    L2.lean_tyr_gpu_rope_fwd.restype = ctypes.c_void_p
    assert L2.tyr_test_is_io_error(L2.lean_tyr_gpu_rope_fwd(None))
