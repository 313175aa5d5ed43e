"""The LDS-DMA helpers of tyr_amd/csrc/common.hpp write M0 inside opaque asm.  That is only safe
while nothing the compiler generates reads M0 with a value it set earlier.  This test compiles the
kernel files that use the helpers to gfx950 assembly (no GPU needed) and checks that
  * every instruction that names m0 is an `s_mov_b32 m0, <sgpr>` (the helpers' own write),
  * each such write is followed, before any other m0 write, by a `buffer_load_dwordx4 ... lds`,
  * no instruction with an implicit M0 operand (movrel, GWS, sendmsg, interpolation, LDS-direct) appears.
"""
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tyr_amd", "csrc")
FILES = ["flash_attn_fwd.hip", "flash_attn_bwd.hip", "gemm_bf16.hip", "gemm_fp8.hip"]
HIPCC = "/opt/rocm/bin/hipcc"
IMPLICIT_M0 = re.compile(r"^\s*(s_movrel|v_movrel|ds_gws|s_sendmsg|v_interp|s_ttrace|ds_.*_gs_reg|v_readlane_b32\s+\S+,\s*\S+,\s*m0)")


def _asm(name, out_dir):
    out = os.path.join(out_dir, name + ".s")
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                           "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S", os.path.join(CSRC, name),
                           "-o", out], stderr=subprocess.DEVNULL)
    with open(out) as f:
        return [ln.split(";")[0].rstrip() for ln in f]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_only_the_lds_dma_helpers_touch_m0():
    with tempfile.TemporaryDirectory() as d, ThreadPoolExecutor(4) as pool:
        listings = dict(zip(FILES, pool.map(lambda n: _asm(n, d), FILES)))
    for name, lines in listings.items():
        code = [ln for ln in lines if ln.startswith("\t") and not ln.startswith("\t.")]
        assert not [ln for ln in code if IMPLICIT_M0.match(ln)], name
        writes = 0
        pending = False            # an M0 write not yet followed by its LDS-DMA load
        for ln in code:
            if re.search(r"\bm0\b", ln):
                assert re.match(r"^\s*s_mov_b32 m0, (s\d+|vcc_lo|vcc_hi|ttmp\d+)$", ln), (name, ln)
                assert not pending, (name, "M0 written twice without an LDS-DMA load in between")
                pending, writes = True, writes + 1
            elif re.match(r"^\s*buffer_load_dwordx4 .* lds$", ln):
                pending = False
        assert writes > 0 and not pending, name
