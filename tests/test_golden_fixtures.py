"""Known answers frozen under tests/golden (LibTorch float64 results on bf16-rounded inputs, stored as
float32; tests/golden/make_fixtures.py writes them).  The CPU checker has to reproduce them, and on a GPU
the library has to match them through the C ABI at the tolerances of the parity tests."""
import os

import numpy as np
import pytest
import torch

import oracle
from tests.util import from_bits

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ATTN = ["attn_mha_n40_d64_causal", "attn_mha_n70_d128_full", "attn_gqa_n130_d128_causal"]


def load(name):
    return np.load(os.path.join(G, name + ".npz"), allow_pickle=False)


@pytest.mark.parametrize("name", ATTN)
def test_checker_reproduces_frozen_attention(name):
    f = load(name)
    rep = f["q"].shape[1] // f["k"].shape[1]
    k, v = np.repeat(f["k"], rep, axis=1), np.repeat(f["v"], rep, axis=1)
    o, lse = oracle.attn_fwd_f64(f["q"], k, v, bool(f["causal"]), float(f["scale"]))
    assert np.abs(o - f["o"]).max() <= 2e-6
    assert np.abs(lse - f["lse"]).max() <= 2e-6


def test_checker_reproduces_frozen_decode():
    f = load("decode_gqa_l300_d128")
    for splits in (1, 3):
        o, lse = oracle.gqa_decode(f["q"], f["k"], f["v"], float(f["scale"]), num_splits=splits)
        o = oracle.bf16_bits_to_f32(o)                   # the checker rounds O to bf16 like the kernel
        assert np.abs(o - f["o"]).max() <= 2 ** -8 * np.abs(f["o"]).max()
        assert np.abs(lse - f["lse"]).max() <= 1e-5


def test_checker_reproduces_frozen_gemm_and_e4m3_codes():
    f = load("gemm_bf16_48x40x64")
    c = oracle.bf16_bits_to_f32(oracle.gemm_bf16(f["a"], f["b"]))
    assert np.abs(c - f["c"]).max() <= 2 ** -8 * np.abs(f["c"]).max()      # one bf16 rounding of the result
    want = load("e4m3fn_codes")["value"]
    got = oracle.e4m3_table()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


@pytest.mark.gpu
@pytest.mark.parametrize("name", ATTN)
def test_gpu_attention_matches_frozen_answers(name):
    import tyr_amd
    f = load(name)
    q, k, v = (from_bits(f[n]).cuda() for n in ("q", "k", "v"))
    o, lse = tyr_amd.flash_attn_fwd(q, k, v, causal=bool(f["causal"]), scale=float(f["scale"]))
    assert np.abs(o.float().cpu().numpy() - f["o"]).max() <= 2e-2
    assert np.abs(lse.cpu().numpy() - f["lse"]).max() <= 2e-2


@pytest.mark.gpu
def test_gpu_decode_and_gemm_match_frozen_answers():
    import tyr_amd
    f = load("decode_gqa_l300_d128")
    q, k, v = (from_bits(f[n]).cuda() for n in ("q", "k", "v"))
    for splits in (0, 1, 5):
        o, lse = tyr_amd.gqa_decode(q, k, v, scale=float(f["scale"]), num_splits=splits)
        assert np.abs(o.float().cpu().numpy() - f["o"]).max() <= 2e-2
        assert np.abs(lse.cpu().numpy() - f["lse"]).max() <= 2e-2
    f = load("gemm_bf16_48x40x64")
    c = tyr_amd.gemm_bf16(from_bits(f["a"]).cuda(), from_bits(f["b"]).cuda()).float().cpu().numpy()
    assert np.linalg.norm(c - f["c"]) / np.linalg.norm(f["c"]) <= 1e-2
