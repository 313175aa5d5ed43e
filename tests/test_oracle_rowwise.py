"""Pins the rotary and fused-LayerNorm functions of the CPU checker against independent statements
of the same math: the LibTorch call sequences of the reference, closed forms and invariants.  No GPU."""
import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt
from tests.util import bits, from_bits


def test_rotary_freqs_closed_form():
    cos, sin = lt.compute_rotary_freqs(7, 8, 10000.0)
    t = np.arange(7, dtype=np.float64)[:, None]
    inv = 1.0 / 10000.0 ** (np.arange(0, 8, 2, dtype=np.float64) / 8.0)
    np.testing.assert_allclose(cos.numpy(), np.cos(t * inv), atol=1e-5)
    np.testing.assert_allclose(sin.numpy(), np.sin(t * inv), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_matches_libtorch_sequence(dtype):
    # (1,64,1,64) f32 is the reference's own rotary fixture shape.
    for (B, S, H, D) in ((1, 64, 1, 64), (2, 5, 3, 32), (1, 9, 2, 128)):
        torch.manual_seed(B + S + D)
        x = torch.rand(B, S, H, D).to(dtype)
        cos, sin = lt.compute_rotary_freqs(S, D)
        want = lt.apply_rotary_emb(x, cos, sin)
        xin = bits(x) if dtype == torch.bfloat16 else x.numpy()
        got = oracle.rope(xin, cos.numpy(), sin.numpy())
        if dtype == torch.bfloat16:
            assert np.array_equal(got, bits(want))
        else:
            np.testing.assert_allclose(got, want.numpy(), rtol=0, atol=1e-6)


def test_rope_closed_forms():
    B, S, H, D = 1, 4, 2, 16
    x = torch.randn(B, S, H, D)
    one, zero = np.ones((S, D // 2), np.float32), np.zeros((S, D // 2), np.float32)
    # angle 0: identity ; angle pi/2: [x1 | x2] -> [-x2 | x1]
    np.testing.assert_array_equal(oracle.rope(x.numpy(), one, zero), x.numpy())
    quarter = oracle.rope(x.numpy(), zero, one)
    np.testing.assert_array_equal(quarter[..., :D // 2], -x.numpy()[..., D // 2:])
    np.testing.assert_array_equal(quarter[..., D // 2:], x.numpy()[..., :D // 2])
    # a rotation preserves x1^2 + x2^2 pairwise, and position 0 of the real table is the identity
    cos, sin = lt.compute_rotary_freqs(S, D)
    y = oracle.rope(x.numpy(), cos.numpy(), sin.numpy())
    n_in = x.numpy()[..., :D // 2] ** 2 + x.numpy()[..., D // 2:] ** 2
    n_out = y[..., :D // 2] ** 2 + y[..., D // 2:] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(y[:, 0], x.numpy()[:, 0])


def test_layernorm_residual_matches_libtorch_and_closed_forms():
    # [1,64,1024] is the reference's own layernorm fixture shape.
    torch.manual_seed(0)
    rows, d = 64, 1024
    x, res = torch.rand(rows, d).bfloat16(), torch.rand(rows, d).bfloat16()
    w, b = torch.rand(d).bfloat16(), torch.rand(d).bfloat16()
    out, resid = oracle.layernorm_residual(bits(x), bits(res), bits(w), bits(b), 1e-5)
    want_out, want_resid = lt.layer_norm_residual(x, res, w, b, 1e-5)
    assert np.array_equal(resid, bits(want_resid))
    # torch rounds once from f32; the checker from f64: at most one bf16 ulp apart
    diff = (from_bits(out).float() - want_out.float()).abs()
    assert float(diff.max()) <= 2 ** -7 * float(want_out.float().abs().max())
    # weight 1, bias 0: rows have mean 0 and variance 1 ; constant rows give the bias
    one, zero = torch.ones(d).bfloat16(), torch.zeros(d).bfloat16()
    out1, _ = oracle.layernorm_residual(bits(x), bits(res), bits(one), bits(zero), 0.0)
    o = from_bits(out1).double()
    assert float(o.mean(-1).abs().max()) <= 5e-3 and float((o.var(-1, unbiased=False) - 1).abs().max()) <= 2e-2
    const = torch.full((3, d), 0.75).bfloat16()
    outc, _ = oracle.layernorm_residual(bits(const), bits(const), bits(w), bits(b), 1e-5)
    assert np.array_equal(outc, np.broadcast_to(bits(b), (3, d)))
