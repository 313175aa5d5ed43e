"""Pins the attention-backward function of the CPU checker (oracle_attn_bwd_f64) against
independent statements of the same math: LibTorch autograd (what the reference's runner uses
for its expected dQ/dK/dV), central finite differences of the forward checker, and closed
forms.  No GPU needed."""
import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint16).numpy().copy()


def rand4(seed, B, H, N, D):
    return lt.make_inputs(seed, *[(B, H, N, D)] * 4)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 128, 64), (2, 3, 75, 32), (1, 2, 130, 128)])
def test_bwd_matches_libtorch_autograd(shape, causal):
    # (1,1,128,64) non-causal is the shape of the reference's own backward fixture.
    B, H, N, D = shape
    q, k, v, g = rand4(11 + N, B, H, N, D)
    dq, dk, dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(g), causal, D ** -0.5)
    wq, wk, wv = lt.sdpa_4d_backward(q, k, v, g, causal)
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        np.testing.assert_allclose(got, want.numpy(), rtol=2e-4, atol=2e-4)


def test_bwd_is_the_directional_derivative_of_the_forward_checker():
    # <dO, O(x + h e) - O(x - h e)> / 2h  ==  <grad, e> for random directions e, with the
    # forward evaluated in double on unrounded inputs.  A wrong sign, a dropped delta term or
    # a missing scale factor changes these numbers at first order.
    torch.manual_seed(5)
    B, H, N, D = 1, 1, 24, 16
    q, k, v, g = rand4(3, B, H, N, D)
    scale = 0.3
    dq, dk, dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(g), True, scale)

    def fwd(q64, k64, v64):
        s = (q64 @ k64.transpose(-1, -2)) * scale
        mask = torch.ones(N, N, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
        return torch.softmax(s, -1) @ v64

    q64, k64, v64, g64 = (t.double() for t in (q, k, v, g))
    h = 1e-5
    for which, grad in (("q", dq), ("k", dk), ("v", dv)):
        e = torch.randn(B, H, N, D, dtype=torch.float64)
        args_p = {"q": q64, "k": k64, "v": v64}
        args_m = dict(args_p)
        args_p = dict(args_p)
        args_p[which] = args_p[which] + h * e
        args_m[which] = args_m[which] - h * e
        num = float(((fwd(**{n + "64": t for n, t in args_p.items()}) -
                      fwd(**{n + "64": t for n, t in args_m.items()})) * g64).sum()) / (2 * h)
        ana = float((torch.from_numpy(grad).double() * e).sum())
        assert abs(num - ana) <= 1e-5 * max(1.0, abs(ana)), (which, num, ana)


def test_bwd_closed_form_uniform_attention():
    # K = 0: P is uniform (1/n over the visible keys), so
    #   dV[j] = sum_{i >= j} dO[i] / (i+1)        (causal)
    #   dS = P o (dP - delta),  dQ = scale * dS K = 0,
    #   dK[j] = scale * sum_i dS[i,j] Q[i] with dS[i,j] = (dO[i].V[j] - dO[i].O[i]) / (i+1).
    B, H, N, D = 1, 1, 19, 8
    q, _, v, g = rand4(9, B, H, N, D)
    k = torch.zeros_like(q)
    scale = 0.5
    dq, dk, dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(g), True, scale)
    q64, v64, g64 = q.double()[0, 0], v.double()[0, 0], g.double()[0, 0]
    n = torch.arange(1, N + 1, dtype=torch.float64)
    tri = torch.ones(N, N, dtype=torch.float64).tril()
    P = tri / n[:, None]
    O = P @ v64
    want_dv = P.t() @ g64
    dS = P * (g64 @ v64.t() - (g64 * O).sum(-1, keepdim=True))
    want_dk = scale * dS.t() @ q64
    np.testing.assert_allclose(dq[0, 0], np.zeros((N, D)), atol=1e-7)
    np.testing.assert_allclose(dv[0, 0], want_dv.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(dk[0, 0], want_dk.numpy(), rtol=1e-6, atol=1e-6)


def test_bwd_invariants():
    # rows of dS sum to zero => dQ is orthogonal to nothing in particular, but a constant shift of
    # all keys (K + c) leaves P unchanged and therefore dV unchanged; and sum_j dK[j] equals
    # scale * sum_i (sum_j dS[i,j]) Q[i] = 0.
    B, H, N, D = 1, 2, 40, 16
    q, k, v, g = rand4(21, B, H, N, D)
    dq, dk, dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(g), False, 0.25)
    np.testing.assert_allclose(dk.sum(axis=2), np.zeros((B, H, D)), atol=2e-5)
    # causal: the gradient w.r.t. the last key/value only sees the last query
    dq, dk, dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(g), True, 0.25)
    o, _ = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), True, 0.25)
    # P[N-1, N-1] from the forward: O[N-1] = sum_j P_j V_j; recover via dV = P^T dO on the last row
    s = (q.double()[:, :, -1:, :] @ k.double().transpose(-1, -2)) * 0.25
    p_last = torch.softmax(s, -1)[:, :, 0, -1]
    want = p_last[..., None] * g.double()[:, :, -1, :]
    np.testing.assert_allclose(dv[:, :, -1, :], want.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("mode", ["gqa", "window", "lens", "all"])
def test_bwd_ex_matches_autograd_of_the_libtorch_mask_sequences(mode):
    # gradients of lean_torch_sdpa_gqa / _window / _mask taken by autograd (repeat_interleave's
    # gradient sums dK / dV over the query heads of a kv head)
    B, Hq, Hkv, N, D = 2, 4, 2, 50, 16
    q, g = lt.make_inputs(61, (B, Hq, N, D), (B, Hq, N, D))
    k, v = lt.make_inputs(62, (B, Hkv, N, D), (B, Hkv, N, D))
    window = 9 if mode in ("window", "all") else 0
    lens = [50, 13] if mode in ("lens", "all") else None
    causal = mode != "lens"
    dq, dk, dv = oracle.attn_bwd_f64_ex(bits(q), bits(k), bits(v), bits(g), causal, 0.25, window=window, kv_lens=lens)
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    n = N
    row, col = torch.arange(n).unsqueeze(1), torch.arange(n).unsqueeze(0)
    hidden = torch.zeros(B, 1, n, n, dtype=torch.bool)
    if causal:
        hidden = hidden | (col > row)
    if window:
        hidden = hidden | ((row - col) >= window)
    if lens is not None:
        hidden = hidden | (col[None, None] >= torch.tensor(lens).view(B, 1, 1, 1))
    mask = torch.zeros(B, 1, n, n, dtype=torch.float64).masked_fill(hidden, float("-inf"))
    kr, vr = k64.repeat_interleave(Hq // Hkv, 1), v64.repeat_interleave(Hq // Hkv, 1)
    # rows that see no key would be NaN in torch; give them one dummy visible key and zero their upstream gradient
    dead = hidden.all(-1, keepdim=True)
    mask = torch.where(dead.expand_as(mask), torch.zeros_like(mask), mask)
    out = torch.nn.functional.scaled_dot_product_attention(q64, kr, vr, mask, 0.0, False, scale=0.25)
    gg = g.double() * (~dead).double()
    out.backward(gg)
    dq_ref = q64.grad
    np.testing.assert_allclose(dq, dq_ref.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dk, k64.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dv, v64.grad.numpy(), rtol=1e-4, atol=1e-5)


def test_bwd_ex_reduces_to_plain_backward():
    B, H, N, D = 1, 3, 33, 16
    q, k, v, g = rand4(71, B, H, N, D)
    a = oracle.attn_bwd_f64_ex(bits(q), bits(k), bits(v), bits(g), True, 0.3)
    b = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(g), True, 0.3)
    for x, y in zip(a, b):
        np.testing.assert_allclose(x, y, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("causal", [False, True])
def test_bwd_ex_arbitrary_key_mask_matches_autograd_of_the_libtorch_padding_mask(causal):
    from oracle import libtorch_path as lt
    B, Hq, Hkv, N, D = 2, 4, 2, 40, 16
    q, g = lt.make_inputs(71, (B, Hq, N, D), (B, Hq, N, D))
    k, v = lt.make_inputs(72, (B, Hkv, N, D), (B, Hkv, N, D))
    gen = torch.Generator().manual_seed(73)
    km = torch.rand(B, N, generator=gen) < 0.6
    km[:, 0] = True
    dq, dk, dv = oracle.attn_bwd_f64_ex(bits(q), bits(k), bits(v), bits(g), causal, 0.25, key_mask=km.numpy())
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    # lean_torch_sdpa_gqa_mask scales by 1/sqrt(D) = 0.25 at D = 16
    out = lt.sdpa_gqa_mask(q64, k64, v64, km.long(), causal)
    out.backward(g.double())
    np.testing.assert_allclose(dq, q64.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dk, k64.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dv, v64.grad.numpy(), rtol=1e-4, atol=1e-5)
    # hidden keys get no gradient
    hidden = ~km.unsqueeze(1).expand(B, Hkv, N)
    assert np.all(dk[hidden.numpy()] == 0) and np.all(dv[hidden.numpy()] == 0)
