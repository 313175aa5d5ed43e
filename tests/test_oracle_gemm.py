"""Pins the GEMM and FP8 functions of the CPU checker.  No GPU needed."""
import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt


def bits(t):
    return t.contiguous().view(torch.uint16).numpy().copy()


def from_bits(a):
    return torch.from_numpy(a.copy()).view(torch.bfloat16)


def test_bf16_round_to_nearest_even_matches_torch_cast():
    x = torch.randn(4096) * torch.logspace(-20, 20, 4096)
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, float("inf"), -float("inf"), 3.3895e38])])
    assert np.array_equal(oracle.f32_to_bf16_bits(x.numpy()), bits(x.to(torch.bfloat16)))
    L = oracle.lib()
    for v in (1.00390625, 1.01171875, -2.5, 3.3895e38, 1e-40):
        assert L.oracle_f32_to_bf16(v) == int(bits(torch.tensor([v]).to(torch.bfloat16))[0])


def test_gemm_identity_and_permutation_are_exact():
    a, = lt.make_inputs(0, (48, 48))
    eye = torch.eye(48).to(torch.bfloat16)
    perm = torch.randperm(48, generator=torch.Generator().manual_seed(0))
    P = torch.eye(48)[perm].to(torch.bfloat16)          # (P A)[i] = A[perm[i]]
    assert np.array_equal(oracle.gemm_bf16(bits(a), bits(eye)), bits(a))
    assert np.array_equal(oracle.gemm_bf16(bits(eye), bits(a)), bits(a))
    assert np.array_equal(oracle.gemm_bf16(bits(P), bits(a)), bits(a[perm]))
    assert np.array_equal(oracle.gemm_bf16(bits(a), bits(P)), bits(a[:, torch.argsort(perm)]))  # catches a transposed B


@pytest.mark.parametrize("M,N,K", [(33, 17, 65), (128, 96, 256), (1, 1, 1)])
def test_gemm_bf16_vs_double_and_libtorch(M, N, K):
    a, b = lt.make_inputs(1, (M, K), (K, N), std=K ** -0.25)
    c = from_bits(oracle.gemm_bf16(bits(a), bits(b))).double()
    want = a.double() @ b.double()
    rel = float((c - want).norm() / want.norm())
    assert rel <= 4e-3, rel
    # same rounding as LibTorch's f32 mm of the bf16-rounded inputs up to one bf16 ulp of accumulation noise
    lt32 = lt.mm(a.float(), b.float())
    assert float((c.float() - lt32).abs().max()) <= float(lt32.abs().max()) * 2 ** -7
    # NT form on B^T gives bit-identical results (same k order)
    cnt = oracle.gemm_bf16(bits(a), bits(b.t().contiguous()), trans_b=True)
    assert np.array_equal(cnt, oracle.gemm_bf16(bits(a), bits(b)))


def test_gemm_is_exactly_linear_in_powers_of_two():
    a, b = lt.make_inputs(2, (40, 72), (72, 24))
    c1 = from_bits(oracle.gemm_bf16(bits(a), bits(b))).float()
    c2 = from_bits(oracle.gemm_bf16(bits((a.float() * 2).to(torch.bfloat16)), bits(b))).float()
    assert torch.equal(c2, c1 * 2)


# ---------------------------------------------------------------- E4M3

def test_e4m3_table_is_ocp_e4m3fn():
    tab = oracle.e4m3_table()
    want = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(want))
    assert np.array_equal(tab[~np.isnan(tab)], want[~np.isnan(want)])
    # closed-form anchors: max 448, no infinity, NaN only at 0x7f/0xff, smallest subnormal 2^-9
    assert tab[0x7E] == 448.0 and tab[0xFE] == -448.0 and np.isnan(tab[0x7F]) and np.isnan(tab[0xFF])
    assert not np.isinf(tab).any() and tab[0x01] == 2.0 ** -9 and tab[0x08] == 2.0 ** -6 and tab[0x38] == 1.0


def test_e4m3_encode_round_trip_and_libtorch_cast():
    tab = oracle.e4m3_table()
    codes = np.array([c for c in range(256) if not np.isnan(tab[c]) and c != 0x80], dtype=np.uint8)
    assert np.array_equal(oracle.e4m3_encode(tab[codes]), codes)
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(size=3000) * 100, rng.normal(size=3000), rng.normal(size=2000) * 1e-2,
                        (tab[codes][:-1] + tab[codes][1:]) / 2]).astype(np.float32)   # includes exact ties
    x = x[np.abs(x) <= 448]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = oracle.e4m3_encode(x)
    same = (got == want) | ((got & 0x7F) == 0) & ((want & 0x7F) == 0)   # +-0 are the same value
    assert same.all(), (x[~same][:5], got[~same][:5], want[~same][:5])
    assert oracle.e4m3_encode(np.array([1e9, -1e9, 460.0], np.float32)).tolist() == [0x7E, 0xFE, 0x7E]  # saturates


def test_quantize_recipe_scale_is_absmax_over_448():
    x = torch.randn(64, 64)
    xq, s = lt.quantize_e4m3(x)
    assert abs(s - float(x.abs().max()) / 448) < 1e-12
    assert float(xq.float().abs().max()) == 448.0
    assert float((xq.float() * s - x).abs().max()) <= float(x.abs().max()) * 2 ** -4


@pytest.mark.parametrize("M,N,K", [(32, 48, 64), (17, 9, 130)])
def test_gemm_fp8_vs_dequantised_f32(M, N, K):
    torch.manual_seed(3)
    a, b = torch.randn(M, K), torch.randn(K, N)
    aq, sa = lt.quantize_e4m3(a)
    bq, sb = lt.quantize_e4m3(b)
    c, cf = oracle.gemm_fp8(aq.view(torch.uint8).numpy(), bq.view(torch.uint8).numpy(), sa, sb)
    want = (aq.double() @ bq.double()) * (np.float32(sa) * np.float32(sb))
    np.testing.assert_allclose(cf, want.numpy(), rtol=2e-5, atol=1e-6)       # products exact, only sum order
    np.testing.assert_allclose(cf, lt.fp8_mm(aq, bq, sa, sb).numpy(), rtol=2e-5, atol=1e-5)
    assert np.array_equal(c, oracle.f32_to_bf16_bits(cf))
    cnt, _ = oracle.gemm_fp8(aq.view(torch.uint8).numpy(), bq.t().contiguous().view(torch.uint8).numpy(), sa, sb, True)
    assert np.array_equal(cnt, c)


def test_gemm_fp8_identity_returns_decoded_operand_times_scales():
    tab = oracle.e4m3_table()
    codes = np.array([c for c in range(256) if not np.isnan(tab[c])], dtype=np.uint8)[:64 * 3].reshape(3, 64)
    eye = np.zeros((64, 64), np.uint8)
    np.fill_diagonal(eye, 0x38)  # 1.0
    _, cf = oracle.gemm_fp8(codes, eye, 0.5, 4.0)
    assert np.array_equal(cf, tab[codes] * 2.0)
