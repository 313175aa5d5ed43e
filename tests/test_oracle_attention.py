"""Pins the attention functions of the CPU checker (oracle/tyr_oracle.c) against
independent statements of the same math: closed forms, LibTorch library routines
and invariants.  No GPU needed."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint16).numpy().copy() if t.dtype == torch.bfloat16 else None


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.copy()).view(torch.bfloat16)


def rand_qkv(seed, B, H, N, D):
    return lt.make_inputs(seed, (B, H, N, D), (B, H, N, D), (B, H, N, D))


# ---------------------------------------------------------------- closed forms

@pytest.mark.parametrize("causal", [False, True])
def test_f64_uniform_scores_give_prefix_means(causal):
    # K = 0  =>  every score is 0  =>  P is uniform over the visible keys:
    # O[i] = mean(V[:i+1]) (causal) or mean(V) ; LSE[i] = ln(#visible keys).
    B, H, N, D = 1, 2, 37, 16
    q, _, v = rand_qkv(0, B, H, N, D)
    k = torch.zeros_like(q)
    o, lse = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), causal, 0.25)
    v64 = v.double()
    if causal:
        want = torch.cumsum(v64, dim=2) / torch.arange(1, N + 1, dtype=torch.float64).view(1, 1, N, 1)
        want_lse = torch.log(torch.arange(1, N + 1, dtype=torch.float64)).expand(B, H, N)
    else:
        want = v64.mean(dim=2, keepdim=True).expand(B, H, N, D)
        want_lse = torch.full((B, H, N), math.log(N), dtype=torch.float64)
    np.testing.assert_allclose(o, want.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(lse, want_lse.numpy(), rtol=1e-6, atol=1e-6)


def test_f64_one_hot_attention_selects_value_row():
    # q_i = 64 * e_{pi(i)}, k_j = e_j  =>  score(i, pi(i)) = 64 dominates by e^-64:
    # O[i] = V[pi(i)] to float precision, LSE[i] = 64*scale + ln(1 + (N-1)e^{-64 scale}).
    N = D = 32
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(1))
    k = torch.eye(N).view(1, 1, N, D).to(torch.bfloat16)
    q = (64.0 * torch.eye(N)[perm]).view(1, 1, N, D).to(torch.bfloat16)
    v = lt.make_inputs(2, (1, 1, N, D))[0]
    o, lse = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), False, 1.0)
    np.testing.assert_allclose(o[0, 0], v.float()[0, 0][perm].numpy(), atol=1e-5)
    np.testing.assert_allclose(lse[0, 0], np.full(N, 64.0), atol=1e-5)


def test_causal_row0_is_v0_and_a_dropped_mask_is_caught():
    q, k, v = rand_qkv(3, 2, 2, 50, 32)
    o, lse = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), True, 1 / math.sqrt(32))
    np.testing.assert_allclose(o[:, :, 0], v.float()[:, :, 0].numpy(), atol=1e-6)
    s00 = (q.float()[:, :, 0] * k.float()[:, :, 0]).sum(-1) / math.sqrt(32)
    np.testing.assert_allclose(lse[:, :, 0], s00.numpy(), rtol=1e-5, atol=1e-5)
    ob, _ = oracle.attn_fwd_tiled(bits(q), bits(k), bits(v), True, 1 / math.sqrt(32), 16)
    assert np.array_equal(ob[:, :, 0], bits(v)[:, :, 0])  # exact: P = 1.0, O = bf16(V[0])


# ---------------------------------------------------------------- library routines

@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 4, 256, 64), (2, 3, 77, 128), (1, 1, 1, 64)])
def test_f64_matches_libtorch_sdpa_and_logsumexp(causal, shape):
    # (1,4,256,64) causal with scale 1/8 is the reference's CPU-runnable configuration.
    q, k, v = rand_qkv(4, *shape)
    D = shape[-1]
    o, lse = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), causal, 1 / math.sqrt(D))
    want = lt.sdpa_4d(q.double(), k.double(), v.double(), causal)
    np.testing.assert_allclose(o, want.float().numpy(), rtol=2e-6, atol=2e-6)
    s = torch.matmul(q.double(), k.double().transpose(-1, -2)) / math.sqrt(D)
    if causal:
        s = s.masked_fill(~torch.ones(shape[2], shape[2], dtype=torch.bool).tril(), float("-inf"))
    np.testing.assert_allclose(lse, torch.logsumexp(s, -1).float().numpy(), rtol=2e-6, atol=2e-6)
    # the f32 recipe of the reference's runner agrees too
    o32, lse32 = lt.reference_attention(q, k, v, causal)
    np.testing.assert_allclose(o, o32.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(lse, lse32.numpy(), rtol=1e-5, atol=1e-5)


def test_libtorch_f32_path_on_reference_cpu_config():
    # fp32 inputs, B=1 H=4 N=256 D=64, causal, scale 1/8: LibTorch f32 vs double brute force <= 1e-5.
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 4, 256, 64) for _ in range(3))
    got = lt.sdpa_4d(q, k, v, True)
    want = lt.sdpa_4d(q.double(), k.double(), v.double(), True)
    assert float((got.double() - want).abs().max()) <= 1e-5


# ---------------------------------------------------------------- tiled kernel order

@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape,tile", [((1, 4, 256, 64), 64), ((1, 2, 200, 128), 64),
                                        ((2, 1, 65, 64), 32), ((1, 1, 130, 128), 128)])
def test_tiled_within_tolerance_of_f64(causal, shape, tile):
    q, k, v = rand_qkv(5, *shape)
    sc = 1 / math.sqrt(shape[-1])
    ob, lse = oracle.attn_fwd_tiled(bits(q), bits(k), bits(v), causal, sc, tile)
    o64, lse64 = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), causal, sc)
    assert np.abs(from_bits(ob).float().numpy() - o64).max() <= 2e-2
    assert np.abs(lse - lse64).max() <= 1e-4
    # softmax rows sum to one: sum_j exp(s_ij - lse_i) == 1
    s = torch.matmul(q.double(), k.double().transpose(-1, -2)) * sc
    if causal:
        s = s.masked_fill(~torch.ones(shape[2], shape[2], dtype=torch.bool).tril(), float("-inf"))
    ones = torch.exp(s - torch.from_numpy(lse).double().unsqueeze(-1)).sum(-1)
    np.testing.assert_allclose(ones.numpy(), 1.0, atol=1e-4)


def test_tiled_is_tile_size_independent_within_rounding():
    q, k, v = rand_qkv(6, 1, 2, 192, 64)
    outs = [oracle.attn_fwd_tiled(bits(q), bits(k), bits(v), True, 0.125, t) for t in (16, 64, 192)]
    for ob, lse in outs[1:]:
        assert np.abs(from_bits(ob).float().numpy() - from_bits(outs[0][0]).float().numpy()).max() <= 8e-3
        np.testing.assert_allclose(lse, outs[0][1], atol=2e-5)


def test_causal_future_keys_do_not_change_earlier_rows_bitwise():
    q, k, v = rand_qkv(7, 1, 1, 96, 64)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 60:] = 9.0
    v2[:, :, 60:] = -7.0
    a, la = oracle.attn_fwd_tiled(bits(q), bits(k), bits(v), True, 0.125, 32)
    b, lb = oracle.attn_fwd_tiled(bits(q), bits(k2), bits(v2), True, 0.125, 32)
    assert np.array_equal(a[:, :, :60], b[:, :, :60]) and np.array_equal(la[:, :, :60], lb[:, :, :60])
    assert not np.array_equal(a[:, :, 60:], b[:, :, 60:])


# ---------------------------------------------------------------- GQA decode

@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(2, 8, 2, 300, 64), (1, 32, 8, 513, 128), (3, 4, 4, 40, 128)])
def test_decode_matches_libtorch_gqa_path(B, Hq, Hkv, L, D):
    q, = lt.make_inputs(8, (B, Hq, 1, D))
    k, v = lt.make_inputs(9, (B, Hkv, L, D), (B, Hkv, L, D))
    sc = 1 / math.sqrt(D)
    ob, lse = oracle.gqa_decode(bits(q), bits(k), bits(v), sc, 1)
    want = lt.sdpa_gqa_qkv(q.float(), k.float(), v.float(), False, True)
    assert float((from_bits(ob).float() - want).abs().max()) <= 1e-2
    kr = k.float().repeat_interleave(Hq // Hkv, 1)
    s = torch.matmul(q.float(), kr.transpose(-1, -2)) * sc
    np.testing.assert_allclose(lse, torch.logsumexp(s, -1)[:, :, 0].numpy(), atol=1e-4)


def test_decode_head_mapping_is_repeat_interleave_not_tile():
    # make kv-head g's V constant = g: the output of q-head h must be h // (Hq/Hkv).
    B, Hq, Hkv, L, D = 1, 8, 4, 20, 64
    q, = lt.make_inputs(10, (B, Hq, 1, D))
    k, = lt.make_inputs(11, (B, Hkv, L, D))
    v = torch.arange(Hkv, dtype=torch.float32).view(1, Hkv, 1, 1).expand(B, Hkv, L, D).to(torch.bfloat16).contiguous()
    ob, _ = oracle.gqa_decode(bits(q), bits(k), bits(v), 0.125, 2)
    got = from_bits(ob).float()[0, :, 0, 0].numpy()
    np.testing.assert_allclose(got, np.arange(Hq) // 2, atol=1e-2)


def test_decode_split_count_invariance_and_partial_cache():
    B, Hq, Hkv, Lmax, D = 2, 8, 2, 257, 128
    q, = lt.make_inputs(12, (B, Hq, 1, D))
    k, v = lt.make_inputs(13, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
    base_o, base_l = oracle.gqa_decode(bits(q), bits(k), bits(v), 0.088, 1)
    for s in (2, 3, 8, 300):
        o, l = oracle.gqa_decode(bits(q), bits(k), bits(v), 0.088, s)
        assert np.abs(from_bits(o).float().numpy() - from_bits(base_o).float().numpy()).max() <= 4e-3
        np.testing.assert_allclose(l, base_l, atol=2e-5)
    # kv_len < allocated rows: equals decoding over the sliced, re-packed cache
    o1, l1 = oracle.gqa_decode(bits(q), bits(k), bits(v), 0.088, 4, kv_len=100)
    o2, l2 = oracle.gqa_decode(bits(q), bits(k[:, :, :100].contiguous()), bits(v[:, :, :100].contiguous()), 0.088, 4)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)


def test_decode_equals_last_row_of_causal_prefill():
    # the property the reference's cached-vs-uncached greedy decoding test relies on
    B, H, N, D = 1, 4, 90, 64
    q, k, v = rand_qkv(14, B, H, N, D)
    pre, lse_pre = oracle.attn_fwd_tiled(bits(q), bits(k), bits(v), True, 0.125, 30)
    dec, lse_dec = oracle.gqa_decode(bits(q[:, :, -1:].contiguous()), bits(k), bits(v), 0.125, 3)
    assert np.abs(from_bits(dec).float().numpy()[:, :, 0] - from_bits(pre).float().numpy()[:, :, -1]).max() <= 4e-3
    np.testing.assert_allclose(lse_dec, lse_pre[:, :, -1], atol=2e-5)


# ------------------------------------------------- grouped queries, window, key lengths

@pytest.mark.parametrize("causal", [False, True])
def test_f64_ex_grouped_queries_equal_repeat_interleave(causal):
    B, Hq, Hkv, N, D = 2, 6, 2, 45, 16
    q, = lt.make_inputs(31, (B, Hq, N, D))
    k, v = lt.make_inputs(32, (B, Hkv, N, D), (B, Hkv, N, D))
    o, lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25)
    kr, vr = k.repeat_interleave(3, 1), v.repeat_interleave(3, 1)
    o2, lse2 = oracle.attn_fwd_f64(bits(q), bits(kr), bits(vr), causal, 0.25)
    np.testing.assert_array_equal(o, o2)
    np.testing.assert_array_equal(lse, lse2)
    ref = lt.sdpa_gqa(q.double(), k.double(), v.double(), causal)
    np.testing.assert_allclose(o, ref.numpy(), atol=1e-5)


@pytest.mark.parametrize("window", [1, 5, 72, 1000])
def test_f64_ex_window_matches_libtorch_sequence(window):
    B, Hq, Hkv, N, D = 1, 4, 2, 90, 16
    q, = lt.make_inputs(33, (B, Hq, N, D))
    k, v = lt.make_inputs(34, (B, Hkv, N, D), (B, Hkv, N, D))
    o, lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), True, 0.25, window=window)
    ref = lt.sdpa_gqa_window(q.double(), k.double(), v.double(), window)
    np.testing.assert_allclose(o, ref.numpy(), atol=1e-5)
    if window == 1:                                   # each query sees only itself: O = V, LSE = score
        np.testing.assert_allclose(o, v.repeat_interleave(2, 1).float().numpy(), atol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
def test_f64_ex_key_lengths_match_libtorch_padding_mask(causal):
    B, Hq, Hkv, N, D = 3, 2, 1, 40, 16
    lens = [40, 7, 1]
    q, = lt.make_inputs(35, (B, Hq, N, D))
    k, v = lt.make_inputs(36, (B, Hkv, N, D), (B, Hkv, N, D))
    o, lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25, kv_lens=lens)
    pm = (torch.arange(N)[None, :] < torch.tensor(lens)[:, None]).long()
    ref = lt.sdpa_gqa_mask(q.double(), k.double(), v.double(), pm, causal)
    np.testing.assert_allclose(o, ref.numpy(), atol=1e-5)
    # changing keys / values beyond a sequence's length changes nothing
    k2, v2 = k.clone(), v.clone()
    k2[1, :, 7:] = 9.0
    v2[1, :, 7:] = -9.0
    o2, _ = oracle.attn_fwd_f64_ex(bits(q), bits(k2), bits(v2), causal, 0.25, kv_lens=lens)
    np.testing.assert_array_equal(o, o2)


def _scattered_mask(B, N, seed, keep_first):
    g = torch.Generator().manual_seed(seed)
    m = (torch.rand(B, N, generator=g) < 0.6)
    if keep_first:
        m[:, 0] = True                              # causal row 0 then sees a key (LibTorch gives NaN otherwise)
    m[0] = True                                     # one sequence without padding
    return m


@pytest.mark.parametrize("causal", [False, True])
def test_f64_ex_arbitrary_key_mask_matches_libtorch_padding_mask(causal):
    # lean_torch_sdpa_gqa_mask with a mask that is not a prefix: holes anywhere in the sequence
    B, Hq, Hkv, N, D = 3, 4, 2, 70, 16
    q, = lt.make_inputs(41, (B, Hq, N, D))
    k, v = lt.make_inputs(42, (B, Hkv, N, D), (B, Hkv, N, D))
    km = _scattered_mask(B, N, 43, keep_first=True)
    o, lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25, key_mask=km.numpy())
    ref = lt.sdpa_gqa_mask(q.double(), k.double(), v.double(), km.long(), causal)
    np.testing.assert_allclose(o, ref.numpy(), atol=1e-5)
    # a hidden key's contents do not matter; an all-visible mask is no mask; a prefix mask is a key length
    k2, v2 = k.clone(), v.clone()
    k2[~km.unsqueeze(1).expand(B, Hkv, N)] = 7.0
    v2[~km.unsqueeze(1).expand(B, Hkv, N)] = -7.0
    o2, lse2 = oracle.attn_fwd_f64_ex(bits(q), bits(k2), bits(v2), causal, 0.25, key_mask=km.numpy())
    np.testing.assert_array_equal(o, o2)
    np.testing.assert_array_equal(lse, lse2)
    o3, _ = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25, key_mask=np.ones((B, N), np.uint8))
    o4, _ = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25)
    np.testing.assert_array_equal(o3, o4)
    lens = [70, 9, 31]
    pm = (torch.arange(N)[None, :] < torch.tensor(lens)[:, None])
    o5, l5 = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25, key_mask=pm.numpy())
    o6, l6 = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, 0.25, kv_lens=lens)
    np.testing.assert_array_equal(o5, o6)
    np.testing.assert_array_equal(l5, l6)


def test_f64_ex_row_with_every_key_hidden_is_zero():
    B, H, N, D = 1, 1, 12, 16
    q, k, v = lt.make_inputs(44, (B, H, N, D), (B, H, N, D), (B, H, N, D))
    km = np.ones((B, N), np.uint8)
    km[0, :3] = 0                                   # causal rows 0..2 see nothing
    o, lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), True, 0.25, key_mask=km)
    assert np.all(o[0, 0, :3] == 0) and np.all(np.isneginf(lse[0, 0, :3]))
    assert np.all(np.isfinite(lse[0, 0, 3:]))
    np.testing.assert_allclose(o[0, 0, 3], v[0, 0, 3].float().numpy(), atol=1e-6)      # row 3 sees only key 3
