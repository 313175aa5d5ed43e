"""Parity of the memory-bound row kernels (copy, rotary embedding, fused residual + LayerNorm, the
decode step's rotate-and-append) with the CPU checker, through the C ABI.

Bars: copy and rotary are bit-exact (rotary evaluates the reference's expression in f32 without
fused multiply-add); LayerNorm within one bf16 ulp of the float64 checker and inside the reference
runner's allclose(5e-3, 5e-3) (Examples/GPU/RunLayerNorm.lean:77-78); the decode step bit-exact for the
cache rows and the rotated q."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt
from tests.util import bits, from_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import tyr_amd
    return tyr_amd


@pytest.mark.parametrize("n,dtype", [(64 * 64, torch.float32), (1, torch.float32), (1000003, torch.uint8),
                                     (7, torch.bfloat16), (1 << 24, torch.float32)])
def test_copy_is_exact(gpu, n, dtype):
    # 64x64 f32 is the reference's copy fixture.
    g = torch.Generator().manual_seed(n)
    src = torch.randint(0, 255, (n * torch.empty((), dtype=dtype).element_size(),), dtype=torch.uint8,
                        generator=g).view(dtype)
    out = gpu.copy(src.cuda())
    assert torch.equal(out.cpu().view(torch.uint8), src.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,S,H,D", [(1, 64, 1, 64), (2, 5, 3, 32), (1, 9, 2, 128), (3, 130, 4, 128), (1, 1, 1, 16)])
def test_rope_matches_oracle_bit_exact(gpu, B, S, H, D, dtype):
    torch.manual_seed(B * 1000 + S + D)
    x = torch.randn(B, S, H, D).to(dtype)
    cos, sin = lt.compute_rotary_freqs(S, D)
    y = gpu.rope_fwd(x.cuda(), cos.cuda(), sin.cuda()).cpu()
    if dtype == torch.bfloat16:
        assert np.array_equal(bits(y), oracle.rope(bits(x), cos.numpy(), sin.numpy()))
    else:
        assert np.array_equal(y.numpy(), oracle.rope(x.numpy(), cos.numpy(), sin.numpy()))


def test_rope_large_is_a_rotation(gpu):
    # [16, 4096, 16, 128] bf16: norms of the (x1, x2) pairs are preserved, position 0 is untouched,
    # and a slab matches the checker.
    B, S, H, D = 16, 4096, 16, 128
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(B, S, H, D, device="cuda", generator=gen).to(torch.bfloat16)
    cos, sin = lt.compute_rotary_freqs(S, D)
    y = gpu.rope_fwd(x, cos.cuda(), sin.cuda())
    assert torch.equal(y[:, 0], x[:, 0])
    n_in = x[3].float()[..., :64] ** 2 + x[3].float()[..., 64:] ** 2
    n_out = y[3].float()[..., :64] ** 2 + y[3].float()[..., 64:] ** 2
    assert float(((n_out - n_in).abs() / (n_in + 1e-3)).max()) <= 2e-2
    sl = slice(1000, 1016)
    want = oracle.rope(bits(x[5:6, sl]), cos[sl].numpy(), sin[sl].numpy())
    assert np.array_equal(bits(y[5:6, sl]), want)


@pytest.mark.parametrize("rows,d", [(64, 1024), (1, 8), (37, 264), (5, 4096), (3, 8192), (1000, 1024)])
def test_layernorm_residual_matches_oracle(gpu, rows, d):
    # (64, 1024) is the reference's layernorm fixture (x, residual, weight, bias ~ U[0,1)).
    torch.manual_seed(rows + d)
    x, res = torch.rand(rows, d).bfloat16(), torch.rand(rows, d).bfloat16()
    w, b = torch.rand(d).bfloat16(), torch.rand(d).bfloat16()
    out, resid = gpu.layernorm_residual(x.cuda(), res.cuda(), w.cuda(), b.cuda(), 1e-5)
    want_out, want_resid = oracle.layernorm_residual(bits(x), bits(res), bits(w), bits(b), 1e-5)
    assert np.array_equal(bits(resid), want_resid)
    got, want = out.cpu().float(), from_bits(want_out).float()
    assert float((got - want).abs().max()) <= 2 ** -7 * float(want.abs().max()) + 1e-6
    assert torch.allclose(got, want, rtol=5e-3, atol=5e-3)


def test_layernorm_residual_full_rows(gpu):
    # 65536 rows of 1024: row statistics of the output with weight 1 / bias 0, and a slab vs the checker
    rows, d = 65536, 1024
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.rand(rows, d, device="cuda", generator=gen).bfloat16()
    res = torch.rand(rows, d, device="cuda", generator=gen).bfloat16()
    one, zero = torch.ones(d, device="cuda").bfloat16(), torch.zeros(d, device="cuda").bfloat16()
    out, resid = gpu.layernorm_residual(x, res, one, zero, 1e-5)
    o = out.float()
    assert float(o.mean(-1).abs().max()) <= 1e-2
    assert float((o.var(-1, unbiased=False) - 1).abs().max()) <= 3e-2
    assert torch.equal(resid, x + res)
    sl = slice(40000, 40032)
    want_out, _ = oracle.layernorm_residual(bits(x[sl]), bits(res[sl]), bits(one), bits(zero), 1e-5)
    assert float((o[sl].cpu() - from_bits(want_out).float()).abs().max()) <= 2 ** -6


@pytest.mark.parametrize("B,Hq,Hkv,D,Lmax,pos", [(2, 8, 2, 128, 64, 0), (32, 32, 8, 128, 300, 299),
                                                 (1, 4, 4, 64, 17, 5), (3, 6, 2, 32, 9, 8)])
def test_decode_rope_append_matches_libtorch_sequence(gpu, B, Hq, Hkv, D, Lmax, pos):
    torch.manual_seed(pos + D)
    q = torch.randn(B, 1, Hq, D).bfloat16()
    k_new, v_new = torch.randn(B, 1, Hkv, D).bfloat16(), torch.randn(B, 1, Hkv, D).bfloat16()
    k_cache, v_cache = torch.randn(B, Hkv, Lmax, D).bfloat16(), torch.randn(B, Hkv, Lmax, D).bfloat16()
    cos_t, sin_t = lt.compute_rotary_freqs(Lmax, D)
    cos, sin = cos_t[pos:pos + 1].contiguous(), sin_t[pos:pos + 1].contiguous()
    want_q, want_k, want_v = lt.decode_step_cache_update(q, k_new, v_new, cos, sin, k_cache, v_cache, pos)
    kc, vc = k_cache.cuda(), v_cache.cuda()
    q_rot = gpu.decode_rope_append(q.cuda(), k_new.cuda().transpose(1, 2).contiguous(),
                                   v_new.cuda().transpose(1, 2).contiguous(), cos.cuda(), sin.cuda(), kc, vc, pos)
    # rotated q against the checker (bit-exact) and against the LibTorch sequence (bf16 products: one ulp)
    want_q_bits = oracle.rope(bits(q), cos.numpy(), sin.numpy())
    assert np.array_equal(bits(q_rot), want_q_bits)
    assert float((q_rot.cpu().float().view(B, Hq, D) - want_q.float().reshape(B, Hq, D)).abs().max()) <= 2 ** -6 * 8
    # the cache: only row pos changed, and it holds rope(k_new) / v_new
    assert torch.equal(vc.cpu(), want_v)
    want_k_bits = oracle.rope(bits(k_new), cos.numpy(), sin.numpy()).reshape(B, Hkv, D)
    assert np.array_equal(bits(kc[:, :, pos]), want_k_bits)
    mask = torch.ones(Lmax, dtype=torch.bool)
    mask[pos] = False
    assert torch.equal(kc.cpu()[:, :, mask], k_cache[:, :, mask])


def test_decode_step_end_to_end(gpu):
    # rotate + append, then attention over the cache prefix: equals the checker's decode on the
    # updated cache (the reference's forwardStep order, Tyr/Model/Qwen/Attention.lean:172-200).
    B, Hq, Hkv, D, Lmax, pos = 4, 16, 4, 128, 512, 300
    torch.manual_seed(9)
    q = torch.randn(B, Hq, 1, D).bfloat16()
    k_new, v_new = torch.randn(B, Hkv, 1, D).bfloat16(), torch.randn(B, Hkv, 1, D).bfloat16()
    k_cache, v_cache = torch.randn(B, Hkv, Lmax, D).bfloat16(), torch.randn(B, Hkv, Lmax, D).bfloat16()
    cos_t, sin_t = lt.compute_rotary_freqs(Lmax, D)
    cos, sin = cos_t[pos:pos + 1].contiguous().cuda(), sin_t[pos:pos + 1].contiguous().cuda()
    kc, vc = k_cache.cuda(), v_cache.cuda()
    q_rot = gpu.decode_rope_append(q.cuda(), k_new.cuda(), v_new.cuda(), cos, sin, kc, vc, pos)
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q_rot, kc, vc, scale=sc, kv_len=pos + 1)
    wo, wl = oracle.gqa_decode(bits(q_rot), bits(kc), bits(vc), sc, 1, kv_len=pos + 1)
    assert float((o.cpu().float() - from_bits(wo).float()).abs().max()) <= 2e-2
    assert float(np.abs(lse.cpu().numpy() - wl).max()) <= 2e-2


def test_rowwise_error_convention(gpu):
    x = torch.zeros(1, 4, 2, 24, dtype=torch.bfloat16, device="cuda")
    cs = torch.zeros(4, 12, device="cuda")
    with pytest.raises(gpu.TyrGpuError, match="not supported"):
        gpu.rope_fwd(x, cs, cs)                      # D % 16 != 0 for bf16
    with pytest.raises(gpu.TyrGpuError, match="must be a CUDA tensor"):
        gpu.copy(torch.zeros(4))
    a = torch.zeros(2, 12, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(12, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(gpu.TyrGpuError, match="not supported"):
        gpu.layernorm_residual(a, a, w, w)           # d_model % 8 != 0
