"""Writes the known-answer fixtures of this folder with LibTorch on the CPU.

The reference commits no golden vectors for this path (its runners draw their inputs at run time and
compare against LibTorch on the spot, e.g. Examples/GPU/RunFlashAttn.lean:19-95), so the answers
frozen here are those of the library routines the reference calls: scaled_dot_product_attention
(cc/src/tyr.cpp:2563-2589), logsumexp, repeat_interleave (cc/src/tyr.cpp:3930-3936), mm
(cc/src/tyr.cpp:1602-1607) and the float8_e4m3fn cast, all evaluated in float64 on bf16-rounded
inputs.  Run:  python tests/golden/make_fixtures.py   (rewrites tests/golden/*.npz)
"""
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_bits(t):
    return t.to(torch.bfloat16).contiguous().view(torch.uint16).numpy().copy()


def attention(seed, B, Hq, Hkv, N, D, causal):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    rep = Hq // Hkv
    kd = k.double().repeat_interleave(rep, dim=1)
    vd = v.double().repeat_interleave(rep, dim=1)
    o = torch.nn.functional.scaled_dot_product_attention(q.double(), kd, vd, is_causal=causal, scale=scale)
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), kd) * scale
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(N, N, dtype=torch.bool), 1), float("-inf"))
    lse = torch.logsumexp(s, -1)
    return dict(q=bf16_bits(q), k=bf16_bits(k), v=bf16_bits(v), o=o.float().numpy(), lse=lse.float().numpy(),
                causal=np.array(causal), scale=np.array(scale))


def main():
    cases = {"attn_mha_n40_d64_causal": attention(11, 1, 2, 2, 40, 64, True),
             "attn_mha_n70_d128_full": attention(12, 2, 2, 2, 70, 128, False),
             "attn_gqa_n130_d128_causal": attention(13, 1, 4, 2, 130, 128, True)}
    for name, c in cases.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **c)
    # decode: one query token against a cache, grouped heads
    g = torch.Generator().manual_seed(21)
    q = torch.randn(2, 8, 1, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(2, 2, 300, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(2, 2, 300, 128, generator=g).to(torch.bfloat16)
    sc = 1.0 / math.sqrt(128)
    kd, vd = k.double().repeat_interleave(4, dim=1), v.double().repeat_interleave(4, dim=1)
    o = torch.nn.functional.scaled_dot_product_attention(q.double(), kd, vd, is_causal=False, scale=sc)
    lse = torch.logsumexp(torch.einsum("bhqd,bhkd->bhqk", q.double(), kd) * sc, -1)[..., 0]
    np.savez_compressed(os.path.join(HERE, "decode_gqa_l300_d128.npz"), q=bf16_bits(q), k=bf16_bits(k), v=bf16_bits(v),
             o=o.float().numpy(), lse=lse.float().numpy(), scale=np.array(sc))
    # GEMM: bf16 operands, float64 product
    g = torch.Generator().manual_seed(31)
    a = (torch.randn(48, 64, generator=g) * 0.5).to(torch.bfloat16)
    b = (torch.randn(64, 40, generator=g) * 0.5).to(torch.bfloat16)
    np.savez_compressed(os.path.join(HERE, "gemm_bf16_48x40x64.npz"), a=bf16_bits(a), b=bf16_bits(b),
             c=torch.mm(a.double(), b.double()).float().numpy())
    # the 256 codes of float8_e4m3fn as LibTorch decodes them
    codes = torch.arange(256, dtype=torch.uint8)
    np.savez_compressed(os.path.join(HERE, "e4m3fn_codes.npz"), value=codes.view(torch.float8_e4m3fn).to(torch.float32).numpy())
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
