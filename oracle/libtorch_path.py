"""The reference's LibTorch path, restated call for call -- TEST INFRASTRUCTURE.

The reference computes its parity targets by handing tensors to LibTorch (a
third-party dependency pinned at 2.9.1 in the reference's Readme.md:37; the
``torch`` package importable here is 2.10).  Its FFI adds nothing but
refcounting around these calls, so the restatement is the calls themselves:

* ``sdpa_4d``       cc/src/tyr.cpp:2563-2589  torch::scaled_dot_product_attention(q,k,v,nullopt,p,is_causal)
* ``sdpa_gqa_qkv``  cc/src/tyr.cpp:4100-4133  repeat_interleave(n_head/n_kv_head, dim=1) on K and V, then the same call
* ``mm``            cc/src/tyr.cpp:1602-1607  torch::mm
* ``fp8_mm``        no LibTorch fp8 GEMM exists in the reference; the parity target for the DSL kernel
                    (Tyr/GPU/Kernels/PrecisionGemm.lean:97-115) is dequantise -> f32 torch::mm -> scale
* ``reference_attention`` Examples/GPU/RunFlashAttn.lean:26-48: bf16-rounded inputs, f32 math, O and LSE
* ``make_inputs``   cc/src/tyr.cpp:424-432,545-551,4246-4250: manual_seed, randn, .to(bfloat16)

Everything here runs on CPU tensors.  It is used as a checker and as the timed
CPU baseline; the product never imports it.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def make_inputs(seed: int, *shapes, dtype=torch.bfloat16, std: float = 1.0):
    """manual_seed(seed) then one randn per shape, in order, each cast to ``dtype``."""
    torch.manual_seed(seed)
    out = []
    for s in shapes:
        t = torch.randn(*s, dtype=torch.float32)
        if std != 1.0:
            t = t * std
        out.append(t.to(dtype))
    return out


def sdpa_4d(q, k, v, is_causal: bool, dropout_p: float = 0.0):
    return F.scaled_dot_product_attention(q, k, v, None, dropout_p, is_causal)


def sdpa_4d_backward(q, k, v, d_o, is_causal: bool):
    """Gradients of sdpa_4d with respect to q, k, v for the upstream gradient d_o, taken from
    autograd the way the reference's runner takes them (set_requires_grad, backward(out, dO),
    grad_of).  Inputs are converted to f32 first so the result is the f32 gradient of the
    rounded inputs."""
    q32, k32, v32 = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    out = F.scaled_dot_product_attention(q32, k32, v32, None, 0.0, is_causal)
    out.backward(d_o.float())
    return q32.grad, k32.grad, v32.grad


def loss_and_grad_out(out, target):
    """`lossAndGradOut` (Examples/GPU/RunMhaH100Train.lean:60-67), call for call: (loss, dO bf16)."""
    out32, tgt32 = out.float(), target.float()
    diff = out32 - tgt32
    loss = (diff * diff).mean() * 0.5
    return loss, (diff / float(diff.numel())).to(torch.bfloat16)


def sgd_update(param, grad, lr: float):
    """`sgdUpdate` (Examples/GPU/RunMhaH100Train.lean:69-70) on an f32 master and a bf16 gradient."""
    return param - (grad.float() * lr)


def train_step(q_m, k_m, v_m, target32, lr: float, is_causal: bool = False):
    """`oneTorchTrainStep` (Examples/GPU/RunMhaH100Train.lean:95-113): f32 SDPA of the detached masters, loss =
    0.5 mean((out - target)^2), autograd, SGD.  Returns the updated masters and the loss."""
    ql, kl, vl = (t.detach().requires_grad_(True) for t in (q_m, k_m, v_m))
    out = F.scaled_dot_product_attention(ql, kl, vl, None, 0.0, is_causal)
    diff = out - target32
    loss = (diff * diff).mean() * 0.5
    loss.backward()
    return q_m - ql.grad * lr, k_m - kl.grad * lr, v_m - vl.grad * lr, loss.detach()


def sdpa_gqa_qkv(q, k, v, is_causal: bool = False, enable_gqa: bool = True, dropout_p: float = 0.0):
    n_head, n_kv_head = q.shape[1], k.shape[1]
    if enable_gqa and n_head != n_kv_head and n_kv_head > 0:
        rep = n_head // n_kv_head
        k = k.repeat_interleave(rep, 1)
        v = v.repeat_interleave(rep, 1)
    return F.scaled_dot_product_attention(q, k, v, None, dropout_p, is_causal)


def compute_rotary_freqs(seq_len: int, head_dim: int, base: float = 10000.0):
    """(cos, sin) f32 [seq_len, head_dim/2] -- the call sequence of compute_rotary_freqs_impl."""
    channel_range = torch.arange(0, head_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / torch.pow(base, channel_range / float(head_dim))
    t = torch.arange(seq_len, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos(), freqs.sin()


def apply_rotary_emb(x, cos, sin):
    """x [B,S,H,D]; cos, sin [S,D/2] -- the call sequence of lean_torch_apply_rotary_emb."""
    d = x.size(3) // 2
    x1, x2 = x[..., :d], x[..., d:2 * d]
    cos_b, sin_b = cos.unsqueeze(0).unsqueeze(2), sin.unsqueeze(0).unsqueeze(2)
    y1 = x1 * cos_b - x2 * sin_b
    y2 = x1 * sin_b + x2 * cos_b
    return torch.cat([y1, y2], 3).to(x.dtype)


def layer_norm_residual(x, residual, weight, bias, eps: float = 1e-5):
    """(out, out_resid) as the reference's layernorm runner computes its expected values."""
    resid = x + residual
    return F.layer_norm(resid, (resid.shape[-1],), weight, bias, eps), resid


def decode_step_cache_update(q, k_new, v_new, cos, sin, k_cache, v_cache, pos: int):
    """forwardStep's RoPE + cache write: q [B,1,Hq,D], k_new / v_new [B,1,Hkv,D], cos / sin [1,D/2],
    caches [B,Hkv,maxLen,D] -> (q_rot [B,Hq,1,D], k_cache', v_cache')."""
    q_rot = apply_rotary_emb(q, cos, sin).transpose(1, 2)
    k_rot = apply_rotary_emb(k_new, cos, sin).transpose(1, 2)
    k2 = torch.slice_scatter(k_cache, k_rot, 2, pos, pos + 1)
    v2 = torch.slice_scatter(v_cache, v_new.transpose(1, 2), 2, pos, pos + 1)
    return q_rot, k2, v2


def sdpa_gqa(q, k, v, is_causal: bool, enable_gqa: bool = True, dropout_p: float = 0.0):
    """The call sequence of lean_torch_sdpa_gqa (equal q and kv lengths)."""
    return sdpa_gqa_qkv(q, k, v, is_causal, enable_gqa, dropout_p)


def _repeat_kv(q, k, v):
    n_head, n_kv_head = q.shape[1], k.shape[1]
    if n_head != n_kv_head and n_kv_head > 0:
        rep = n_head // n_kv_head
        k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    return k, v


def sdpa_gqa_window(q, k, v, window_size: int):
    """The call sequence of lean_torch_sdpa_gqa_window: explicit -inf / 0 mask from
    (col > row) | (row - col >= window)."""
    k, v = _repeat_kv(q, k, v)
    n = q.size(2)
    row = torch.arange(n).unsqueeze(1)
    col = torch.arange(n).unsqueeze(0)
    combined = (col > row) | ((row - col) >= int(window_size))
    mask = torch.where(combined, torch.full((n, n), float("-inf"), dtype=q.dtype), torch.zeros((n, n), dtype=q.dtype))
    return F.scaled_dot_product_attention(q, k, v, mask.unsqueeze(0).unsqueeze(0), 0.0, False)


def sdpa_gqa_mask(q, k, v, padding_mask, is_causal: bool):
    """The call sequence of lean_torch_sdpa_gqa_mask: padding_mask [B, N], 1 = valid key."""
    k, v = _repeat_kv(q, k, v)
    n = q.size(2)
    key_mask = padding_mask.unsqueeze(1).unsqueeze(2)
    if is_causal:
        row = torch.arange(n).unsqueeze(1)
        col = torch.arange(n).unsqueeze(0)
        combined = (col > row).unsqueeze(0).unsqueeze(0) | (key_mask == 0)
    else:
        combined = (key_mask == 0)
    mask = torch.where(combined, torch.tensor(float("-inf"), dtype=q.dtype), torch.tensor(0.0, dtype=q.dtype))
    return F.scaled_dot_product_attention(q, k, v, mask, 0.0, False)


def mm(a, b):
    return torch.mm(a, b)


def fp8_mm(aq, bq, scale_a: float, scale_b: float):
    """aq [M,K], bq [K,N] float8_e4m3fn -> f32 (scale_a*scale_b) * (deq(aq) @ deq(bq))."""
    return torch.mm(aq.to(torch.float32), bq.to(torch.float32)) * (float(scale_a) * float(scale_b))


def quantize_e4m3(x: torch.Tensor):
    """Per-tensor absmax quantisation: s = absmax/448, xq = e4m3fn(x/s).  -> (xq, s)"""
    s = float(x.abs().max()) / 448.0
    if s == 0.0:
        s = 1.0
    xq = (x.to(torch.float32) / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return xq, s


def reference_attention(q, k, v, is_causal: bool, scale: float | None = None):
    """f32 attention from the (already rounded) inputs, with LSE = ln sum exp(scaled scores)."""
    q32, k32, v32 = q.float(), k.float(), v.float()
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    s = torch.matmul(q32, k32.transpose(-1, -2)) * scale
    if is_causal:
        n, m = s.shape[-2], s.shape[-1]
        mask = torch.ones(n, m, dtype=torch.bool).tril(diagonal=m - n)
        s = s.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    o = torch.matmul(torch.softmax(s, dim=-1), v32)
    return o, lse
