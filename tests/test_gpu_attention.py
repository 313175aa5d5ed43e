"""Parity of the gfx950 flash-attention forward and GQA decode kernels (through the C ABI)
with the CPU checker.

Tolerance (stated by the task): max-abs error of O <= 2e-2 and of LSE <= 2e-2 against an fp32
(here fp64) reference computed from the bf16-rounded inputs.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt
from tests.util import bits, from_bits, max_abs

pytestmark = pytest.mark.gpu
TOL = 2e-2


@pytest.fixture(scope="module")
def gpu():
    import tyr_amd
    return tyr_amd


def qkv(seed, B, H, N, D):
    return lt.make_inputs(seed, (B, H, N, D), (B, H, N, D), (B, H, N, D))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,H,N,D", [(1, 1, 128, 64), (1, 4, 256, 64), (1, 1, 128, 128), (2, 3, 200, 128),
                                     (1, 2, 1, 128), (1, 1, 77, 64), (1, 2, 64, 128), (1, 8, 384, 128),
                                     (1, 1, 129, 128), (1, 1, 768, 64)])
def test_flash_attn_matches_oracle(gpu, B, H, N, D, causal):
    # (1,1,128,64) and (1,1,768,64) are the reference's own e2e shapes; (1,4,256,64) is its CPU configuration.
    q, k, v = qkv(300 + N + D, B, H, N, D)
    sc = 1 / math.sqrt(D)
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc)
    o64, lse64 = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), causal, sc)
    assert max_abs(o.cpu().float(), o64) <= TOL
    assert max_abs(lse.cpu(), lse64) <= TOL
    # and within bf16 rounding of the restated reference kernel (same op order, 64-row tiles)
    ot, lset = oracle.attn_fwd_tiled(bits(q), bits(k), bits(v), causal, sc, 64)
    assert max_abs(o.cpu().float(), from_bits(ot).float()) <= TOL
    assert max_abs(lse.cpu(), lset) <= 1e-3


@pytest.mark.parametrize("seed", range(6))
def test_flash_attn_random_shapes(gpu, seed):
    # randomised e2e in the spirit of the reference's E2E_TRIALS runs: ragged lengths, odd head counts
    rng = np.random.default_rng(1000 + seed)
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 6))
    N, D = int(rng.integers(1, 1100)), int(rng.choice([64, 128]))
    causal = bool(rng.integers(0, 2))
    q, k, v = qkv(500 + seed, B, H, N, D)
    sc = float(rng.uniform(0.05, 0.2))
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc)
    o64, lse64 = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), causal, sc)
    assert max_abs(o.cpu().float(), o64) <= TOL, (B, H, N, D, causal)
    assert max_abs(lse.cpu(), lse64) <= 1e-3, (B, H, N, D, causal)


def test_flash_attn_large_scores_trigger_rescales(gpu):
    # keys whose scores grow along the sequence force the running maximum to move repeatedly
    B, H, N, D = 1, 2, 700, 128
    q, k, v = qkv(31, B, H, N, D)
    ramp = torch.linspace(0.2, 6.0, N).view(1, 1, N, 1)
    k = (k.float() * ramp).to(torch.bfloat16)
    for causal in (False, True):
        o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal)
        o64, lse64 = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), causal, 1 / math.sqrt(D))
        assert max_abs(o.cpu().float(), o64) <= TOL
        assert max_abs(lse.cpu(), lse64) <= 2e-3


def test_flash_attn_causal_closed_forms(gpu):
    B, H, N, D = 1, 2, 300, 128
    q, k, v = qkv(11, B, H, N, D)
    # K = 0: uniform weights -> prefix means of V and LSE = ln(i+1)
    o, lse = gpu.flash_attn_fwd(q.cuda(), torch.zeros_like(k).cuda(), v.cuda(), causal=True)
    want = torch.cumsum(v.double(), 2) / torch.arange(1, N + 1, dtype=torch.float64).view(1, 1, N, 1)
    assert max_abs(o.cpu().float(), want) <= TOL
    assert max_abs(lse.cpu(), torch.log(torch.arange(1, N + 1, dtype=torch.float64)).expand(B, H, N)) <= 1e-4
    # row 0 sees only key 0: O[0] = V[0] exactly
    o, _ = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=True)
    assert np.array_equal(bits(o[:, :, 0]), bits(v[:, :, 0]))


def test_flash_attn_future_keys_do_not_leak(gpu):
    q, k, v = qkv(12, 1, 2, 512, 128)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 320:] = 5.0
    v2[:, :, 320:] = -3.0
    a, la = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=True)
    b, lb = gpu.flash_attn_fwd(q.cuda(), k2.cuda(), v2.cuda(), causal=True)
    assert torch.equal(a[:, :, :320], b[:, :, :320]) and torch.equal(la[:, :, :320], lb[:, :, :320])
    assert not torch.equal(a[:, :, 320:], b[:, :, 320:])


@pytest.mark.parametrize("persistent", [0, 1])
@pytest.mark.parametrize("causal", [True, False])
def test_flash_attn_forward_is_reproducible_over_many_launches(gpu, causal, persistent):
    # Regression test for a write-after-read race on the first K stage: the first tile step used to request K(2)
    # into the stage other waves were still reading K(0) from (no barrier after the prologue's scores); whether a
    # wave lost depended on timing, a few dozen waves per launch at this size.  Eight launches must agree bit for bit.
    B, H, N, D = 16, 16, 4096, 128
    torch.manual_seed(11)
    q, k, v = (torch.randn(B, H, N, D, device="cuda").to(torch.bfloat16) for _ in range(3))
    with _persistent(persistent):
        first = gpu.flash_attn_fwd(q, k, v, causal=causal)
        for _ in range(7):
            o, lse = gpu.flash_attn_fwd(q, k, v, causal=causal)
            assert torch.equal(o, first[0]) and torch.equal(lse, first[1])
    # values, not only agreement between launches: two heads against the double-precision checker
    sc = 1 / math.sqrt(D)
    for (b, h) in ((1, 2), (B - 1, H - 1)):
        o64, lse64 = oracle.attn_fwd_f64(bits(q[b:b + 1, h:h + 1]), bits(k[b:b + 1, h:h + 1]), bits(v[b:b + 1, h:h + 1]), causal, sc)
        assert max_abs(first[0][b, h].cpu().float(), o64[0, 0]) <= TOL
        assert max_abs(first[1][b, h].cpu(), lse64[0, 0]) <= TOL


def test_flash_attn_full_size_config(gpu):
    # B=16 H=16 N=4096 D=128 causal, bf16, scale 1/sqrt(128): O and per-row LSE.
    B, H, N, D = 16, 16, 4096, 128
    torch.manual_seed(3)
    q = torch.randn(B, H, N, D, device="cuda").to(torch.bfloat16)
    k = torch.randn(B, H, N, D, device="cuda").to(torch.bfloat16)
    v = torch.randn(B, H, N, D, device="cuda").to(torch.bfloat16)
    sc = 1 / math.sqrt(D)
    o, lse = gpu.flash_attn_fwd(q, k, v, causal=True, scale=sc)
    torch.cuda.synchronize()
    # three heads, every row, against the double-precision checker
    for (b, h) in ((0, 0), (7, 9), (15, 15)):
        o64, lse64 = oracle.attn_fwd_f64(bits(q[b:b + 1, h:h + 1]), bits(k[b:b + 1, h:h + 1]), bits(v[b:b + 1, h:h + 1]), True, sc)
        assert max_abs(o[b, h].cpu().float(), o64[0, 0]) <= TOL
        assert max_abs(lse[b, h].cpu(), lse64[0, 0]) <= TOL
    # every head: fp32 reference on the GPU (checker only), one batch entry at a time
    for b in range(B):
        ref, ref_lse = [], []
        s = torch.matmul(q[b].float(), k[b].float().transpose(-1, -2)) * sc
        s.masked_fill_(~torch.ones(N, N, dtype=torch.bool, device="cuda").tril(), float("-inf"))
        ref_lse = torch.logsumexp(s, -1)
        ref = torch.matmul(torch.softmax(s, -1), v[b].float())
        assert max_abs(o[b].float(), ref) <= TOL
        assert max_abs(lse[b], ref_lse) <= TOL
        del s, ref, ref_lse
    # size-independent properties: row 0 is V[0]; softmax weights reconstructed from LSE sum to one
    assert torch.equal(o[:, :, 0], v[:, :, 0])
    assert torch.equal(gpu.flash_attn_fwd(q, k, v, causal=True, scale=sc)[0], o)   # deterministic


# ------------------------------------------- launch shape: one workgroup per job id / persistent workgroups

class _persistent:
    """Forward launches inside the block use persistent workgroups (on = 1) or one workgroup per job id (on = 0)."""

    def __init__(self, on):
        self.on = on

    def __enter__(self):
        from tyr_amd import _lib
        self.prev = _lib.load().tyr_hip_flash_attn_fwd_persistent(int(self.on))

    def __exit__(self, *exc):
        from tyr_amd import _lib
        _lib.load().tyr_hip_flash_attn_fwd_persistent(self.prev)


def _mixed_lengths(B, N):
    """Key lengths that give a persistent workgroup every kind of hand-over: full, empty, one tile or less, odd and even
    tile counts, a ragged last tile."""
    pool = [N, 0, 1, 64, 63, 65, 128, 192, N - 1, N // 2 + 7, 200, N]
    return [pool[i % len(pool)] for i in range(B)]


_MANY_JOBS_CASES = ["noncausal", "causal", "causal_lens", "noncausal_lens", "key_mask", "causal_key_mask",
                    "gqa_causal", "gqa_noncausal", "gqa_lens_odd_groups"]


@pytest.mark.parametrize("case", _MANY_JOBS_CASES)
def test_flash_attn_persistent_launch_walks_many_jobs(gpu, case):
    # More job ids than the 512 persistent workgroups of a 256-CU device, so that workgroups hand over from one job to
    # the next (another head, another batch entry with another key length or mask, the XCD mapping of grouped queries).
    # The persistent launch must equal the one-workgroup-per-job launch bit for bit, and sampled heads must match the
    # double-precision checker.
    D = 128
    causal = "noncausal" not in case
    lens = km = None
    if case.startswith("gqa"):
        B, Hq, Hkv, N = (8, 16, 4, 1280) if case != "gqa_lens_odd_groups" else (9, 12, 3, 1100)
    elif "lens" in case or "mask" in case:
        B, Hq, Hkv, N = 24, 8, 8, 768 if causal else 520
    else:
        B, Hq, Hkv, N = 12, 10, 10, 1280 if causal else 1100
    ntq = (N + 127) // 128
    pair = causal and ntq > 1
    ids = B * Hq * ((ntq + 1) // 2 if pair else ntq)
    assert ids > 512, ids
    g = torch.Generator().manual_seed(1500 + _MANY_JOBS_CASES.index(case))
    q = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16)
    k, v = (torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16) for _ in range(2))
    if "lens" in case:
        lens = _mixed_lengths(B, N)
    if "mask" in case:
        km = torch.rand(B, N, generator=g) < 0.7
        km[1] = False                                   # a sequence without visible keys
        km[2, 128:384] = False                          # whole key tiles hidden
        km[3] = True
        km[:, 0] |= torch.arange(B) % 2 == 0
        km[1] = False
    sc = 1 / math.sqrt(D)
    kw = dict(causal=causal, scale=sc)
    if lens is not None:
        kw["kv_lens"] = torch.tensor(lens, dtype=torch.int32, device="cuda")
    if km is not None:
        kw["key_mask"] = km.cuda()
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    with _persistent(0):
        o0, l0 = gpu.flash_attn_fwd(qd, kd, vd, **kw)
    with _persistent(1):
        o1, l1 = gpu.flash_attn_fwd(qd, kd, vd, **kw)
        o2, l2 = gpu.flash_attn_fwd(qd, kd, vd, **kw)
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    # sampled (batch, query head) pairs, every row, against the checker
    G = Hq // Hkv
    sample = sorted({(0, 0), (1, Hq - 1), (2, G), (3, 1), (B // 2, Hq // 2), (B - 1, Hq - 1), (B - 2, 0)})
    for b, h in sample:
        hk = h // G
        wo, wl = oracle.attn_fwd_f64_ex(bits(q[b:b + 1, h:h + 1]), bits(k[b:b + 1, hk:hk + 1]), bits(v[b:b + 1, hk:hk + 1]),
                                        causal, sc, kv_lens=None if lens is None else lens[b:b + 1],
                                        key_mask=None if km is None else km[b:b + 1].numpy())
        assert max_abs(o1[b, h].cpu().float(), wo[0, 0]) <= TOL, (case, b, h)
        seen = torch.from_numpy(np.isfinite(wl[0, 0]))
        if bool(seen.any()):
            assert max_abs(l1[b, h].cpu()[seen], wl[0, 0][seen.numpy()]) <= TOL, (case, b, h)
        assert bool(torch.isneginf(l1[b, h].cpu()[~seen]).all()), (case, b, h)     # rows that see no key: LSE = -inf


# ------------------------------------------- grouped queries, window, key lengths (prefill)

@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Hq,Hkv,N,D", [(1, 4, 1, 200, 128), (2, 8, 2, 333, 64), (8, 2, 1, 129, 128), (1, 32, 8, 512, 128)])
def test_flash_attn_grouped_queries(gpu, B, Hq, Hkv, N, D, causal):
    # lean_torch_sdpa_gqa: query head h reads kv head h / (Hq/Hkv).  (8,2,1,...) exercises the XCD-dealt mapping.
    q, = lt.make_inputs(1200 + N, (B, Hq, N, D))
    k, v = lt.make_inputs(1201 + N, (B, Hkv, N, D), (B, Hkv, N, D))
    sc = 1 / math.sqrt(D)
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc)
    wo, wl = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, sc)
    assert max_abs(o.cpu().float(), wo) <= TOL
    assert max_abs(lse.cpu(), wl) <= TOL
    # identical to the plain kernel on materialised repeat_interleave'd K / V
    G = Hq // Hkv
    o2, lse2 = gpu.flash_attn_fwd(q.cuda(), k.cuda().repeat_interleave(G, 1).contiguous(),
                                  v.cuda().repeat_interleave(G, 1).contiguous(), causal=causal, scale=sc)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)


@pytest.mark.parametrize("window", [1, 31, 72, 250, 4096])
@pytest.mark.parametrize("N,D", [(600, 128), (257, 64)])
def test_flash_attn_sliding_window(gpu, window, N, D):
    # lean_torch_sdpa_gqa_window: key j visible to query i iff j <= i and i - j < window (72 and 250 are the
    # reference models' windows).
    B, Hq, Hkv = 2, 4, 2
    q, = lt.make_inputs(1300 + window, (B, Hq, N, D))
    k, v = lt.make_inputs(1301 + window, (B, Hkv, N, D), (B, Hkv, N, D))
    sc = 1 / math.sqrt(D)
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=True, scale=sc, window=window)
    wo, wl = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), True, sc, window=window)
    assert max_abs(o.cpu().float(), wo) <= TOL
    assert max_abs(lse.cpu(), wl) <= TOL
    if window >= N:                                   # a window wider than the sequence is plain causal attention
        o2, _ = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=True, scale=sc)
        assert max_abs(o.float(), o2.float()) <= 1e-6


@pytest.mark.parametrize("causal", [False, True])
def test_flash_attn_key_lengths(gpu, causal):
    # prefix padding mask (lean_torch_sdpa_gqa_mask): keys at or beyond a sequence's length are masked,
    # bit-for-bit independent of what the padded keys / values hold.
    B, Hq, Hkv, N, D = 4, 4, 2, 300, 128
    lens = [300, 0, 129, 64]
    q, = lt.make_inputs(1400, (B, Hq, N, D))
    k, v = lt.make_inputs(1401, (B, Hkv, N, D), (B, Hkv, N, D))
    sc = 1 / math.sqrt(D)
    lens_d = torch.tensor(lens, dtype=torch.int32, device="cuda")
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc, kv_lens=lens_d)
    wo, wl = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, sc, kv_lens=lens)
    assert max_abs(o.cpu().float(), wo) <= TOL
    seen = np.isfinite(wl)                              # the sequence of length 0 sees no key: O = 0, LSE = -inf
    assert not seen[1].any() and seen[0].all()
    assert max_abs(lse.cpu()[torch.from_numpy(seen)], wl[seen]) <= TOL
    assert bool(torch.isneginf(lse.cpu()[torch.from_numpy(~seen)]).all())
    assert torch.count_nonzero(o[1].float()) == 0
    k2, v2 = k.clone(), v.clone()
    for b, n in enumerate(lens):
        k2[b, :, n:] = 50.0
        v2[b, :, n:] = -50.0
    o2, lse2 = gpu.flash_attn_fwd(q.cuda(), k2.cuda(), v2.cuda(), causal=causal, scale=sc, kv_lens=lens_d)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)
    # window and lengths together
    o3, lse3 = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=True, scale=sc, kv_lens=lens_d, window=40)
    wo3, wl3 = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), True, sc, window=40, kv_lens=lens)
    assert max_abs(o3.cpu().float(), wo3) <= TOL
    finite = np.isfinite(wl3)
    assert max_abs(lse3.cpu()[torch.from_numpy(finite)], wl3[finite]) <= TOL
    assert bool(torch.isinf(lse3.cpu()[torch.from_numpy(~finite)]).all())


# ------------------------------------------------------------------------- decode

@pytest.mark.parametrize("B,Hq,Hkv,L,splits", [(1, 4, 1, 32, 1), (2, 8, 2, 300, 0), (1, 32, 8, 513, 3),
                                               (3, 4, 4, 40, 2), (1, 16, 1, 1000, 4), (2, 32, 8, 2048, 0),
                                               (1, 8, 2, 1, 1), (1, 8, 2, 33, 8)])
def test_gqa_decode_matches_oracle(gpu, B, Hq, Hkv, L, splits):
    D = 128
    q, = lt.make_inputs(400 + L, (B, Hq, 1, D))
    k, v = lt.make_inputs(401 + L, (B, Hkv, L, D), (B, Hkv, L, D))
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits)
    want_o, want_lse = oracle.gqa_decode(bits(q), bits(k), bits(v), sc, max(splits, 1))
    assert max_abs(o.cpu().float(), from_bits(want_o).float()) <= TOL
    assert max_abs(lse.cpu(), want_lse) <= 1e-3
    # the LibTorch call sequence of the reference (repeat_interleave + SDPA), fp32
    ref = lt.sdpa_gqa_qkv(q.float(), k.float(), v.float(), False, True)
    assert max_abs(o.cpu().float(), ref) <= TOL


@pytest.mark.parametrize("B,Hq,Hkv,L,splits", [(2, 8, 2, 300, 0), (1, 4, 4, 33, 1), (3, 16, 1, 1000, 4), (1, 6, 2, 1, 1)])
def test_gqa_decode_head_dim_64(gpu, B, Hq, Hkv, L, splits):
    D = 64
    q, = lt.make_inputs(450 + L, (B, Hq, 1, D))
    k, v = lt.make_inputs(451 + L, (B, Hkv, L, D), (B, Hkv, L, D))
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits)
    want_o, want_lse = oracle.gqa_decode(bits(q), bits(k), bits(v), sc, max(splits, 1))
    assert max_abs(o.cpu().float(), from_bits(want_o).float()) <= TOL
    assert max_abs(lse.cpu(), want_lse) <= 1e-3
    ref = lt.sdpa_gqa_qkv(q.float(), k.float(), v.float(), False, True)
    assert max_abs(o.cpu().float(), ref) <= TOL
    # decode == last row of the causal prefill kernel at the same head dimension
    if Hq == Hkv:
        qf = torch.zeros(B, Hq, L, D, dtype=torch.bfloat16)
        qf[:, :, -1:] = q
        of, _ = gpu.flash_attn_fwd(qf.cuda(), k.cuda(), v.cuda(), causal=True, scale=sc)
        assert max_abs(o.cpu().float(), of[:, :, -1:].cpu().float()) <= TOL


@pytest.mark.parametrize("seed", range(6))
def test_gqa_decode_random_shapes(gpu, seed):
    rng = np.random.default_rng(2000 + seed)
    Hkv = int(rng.integers(1, 5))
    G = int(rng.choice([1, 2, 4, 7, 16]))
    B, L = int(rng.integers(1, 4)), int(rng.integers(1, 3000))
    Lmax = L + int(rng.integers(0, 100))
    splits = int(rng.choice([0, 1, 2, 5, 16]))
    D = 128
    q, = lt.make_inputs(600 + seed, (B, Hkv * G, 1, D))
    k, v = lt.make_inputs(700 + seed, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits, kv_len=L)
    want_o, want_lse = oracle.gqa_decode(bits(q), bits(k), bits(v), sc, max(splits, 1), kv_len=L)
    assert max_abs(o.cpu().float(), from_bits(want_o).float()) <= TOL, (B, Hkv, G, L, splits)
    assert max_abs(lse.cpu(), want_lse) <= 1e-3, (B, Hkv, G, L, splits)


def test_gqa_decode_split_invariance_and_partial_cache(gpu):
    B, Hq, Hkv, Lmax, D = 2, 32, 8, 1024, 128
    q, = lt.make_inputs(20, (B, Hq, 1, D))
    k, v = lt.make_inputs(21, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    base_o, base_l = gpu.gqa_decode(qc, kc, vc, num_splits=1)
    for s in (2, 3, 5, 8, 32):
        o, l = gpu.gqa_decode(qc, kc, vc, num_splits=s)
        assert max_abs(o.float(), base_o.float()) <= 8e-3
        assert max_abs(l, base_l) <= 1e-4
    # only the first kv_len rows of the preallocated cache are read
    o1, l1 = gpu.gqa_decode(qc, kc, vc, num_splits=2, kv_len=700)
    o2, l2 = gpu.gqa_decode(qc, kc[:, :, :700].contiguous(), vc[:, :, :700].contiguous(), num_splits=2)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    kc2 = kc.clone()
    kc2[:, :, 700:] = 50.0
    o3, _ = gpu.gqa_decode(qc, kc2, vc, num_splits=2, kv_len=700)
    assert torch.equal(o1, o3)


def test_gqa_decode_equals_last_row_of_causal_prefill(gpu):
    B, H, N, D = 1, 8, 640, 128
    q, k, v = qkv(22, B, H, N, D)
    pre, lse_pre = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=True)
    dec, lse_dec = gpu.gqa_decode(q[:, :, -1:].contiguous().cuda(), k.cuda(), v.cuda(), num_splits=3)
    assert max_abs(dec[:, :, 0].float(), pre[:, :, -1].float()) <= 8e-3
    assert max_abs(lse_dec, lse_pre[:, :, -1]) <= 1e-3


@pytest.mark.parametrize("window", [0, 1, 37, 256, 5000])
@pytest.mark.parametrize("splits", [0, 1, 5])
def test_gqa_decode_varlen_and_window(gpu, window, splits):
    # Per-sequence cache lengths (the decode-time form of the reference's padding-mask SDPA,
    # cc/src/tyr.cpp:4019-4095) and a sliding window (cc/src/tyr.cpp:3953-4016): sequence b attends to
    # rows [max(0, len_b - window), len_b).  Checked by slicing exactly those rows out on the host and
    # running the checker (and the LibTorch sequence) on the slice.
    B, Hq, Hkv, Lmax, D = 5, 8, 2, 700, 128
    lens = [700, 1, 333, 64, 513]
    q, = lt.make_inputs(900 + window, (B, Hq, 1, D))
    k, v = lt.make_inputs(901 + window, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
    sc = 1 / math.sqrt(D)
    lens_d = torch.tensor(lens, dtype=torch.int32, device="cuda")
    o, lse = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits, kv_lens=lens_d, window=window)
    for b, n in enumerate(lens):
        lo = max(0, n - window) if window > 0 else 0
        kb, vb = k[b:b + 1, :, lo:n].contiguous(), v[b:b + 1, :, lo:n].contiguous()
        wo, wl = oracle.gqa_decode(bits(q[b:b + 1]), bits(kb), bits(vb), sc, 1)
        assert max_abs(o[b:b + 1].cpu().float(), from_bits(wo).float()) <= TOL, (b, n, lo)
        assert max_abs(lse[b:b + 1].cpu(), wl) <= 1e-3, (b, n, lo)
        ref = lt.sdpa_gqa_qkv(q[b:b + 1].float(), kb.float(), vb.float(), False, True)
        assert max_abs(o[b:b + 1].cpu().float(), ref) <= TOL
    # kv_lens = None with window = 0 is the plain call
    o0, _ = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits)
    full = torch.full((B,), Lmax, dtype=torch.int32, device="cuda")
    o1, _ = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits, kv_lens=full)
    assert torch.equal(o0, o1)


def test_gqa_decode_full_size_config(gpu):
    # batch 32, 32 query heads, 8 kv heads, D=128, contiguous cache of 8192 per sequence.
    B, Hq, Hkv, L, D = 32, 32, 8, 8192, 128
    torch.manual_seed(4)
    q = torch.randn(B, Hq, 1, D, device="cuda").to(torch.bfloat16)
    k = torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)
    v = torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q, k, v, scale=sc)
    # fp32 reference on the GPU (checker only), grouped instead of materialising repeat_interleave
    G = Hq // Hkv
    s = torch.einsum("bkgd,bkld->bkgl", q.view(B, Hkv, G, D).float(), k.float()) * sc
    ref_lse = torch.logsumexp(s, -1).view(B, Hq)
    ref = torch.einsum("bkgl,bkld->bkgd", torch.softmax(s, -1), v.float()).reshape(B, Hq, 1, D)
    assert max_abs(o.float(), ref) <= TOL
    assert max_abs(lse, ref_lse) <= TOL
    # two sequences against the scalar C restatement
    for b in (0, 31):
        wo, wl = oracle.gqa_decode(bits(q[b:b + 1]), bits(k[b:b + 1]), bits(v[b:b + 1]), sc, 4)
        assert max_abs(o[b:b + 1].cpu().float(), from_bits(wo).float()) <= TOL
        assert max_abs(lse[b:b + 1].cpu(), wl) <= 1e-3
    assert torch.equal(gpu.gqa_decode(q, k, v, scale=sc)[0], o)


@pytest.mark.parametrize("splits", [0, 1, 4])
def test_gqa_decode_empty_sequences(gpu, splits):
    # A sequence whose cache length is 0 attends to nothing: O = 0, LSE = -inf (the convention of the masked
    # prefill for a row without visible keys); its neighbours are unaffected.
    B, Hq, Hkv, Lmax, D = 4, 8, 2, 900, 128
    lens = [0, 900, 0, 17]
    q, = lt.make_inputs(950, (B, Hq, 1, D))
    k, v = lt.make_inputs(951, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
    sc = 1 / math.sqrt(D)
    lens_d = torch.tensor(lens, dtype=torch.int32, device="cuda")
    o, lse = gpu.gqa_decode(q.cuda(), k.cuda(), v.cuda(), scale=sc, num_splits=splits, kv_lens=lens_d)
    for b, n in enumerate(lens):
        if n == 0:
            assert torch.count_nonzero(o[b].float()) == 0 and torch.all(torch.isneginf(lse[b]))
        else:
            wo, wl = oracle.gqa_decode(bits(q[b:b + 1]), bits(k[b:b + 1, :, :n].contiguous()), bits(v[b:b + 1, :, :n].contiguous()), sc, 1)
            assert max_abs(o[b:b + 1].cpu().float(), from_bits(wo).float()) <= TOL
            assert max_abs(lse[b:b + 1].cpu(), wl) <= 1e-3


def test_gqa_decode_more_than_65535_groups(gpu):
    # (batch, kv head) groups are folded into a one-dimensional grid: their number is not limited by grid.y.
    B, Hq, Hkv, L, D = 8200, 8, 8, 40, 64
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.randn(B, Hq, 1, D, device="cuda", generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, L, D, device="cuda", generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, L, D, device="cuda", generator=g).to(torch.bfloat16)
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q, k, v, scale=sc)
    s = torch.einsum("bhd,bhld->bhl", q[:, :, 0].float(), k.float()) * sc
    ref = torch.einsum("bhl,bhld->bhd", torch.softmax(s, -1), v.float())
    assert max_abs(o[:, :, 0].float(), ref) <= TOL
    assert max_abs(lse, torch.logsumexp(s, -1)) <= TOL
    for b in (0, 8191, 8199):        # both sides of the old limit, against the scalar C restatement
        wo, wl = oracle.gqa_decode(bits(q[b:b + 1]), bits(k[b:b + 1]), bits(v[b:b + 1]), sc, 1)
        assert max_abs(o[b:b + 1].cpu().float(), from_bits(wo).float()) <= TOL


@pytest.mark.parametrize("splits", [2, 4, 8])
def test_gqa_decode_full_size_config_split_kv_and_combine(gpu, splits):
    # The same configuration through the two-pass path: split pass writing f32 partials + LSE-combine pass.
    B, Hq, Hkv, L, D = 32, 32, 8, 8192, 128
    torch.manual_seed(4)
    q = torch.randn(B, Hq, 1, D, device="cuda").to(torch.bfloat16)
    k = torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)
    v = torch.randn(B, Hkv, L, D, device="cuda").to(torch.bfloat16)
    sc = 1 / math.sqrt(D)
    o, lse = gpu.gqa_decode(q, k, v, scale=sc, num_splits=splits)
    G = Hq // Hkv
    s = torch.einsum("bkgd,bkld->bkgl", q.view(B, Hkv, G, D).float(), k.float()) * sc
    ref_lse = torch.logsumexp(s, -1).view(B, Hq)
    ref = torch.einsum("bkgl,bkld->bkgd", torch.softmax(s, -1), v.float()).reshape(B, Hq, 1, D)
    assert max_abs(o.float(), ref) <= TOL
    assert max_abs(lse, ref_lse) <= TOL
    # three sequences against the scalar C restatement run with the same number of splits
    for b in (0, 13, 31):
        wo, wl = oracle.gqa_decode(bits(q[b:b + 1]), bits(k[b:b + 1]), bits(v[b:b + 1]), sc, splits)
        assert max_abs(o[b:b + 1].cpu().float(), from_bits(wo).float()) <= TOL
        assert max_abs(lse[b:b + 1].cpu(), wl) <= 1e-3
    # split-count invariance at full size: one split (single pass) agrees within one bf16 ulp of the outputs
    o1, lse1 = gpu.gqa_decode(q, k, v, scale=sc, num_splits=1)
    assert max_abs(o.float(), o1.float()) <= 2.0 ** -7 * float(o1.float().abs().max())
    assert max_abs(lse, lse1) <= 1e-4
    assert torch.equal(gpu.gqa_decode(q, k, v, scale=sc, num_splits=splits)[0], o)      # deterministic


def test_attention_error_convention(gpu):
    from tyr_amd import TyrGpuError
    q = torch.zeros(1, 1, 16, 128, dtype=torch.bfloat16)
    with pytest.raises(TyrGpuError, match="q must be a CUDA tensor"):
        gpu.flash_attn_fwd(q, q, q)
    with pytest.raises(TyrGpuError, match="not supported"):
        z = torch.zeros(1, 1, 16, 96, dtype=torch.bfloat16).cuda()
        gpu.flash_attn_fwd(z, z, z)
    with pytest.raises(TyrGpuError, match="must have dim <= 4"):
        z = torch.zeros(1, 1, 1, 16, 128, dtype=torch.bfloat16).cuda()
        gpu.flash_attn_fwd(z, z, z)


def _scattered_key_mask(B, N, seed):
    g = torch.Generator().manual_seed(seed)
    m = torch.rand(B, N, generator=g) < 0.6
    m[0] = True                                              # one sequence without padding
    if B > 1:
        m[1, : N // 3] = False                               # left padding: causal rows there see no key at all
    return m


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B,Hq,Hkv,N,D", [(3, 4, 2, 200, 128), (2, 2, 2, 129, 64), (2, 8, 1, 64, 128), (1, 1, 1, 1, 64)])
def test_flash_attn_arbitrary_key_mask_matches_oracle(gpu, B, Hq, Hkv, N, D, causal):
    # lean_torch_sdpa_gqa_mask (cc/src/tyr.cpp:4019-4095) with holes anywhere, left padding included
    q, = lt.make_inputs(900 + N, (B, Hq, N, D))
    k, v = lt.make_inputs(901 + N, (B, Hkv, N, D), (B, Hkv, N, D))
    km = _scattered_key_mask(B, N, 902 + N)
    sc = 1.0 / math.sqrt(D)
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc, key_mask=km.cuda())
    want_o, want_lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, sc, key_mask=km.numpy())
    assert max_abs(o.cpu().float(), want_o) <= 2e-2
    dead = np.isneginf(want_lse)
    got_lse = lse.cpu().numpy()
    assert np.array_equal(np.isneginf(got_lse), dead)                       # rows that see no key: LSE = -inf ...
    assert float(o.cpu().float().numpy()[dead].__abs__().max(initial=0.0)) == 0.0   # ... and O = 0
    assert float(np.abs(got_lse[~dead] - want_lse[~dead]).max(initial=0.0)) <= 2e-2
    # uint8 masks are the same thing, and an all-visible mask is no mask
    o8, _ = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc, key_mask=km.to(torch.uint8).cuda())
    assert torch.equal(o8, o)
    o1, l1 = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc,
                                key_mask=torch.ones(B, N, dtype=torch.bool).cuda())
    o0, l0 = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc)
    assert max_abs(o1.cpu().float(), o0.cpu().float()) <= 1e-2 and max_abs(l1.cpu(), l0.cpu()) <= 1e-3


@pytest.mark.parametrize("causal", [False, True])
def test_flash_attn_key_mask_with_whole_tiles_hidden(gpu, causal):
    # key tiles of 64 rows that are wholly hidden, wholly visible (those skip the masking) or mixed, over
    # several query tiles (the paired causal schedule); forward and backward against the checker
    B, Hq, Hkv, N, D = 2, 4, 2, 448, 128
    q, g_ = lt.make_inputs(931, (B, Hq, N, D), (B, Hq, N, D))
    k, v = lt.make_inputs(932, (B, Hkv, N, D), (B, Hkv, N, D))
    km = torch.ones(B, N, dtype=torch.bool)
    km[0, 64:192] = False                  # two whole tiles
    km[0, 300:310] = False                 # a hole inside a tile
    km[1, :128] = False                    # left padding of two tiles: causal rows there see nothing
    km[1, 400:] = False                    # and a hidden tail
    sc = 1.0 / math.sqrt(D)
    o, lse = gpu.flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), causal=causal, scale=sc, key_mask=km.cuda())
    want_o, want_lse = oracle.attn_fwd_f64_ex(bits(q), bits(k), bits(v), causal, sc, key_mask=km.numpy())
    dead = np.isneginf(want_lse)
    assert max_abs(o.cpu().float(), want_o) <= 2e-2
    assert np.array_equal(np.isneginf(lse.cpu().numpy()), dead)
    assert float(np.abs(lse.cpu().numpy()[~dead] - want_lse[~dead]).max()) <= 2e-2
    dq, dk, dv = gpu.flash_attn_bwd(q.cuda(), k.cuda(), v.cuda(), o, lse, g_.cuda(), causal=causal, scale=sc,
                                    key_mask=km.cuda())
    wq, wk, wv = oracle.attn_bwd_f64_ex(bits(q), bits(k), bits(v), bits(g_), causal, sc, key_mask=km.numpy())
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        got = got.cpu().float().numpy()
        assert np.all(np.abs(got - want) <= 3e-2 + 3e-2 * np.abs(want))
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-2
    hidden = ~km.numpy()
    assert float(np.abs(dk.cpu().float().numpy()[hidden[:, None, :].repeat(Hkv, 1)]).max()) == 0.0   # hidden keys get no gradient


def test_flash_attn_key_mask_argument_checks(gpu):
    q, k, v = (t.cuda() for t in lt.make_inputs(5, (1, 2, 64, 64), (1, 2, 64, 64), (1, 2, 64, 64)))
    with pytest.raises(gpu.TyrGpuError, match="shape"):
        gpu.flash_attn_fwd(q, k, v, key_mask=torch.ones(1, 63, dtype=torch.bool).cuda())
    with pytest.raises(gpu.TyrGpuError, match="dtype"):
        gpu.flash_attn_fwd(q, k, v, key_mask=torch.ones(1, 64).cuda())
    with pytest.raises(gpu.TyrGpuError, match="CUDA"):
        gpu.flash_attn_fwd(q, k, v, key_mask=torch.ones(1, 64, dtype=torch.bool))
    with pytest.raises(gpu.TyrGpuError, match="combined"):
        gpu.flash_attn_fwd(q, k, v, window=4, key_mask=torch.ones(1, 64, dtype=torch.bool).cuda())
