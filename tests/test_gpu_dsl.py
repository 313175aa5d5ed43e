"""Emitted tile programs on the GPU against the CPU checker, with the inputs and bars of the
reference's own runners: copy exact (Examples/GPU/RunCopy.lean:23-33), rotary allclose(1e-4, 1e-4)
(RunRotary.lean:62-66), LayerNorm out allclose(5e-3, 5e-3) and residual allclose(1e-5, 1e-5)
(RunLayerNorm.lean:66-71), attention O and LSE allclose(3e-2, 3e-2) on q,k,v [128,64], grid (1,2,1)
(RunFlashAttn.lean:79-86) plus this build's own max-abs <= 2e-2, and the example GEMM against a float64
product of the bf16 inputs (relative Frobenius <= 1e-2; the f32 result is far inside it)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt
from tests.util import bits, from_bits, max_abs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from tyr_amd.dsl import kernels, runtime
    runtime.load()
    return kernels, runtime


@pytest.mark.parametrize("block", [128, 32])
@pytest.mark.parametrize("rows,cols,grid", [(64, 64, (1, 1, 1)), (128, 192, (3, 2, 1))])
def test_copy64x64(rt, rows, cols, grid, block):
    kernels, runtime = rt
    g = torch.Generator().manual_seed(rows + cols)
    x = torch.rand(1, 1, rows, cols, generator=g).cuda()
    out = torch.zeros_like(x)
    runtime.launch(kernels.copy64x64(), [x, out], grid=grid, block=(block, 1, 1))
    torch.cuda.synchronize()
    assert torch.equal(out, x)


def test_rotaryFwd(rt):
    kernels, runtime = rt
    g = torch.Generator().manual_seed(7)
    x = torch.rand(64, 64, generator=g)
    cos, sin = lt.compute_rotary_freqs(64, 64)
    want = oracle.rope(x.reshape(1, 64, 1, 64).numpy(), cos.numpy(), sin.numpy()).reshape(64, 64)
    out = torch.zeros(64, 64).cuda()
    runtime.launch(kernels.rotaryFwd(), [x.cuda(), sin.cuda().contiguous(), cos.cuda().contiguous(), out, 64, 64],
                   grid=(1, 1, 1), block=(128, 1, 1))
    torch.cuda.synchronize()
    assert torch.allclose(out.cpu(), torch.from_numpy(want), rtol=1e-4, atol=1e-4)
    assert float((out.cpu() - torch.from_numpy(want)).abs().max()) <= 1e-6


@pytest.mark.parametrize("block", [32, 128])     # the runner's single warp, and four waves sharing the LDS tile
@pytest.mark.parametrize("rows", [64, 192])
def test_tkFusedLayerNormResidual1024(rt, rows, block):
    kernels, runtime = rt
    g = torch.Generator().manual_seed(rows)
    x = torch.rand(1, rows, 1024, generator=g).bfloat16()
    res = torch.rand(1, rows, 1024, generator=g).bfloat16()
    w = torch.rand(1024, generator=g).bfloat16()
    b = torch.rand(1024, generator=g).bfloat16()
    want_out, want_resid = oracle.layernorm_residual(bits(x).reshape(rows, 1024), bits(res).reshape(rows, 1024),
                                                     bits(w), bits(b), 1e-5)
    out, out_resid = torch.zeros_like(x).cuda(), torch.zeros_like(x).cuda()
    runtime.launch(kernels.tkFusedLayerNormResidual1024(), [x.cuda(), res.cuda(), w.cuda(), b.cuda(), out, out_resid],
                   grid=(1, rows // 64, 1), block=(block, 1, 1))
    torch.cuda.synchronize()
    got_out, got_resid = out.cpu().float().reshape(rows, 1024), out_resid.cpu().float().reshape(rows, 1024)
    assert torch.allclose(got_resid, from_bits(want_resid).float(), rtol=1e-5, atol=1e-5)
    assert torch.allclose(got_out, from_bits(want_out).float(), rtol=5e-3, atol=5e-3)


@pytest.mark.parametrize("M,N", [(64, 64), (128, 192)])
def test_simpleGemm(rt, M, N):
    kernels, runtime = rt
    K = 512                                                     # 8 K blocks of 64
    a, b = lt.make_inputs(3, (M, K), (K, N), std=K ** -0.25)
    c = torch.zeros(M, N).cuda()
    runtime.launch(kernels.simpleGemm(), [a.cuda(), b.cuda(), c, M, N, K], grid=(N // 64, M // 64, 1),
                   block=(128, 1, 1))
    torch.cuda.synchronize()
    want = a.double() @ b.double()
    rel = float((c.cpu().double() - want).norm() / want.norm())
    assert rel <= 1e-2 and rel <= 1e-5, rel


def test_tkFlashAttnFwd2BlockLse(rt):
    kernels, runtime = rt
    q, k, v = lt.make_inputs(11, (128, 64), (128, 64), (128, 64))
    o = torch.zeros(128, 64, dtype=torch.bfloat16).cuda()
    lse = torch.zeros(128).cuda()
    runtime.launch(kernels.tkFlashAttnFwd2BlockLse(), [q.cuda(), k.cuda(), v.cuda(), o, lse, 128, 64],
                   grid=(1, 2, 1), block=(128, 1, 1))
    torch.cuda.synchronize()
    want_o, want_lse = oracle.attn_fwd_f64(bits(q).reshape(1, 1, 128, 64), bits(k).reshape(1, 1, 128, 64),
                                           bits(v).reshape(1, 1, 128, 64), False, 0.125)
    want_o, want_lse = torch.from_numpy(want_o).reshape(128, 64).float(), torch.from_numpy(want_lse).reshape(128).float()
    assert torch.allclose(o.cpu().float(), want_o, rtol=3e-2, atol=3e-2)
    assert torch.allclose(lse.cpu(), want_lse, rtol=3e-2, atol=3e-2)
    assert float((o.cpu().float() - want_o).abs().max()) <= 2e-2
    assert float((lse.cpu() - want_lse).abs().max()) <= 2e-2


def test_launcher_rejects_bad_arguments(rt):
    kernels, runtime = rt
    x = torch.zeros(64, 64).cuda()
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        runtime.launch(kernels.copy64x64(), [torch.zeros(64, 64), x])
    with pytest.raises(RuntimeError, match="input must be contiguous"):
        runtime.launch(kernels.copy64x64(), [torch.zeros(64, 128).cuda()[:, ::2], x])
    with pytest.raises(RuntimeError, match="output must have dim <= 4"):
        runtime.launch(kernels.copy64x64(), [x, torch.zeros(1, 1, 1, 64, 64).cuda()])
    with pytest.raises(RuntimeError, match="invalid launch arguments"):
        runtime.launch(kernels.copy64x64(), [x, x.clone()], block=(1024, 1, 1))


def test_mha_h100_forward_prep_and_backward_programs(rt):
    """The sequence of Examples/GPU/RunMhaH100.lean:103-147 on q, k, v, dO [1,1,128,64]: both forward
    programs agree on L = -8 LSE, the prep program gives d = rowsum(dO * O), the backward program gives
    dQ and per-(kv tile, q tile) partials of dK and dV that are summed over q tiles on the host; all
    against the float64 checker at the runner's allclose(3e-2, 3e-2)."""
    kernels, runtime = rt
    q, k, v, dO = lt.make_inputs(21, (1, 1, 128, 64), (1, 1, 128, 64), (1, 1, 128, 64), (1, 1, 128, 64))
    geo = dict(grid=(1, 2, 1), block=(128, 1, 1))
    qc, kc, vc, dOc = (t.cuda() for t in (q, k, v, dO))

    out_lse, lse = torch.zeros_like(qc), torch.zeros(2, 64).cuda()
    runtime.launch(kernels.tkFlashAttnFwd2BlockLse(), [qc, kc, vc, out_lse, lse, 128, 64], **geo)
    out_plain = torch.zeros_like(qc)
    runtime.launch(kernels.tkFlashAttnFwd2Block(), [qc, kc, vc, out_plain, 128, 64], **geo)
    out, l_out = torch.zeros_like(qc), torch.zeros(2, 64).cuda()
    runtime.launch(kernels.tkMhaH100Fwd2Block(), [qc, kc, vc, out, l_out, 128, 64], **geo)
    d_vec = torch.zeros(2, 64).cuda()
    runtime.launch(kernels.tkMhaH100BwdPrep2Block(), [dOc, out, d_vec, 128, 64], **geo)
    dQ = torch.zeros(1, 1, 128, 64).cuda()
    dK_part, dV_part = torch.zeros(1, 1, 128, 128).cuda(), torch.zeros(1, 1, 128, 128).cuda()
    runtime.launch(kernels.tkMhaH100Bwd2BlockPartials(), [qc, kc, vc, dOc, l_out, d_vec, dQ, dK_part, dV_part, 128, 64],
                   **geo)
    torch.cuda.synchronize()
    dK = dK_part.reshape(1, 1, 2, 64, 2, 64).sum(4).reshape(1, 1, 128, 64).cpu()
    dV = dV_part.reshape(1, 1, 2, 64, 2, 64).sum(4).reshape(1, 1, 128, 64).cpu()

    want_o, want_lse = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), False, 0.125)
    want_dq, want_dk, want_dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(dO), False, 0.125)
    T = torch.from_numpy
    close = lambda a, b: torch.allclose(a.cpu().float(), b.float(), rtol=3e-2, atol=3e-2)
    assert torch.equal(out, out_lse) and torch.equal(out, out_plain)          # the three forwards share their O path
    assert close(out, T(want_o))
    assert close(l_out.reshape(128), -8.0 * T(want_lse).reshape(128))
    assert torch.allclose(l_out, -8.0 * lse, rtol=0, atol=1e-5)                # the runner's cross-check of the two L paths
    want_d = (dO.float() * out.cpu().float()).sum(-1).reshape(2, 64)
    assert torch.allclose(d_vec.cpu(), want_d, rtol=1e-5, atol=1e-5)
    assert close(dQ, T(want_dq)) and close(dK, T(want_dk)) and close(dV, T(want_dv))
    for got, want in ((dQ.cpu(), T(want_dq)), (dK, T(want_dk)), (dV, T(want_dv))):
        assert float((got.double() - want.double()).norm() / want.double().norm()) <= 1e-2


def test_mha_h100_seq768_forward_prep_and_backward_programs(rt):
    """Examples/GPU/RunMhaH100Seq768.lean:100-136 on q, k, v, dO [1,1,768,64]: the 12-block forwards, the prep
    program and the 12-block backward with its dK / dV partials summed over the 12 query tiles on the host, at the
    runner's bars (allclose 5e-2 forward, 8e-2 backward) and at a relative Frobenius error of 1e-2."""
    kernels, runtime = rt
    q, k, v, dO = lt.make_inputs(23, (1, 1, 768, 64), (1, 1, 768, 64), (1, 1, 768, 64), (1, 1, 768, 64))
    geo = dict(grid=(1, 12, 1), block=(128, 1, 1))
    qc, kc, vc, dOc = (t.cuda() for t in (q, k, v, dO))
    out_lse, lse = torch.zeros_like(qc), torch.zeros(12, 64).cuda()
    runtime.launch(kernels.tkFlashAttnFwd12BlockLse(), [qc, kc, vc, out_lse, lse, 768, 64], **geo)
    out_plain = torch.zeros_like(qc)
    runtime.launch(kernels.tkFlashAttnFwd12Block(), [qc, kc, vc, out_plain, 768, 64], **geo)
    out, l_out = torch.zeros_like(qc), torch.zeros(12, 64).cuda()
    runtime.launch(kernels.tkMhaH100Fwd12Block(), [qc, kc, vc, out, l_out, 768, 64], **geo)
    d_vec = torch.zeros(12, 64).cuda()
    runtime.launch(kernels.tkMhaH100BwdPrep2Block(), [dOc, out, d_vec, 768, 64], **geo)
    dQ = torch.zeros(1, 1, 768, 64).cuda()
    dK_part, dV_part = torch.zeros(1, 1, 768, 768).cuda(), torch.zeros(1, 1, 768, 768).cuda()
    runtime.launch(kernels.tkMhaH100Bwd12BlockPartials(), [qc, kc, vc, dOc, l_out, d_vec, dQ, dK_part, dV_part, 768, 64],
                   **geo)
    torch.cuda.synchronize()
    dK = dK_part.reshape(1, 1, 12, 64, 12, 64).sum(4).reshape(1, 1, 768, 64).cpu()
    dV = dV_part.reshape(1, 1, 12, 64, 12, 64).sum(4).reshape(1, 1, 768, 64).cpu()
    want_o, want_lse = oracle.attn_fwd_f64(bits(q), bits(k), bits(v), False, 0.125)
    want_dq, want_dk, want_dv = oracle.attn_bwd_f64(bits(q), bits(k), bits(v), bits(dO), False, 0.125)
    T = torch.from_numpy
    close = lambda a, b, tol: torch.allclose(a.cpu().float(), b.float(), rtol=tol, atol=tol)
    assert torch.equal(out, out_lse) and torch.equal(out, out_plain)
    assert close(out, T(want_o), 5e-2) and close(out, T(want_o), 2e-2)
    assert close(l_out.reshape(768), -8.0 * T(want_lse).reshape(768), 5e-2)
    assert torch.allclose(l_out, -8.0 * lse, rtol=0, atol=1e-4)
    assert close(dQ, T(want_dq), 8e-2) and close(dK, T(want_dk), 8e-2) and close(dV, T(want_dv), 8e-2)
    for got, want in ((dQ.cpu(), T(want_dq)), (dK, T(want_dk)), (dV, T(want_dv))):
        assert float((got.double() - want.double()).norm() / want.double().norm()) <= 1e-2


@pytest.mark.parametrize("name,D", [("tkMhaH100LCFFwd64", 64), ("tkMhaH100LCFFwd128", 128)])
def test_mha_h100_lcf_forward_programs(rt, name, D):
    """Tyr/GPU/Kernels/MhaH100LCF.lean:84-132: a stationary 64 x D query tile against 3072 streamed keys (16 tiles of
    192 rows at D = 64, 24 tiles of 128 rows at D = 128), non-causal.  The program is run by a group of two waves
    (64 threads of the reference = 2 warps), K and V staying in LDS.  Checked against softmax(Q K^T scale) V in
    float64 on the same bf16 inputs at the attention bar."""
    kernels, runtime = rt
    nq, nkv = 192, 3072
    q, k, v = lt.make_inputs(41 + D, (1, 1, nq, D), (1, 1, nkv, D), (1, 1, nkv, D))
    o = torch.zeros(1, 1, nq, D, dtype=torch.bfloat16).cuda()
    runtime.launch(getattr(kernels, name)(), [q.cuda(), k.cuda(), v.cuda(), o, nkv, D], grid=(1, nq // 64, 1), block=(64, 1, 1))
    torch.cuda.synchronize()
    sc = 0.125 if D == 64 else 0.08838834764
    p = torch.softmax(q[0, 0].double() @ k[0, 0].double().T * sc, -1)
    want = p @ v[0, 0].double()
    assert max_abs(o[0, 0].cpu().float(), want) <= 2e-2
    assert float((o[0, 0].cpu().double() - want).norm() / want.norm()) <= 1e-2
    # the compiled program is a group of exactly two waves: the launcher starts two, whatever block shape it is given
    # (every warp of the reference's block repeats the whole tile program, so the result does not depend on it)
    o2 = torch.zeros_like(o)
    runtime.launch(getattr(kernels, name)(), [q.cuda(), k.cuda(), v.cuda(), o2, nkv, D], grid=(1, nq // 64, 1), block=(128, 1, 1))
    torch.cuda.synchronize()
    assert torch.equal(o, o2)


@pytest.mark.parametrize("M,N", [(128, 256), (384, 1024)])
def test_tkH100Bf16GemmFwd(rt, M, N):
    """Tyr/GPU/Kernels/Bf16Gemm.lean:64-73: C[128 x 256 tiles] = A[M, 256] B[N, 256]^T, f32 accumulate, bf16 out; the
    128 x 256 accumulator is held by a group of four waves (32 rows each), B is read from LDS by the products."""
    kernels, runtime = rt
    K = 256                                                  # 4 slices of 64, fixed by the program
    a, b = lt.make_inputs(51, (M, K), (N, K), std=K ** -0.25)
    c = torch.zeros(M, N, dtype=torch.bfloat16).cuda()
    runtime.launch(kernels.tkH100Bf16GemmFwd(), [a.cuda(), b.cuda(), c, M, N, K], grid=(N // 256, M // 128, 1),
                   block=(128, 1, 1))
    torch.cuda.synchronize()
    want = from_bits(oracle.gemm_bf16(bits(a), bits(b), trans_b=True)).float()
    got = c.cpu().float()
    assert float((got - a.float() @ b.float().T).norm() / (a.float() @ b.float().T).norm()) <= 1e-2
    assert (got - want).abs().max() <= 2.0 ** -7 * want.abs().max()


def _fp8_inputs(seed, M, N, K):
    torch.manual_seed(seed)
    aq, sa = lt.quantize_e4m3(torch.randn(M, K))
    bq, sb = lt.quantize_e4m3(torch.randn(N, K))          # B is N x K (the reference's tiledAccumulator layout)
    return aq, sa, bq, sb


@pytest.mark.parametrize("M,N", [(64, 256), (192, 512)])
def test_gemmFp8E4M3Fwd(rt, M, N):
    kernels, runtime = rt
    K = 512                                                  # 4 slices of 128
    aq, _, bq, _ = _fp8_inputs(31, M, N, K)
    c = torch.zeros(M, N, dtype=torch.bfloat16).cuda()
    runtime.launch(kernels.gemmFp8E4M3Fwd(), [aq.cuda(), bq.cuda(), c, M, N, K], grid=(N // 256, M // 64, 1),
                   block=(128, 1, 1))
    torch.cuda.synchronize()
    want_bits, want_f32 = oracle.gemm_fp8(aq.view(torch.uint8).numpy(), bq.view(torch.uint8).numpy(), 1.0, 1.0, trans_b=True)
    # products of E4M3 values are exact in f32 and K = 512 terms stay far below 2^24 ulps: the f32 sums differ
    # only by accumulation order, so nearly every bf16 output is bit-identical; the bar is the GEMM tolerance
    got = c.cpu().float()
    rel = float((got - torch.from_numpy(want_f32)).norm() / np.linalg.norm(want_f32))
    assert rel <= 1e-2 and rel <= 3e-3, rel
    want_bf, wf = from_bits(want_bits).float(), torch.from_numpy(want_f32)
    # per element: half a bf16 ulp of rounding plus the slack of the matrix pipe's own accumulation (a 64-term dot
    # product is aligned to its largest product before it is summed; terms reach 448^2 = 2e5)
    assert bool(((got - wf).abs() <= wf.abs() * 2.0 ** -8 * 1.01 + 16.0).all())
    assert float((got != want_bf).float().mean()) <= 0.05                                # bit-identical for more than 95 % of the outputs


def test_tkH100Fp8ScaledGemmFwd(rt):
    kernels, runtime = rt
    M, N, K = 128, 512, 512
    aq, _, bq, _ = _fp8_inputs(32, M, N, K)
    g = torch.Generator().manual_seed(33)
    sa, sb = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5
    c = torch.zeros(M, N).cuda()
    runtime.launch(kernels.tkH100Fp8ScaledGemmFwd(), [aq.cuda(), bq.cuda(), sa.cuda(), sb.cuda(), c, M, N, K],
                   grid=(N // 256, M // 64, 1), block=(128, 1, 1))
    torch.cuda.synchronize()
    _, want_f32 = oracle.gemm_fp8(aq.view(torch.uint8).numpy(), bq.view(torch.uint8).numpy(), 1.0, 1.0, trans_b=True)
    want = torch.from_numpy(want_f32) * sa[:, None] * sb[None, :]
    rel = float((c.cpu() - want).norm() / want.norm())
    assert rel <= 1e-4, rel                                   # f32 accumulation order is the only difference


# ------------------------------------------------------------------ the reference's demonstration programs with makeCausal
def _causal_demo_reference(q, k, v, explicit_softmax):
    """What `flashAttnFwdNew` / `flashAttnFwdWithLse` (FlashAttn.lean:26-95, FlashAttnBwd.lean:25-103) and `flashAttnFwd`
    (Examples.lean:93-144) compute for one 64-row query tile, statement by statement in float64 on the bf16 inputs: no score
    scale, the causal mask inside every 64 x 64 tile (fill -1e10), and a score tile that is never cleared -- the scores of KV
    block j start from the probabilities of block j-1 (zeros for block 0, the value-initialised tile).  P is rounded to bf16
    before P V, as `convert p s` does."""
    q, k, v = q.double(), k.double(), v.double()
    s = torch.zeros(64, 64, dtype=torch.float64)
    o = torch.zeros(64, 64, dtype=torch.float64)
    row_max = torch.full((64,), -float("inf"), dtype=torch.float64)
    row_sum = torch.zeros(64, dtype=torch.float64)
    keep = torch.ones(64, 64, dtype=torch.bool).tril()
    for j in range(4):
        s = q @ k[64 * j:64 * j + 64].T + s
        s = torch.where(keep, s, torch.full_like(s, -1e10))
        prev = row_max
        row_max = torch.maximum(row_max, s.max(dim=1).values)
        if not explicit_softmax:                              # onlineSoftmax rescales what it has accumulated
            scale = torch.exp(prev - row_max)
            o = o * scale[:, None]
            row_sum = row_sum * scale
        s = torch.exp(s - row_max[:, None])
        row_sum = row_sum + s.sum(dim=1)
        o = o + s.bfloat16().double() @ v[64 * j:64 * j + 64]
    return o / row_sum[:, None], torch.log(row_sum) + row_max


@pytest.mark.parametrize("name", ["flashAttnFwdNew", "flashAttnFwdWithLse", "flashAttnFwd"])
def test_causal_demonstration_forwards(rt, name):
    kernels, runtime = rt
    # small scores (inputs of std 0.3), as unscaled 64-term dot products of N(0,1) values would saturate the softmax
    q, k, v = lt.make_inputs(71, (128, 64), (256, 64), (256, 64), std=0.3)
    o = torch.zeros(128, 64, dtype=torch.bfloat16).cuda()
    lse = torch.zeros(128).cuda()
    args = [q.cuda(), k.cuda(), v.cuda(), o] + ([lse] if name == "flashAttnFwdWithLse" else []) + [256, 64]
    runtime.launch(getattr(kernels, name)(), args, grid=(1, 2, 1), block=(32, 1, 1))
    torch.cuda.synchronize()
    for t in range(2):                                        # query tile t (the KV tiles are the same four for both)
        want_o, want_lse = _causal_demo_reference(q[64 * t:64 * t + 64], k, v, explicit_softmax=(name == "flashAttnFwd"))
        got = o[64 * t:64 * t + 64].cpu().float()
        assert torch.allclose(got, want_o.float(), rtol=3e-2, atol=3e-2), (name, t)
        assert max_abs(got, want_o) <= 2e-2, (name, t)
        if name == "flashAttnFwdWithLse":
            assert max_abs(lse[64 * t:64 * t + 64].cpu(), want_lse) <= 2e-2, (name, t)


def test_simpleGemmNew(rt):
    kernels, runtime = rt
    M, N, K = 128, 192, 512
    a, b = lt.make_inputs(4, (M, K), (K, N), std=K ** -0.25)
    c = torch.zeros(M, N).cuda()
    runtime.launch(kernels.simpleGemmNew(), [a.cuda(), b.cuda(), c, M, N, K], grid=(N // 64, M // 64, 1), block=(32, 1, 1))
    torch.cuda.synchronize()
    want = a.double() @ b.double()
    assert float((c.cpu().double() - want).norm() / want.norm()) <= 1e-5


def test_tkH100Fp8E4M3GemmFwd(rt):
    """PrecisionGemm.lean:73-89: E4M3 x E4M3 -> f32 -> E4M3.  Inputs are scaled so that the results lie inside the E4M3
    range; every output must be the E4M3 rounding of its f32 sum (ties and the pipe's accumulation order leave a code of
    slack on a few elements)."""
    kernels, runtime = rt
    M, N, K = 128, 512, 512
    torch.manual_seed(34)
    aq = (torch.randn(M, K) * 0.5).to(torch.float8_e4m3fn)
    bq = (torch.randn(N, K) * 0.5).to(torch.float8_e4m3fn)
    c = torch.zeros(M, N, dtype=torch.uint8).cuda().view(torch.float8_e4m3fn)
    runtime.launch(kernels.tkH100Fp8E4M3GemmFwd(), [aq.cuda(), bq.cuda(), c, M, N, K], grid=(N // 256, M // 64, 1),
                   block=(32, 1, 1))
    torch.cuda.synchronize()
    _, want_f32 = oracle.gemm_fp8(aq.view(torch.uint8).numpy(), bq.view(torch.uint8).numpy(), 1.0, 1.0, trans_b=True)
    wf = torch.from_numpy(want_f32)
    assert float(wf.abs().max()) < 448.0
    got = c.cpu().float()
    want = wf.to(torch.float8_e4m3fn).float()
    assert float((got != want).float().mean()) <= 0.02
    assert bool(((got - wf).abs() <= wf.abs() * 2.0 ** -3 + 2.0 ** -9).all())          # never more than one code away
    rel = float((got - wf).norm() / wf.norm())
    assert rel <= 4e-2, rel                                   # E4M3 keeps 3 mantissa bits: rounding alone is ~2.5e-2


@pytest.mark.parametrize("M,N", [(128, 256), (256, 768)])
def test_tkB200Fp8E4M3Gemm1CtaFwd(rt, M, N):
    """PrecisionGemm.lean:117-133: E4M3 x E4M3 -> f32 -> bf16 on 128 x 256 tiles, run by a group of four waves with the
    E4M3 B tile read from LDS by the products."""
    kernels, runtime = rt
    K = 512
    aq, _, bq, _ = _fp8_inputs(35, M, N, K)
    c = torch.zeros(M, N, dtype=torch.bfloat16).cuda()
    runtime.launch(kernels.tkB200Fp8E4M3Gemm1CtaFwd(), [aq.cuda(), bq.cuda(), c, M, N, K], grid=(N // 256, M // 128, 1),
                   block=(128, 1, 1))
    torch.cuda.synchronize()
    want_bits, want_f32 = oracle.gemm_fp8(aq.view(torch.uint8).numpy(), bq.view(torch.uint8).numpy(), 1.0, 1.0, trans_b=True)
    got, wf = c.cpu().float(), torch.from_numpy(want_f32)
    rel = float((got - wf).norm() / wf.norm())
    assert rel <= 1e-2 and rel <= 3e-3, rel
    assert bool(((got - wf).abs() <= wf.abs() * 2.0 ** -8 * 1.01 + 16.0).all())
    assert float((got != from_bits(want_bits).float()).float().mean()) <= 0.05
