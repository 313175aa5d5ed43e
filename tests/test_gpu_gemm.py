"""Parity of the gfx950 GEMM kernels (through the C ABI) with the CPU checker.

Tolerance (stated by the task): relative Frobenius error <= 1e-2 against an fp32 reference of
the rounded operands.  Small cases are also held to one bf16 ulp of the row magnitude against
the scalar C restatement, and structured operands (identity, permutation) must be bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt
from tests.util import bits, from_bits, rel_fro, u8

pytestmark = pytest.mark.gpu
TOL_FRO = 1e-2


@pytest.fixture(scope="module")
def gpu():
    import tyr_amd
    return tyr_amd


@pytest.fixture
def general_kernels():
    """Every GEMM inside the test takes the general (register-staged) kernels."""
    from tyr_amd import _lib
    L = _lib.load()
    prev = L.tyr_hip_gemm_force_general(1)
    yield
    assert L.tyr_hip_gemm_force_general(prev) == 1


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 256, 192), (256, 512, 4096), (8, 8, 8),
                                   (300, 264, 72), (1, 16, 8), (257, 8, 520), (1024, 768, 256), (768, 512, 320),
                                   (300, 264, 128), (1, 16, 64), (513, 520, 192), (700, 1000, 256),
                                   # K with a last slice shorter than 64: its chunks past K are the next row's data
                                   (64, 64, 40), (129, 80, 1000), (512, 512, 4000)])
def test_gemm_bf16_matches_oracle(gpu, M, N, K, trans_b):
    a, b = lt.make_inputs(100 + M + N + K, (M, K), (K, N), std=K ** -0.25)
    bb = b.t().contiguous() if trans_b else b
    c = gpu.gemm_bf16(a.cuda(), bb.cuda(), trans_b=trans_b).cpu()
    want_bits = oracle.gemm_bf16(bits(a), bits(bb), trans_b=trans_b)
    want = from_bits(want_bits).float()
    f32 = a.float() @ b.float()
    assert rel_fro(c, f32) <= TOL_FRO
    # accumulation order differs, so allow one bf16 ulp of the largest magnitude in the result
    assert float((c.float() - want).abs().max()) <= float(want.abs().max()) * 2 ** -7 + 1e-6


@pytest.mark.parametrize("trans_b", [False, True])
def test_gemm_bf16_identity_and_permutation_bit_exact(gpu, trans_b):
    n = 512
    a, = lt.make_inputs(7, (n, n))
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(0))
    P = torch.eye(n)[perm].to(torch.bfloat16)
    Pb = P.t().contiguous() if trans_b else P
    ab = a.t().contiguous() if trans_b else a
    got_pa = gpu.gemm_bf16(P.cuda(), ab.cuda(), trans_b=trans_b).cpu()      # rows of A permuted
    got_ap = gpu.gemm_bf16(a.cuda(), Pb.cuda(), trans_b=trans_b).cpu()      # columns of A permuted
    assert np.array_equal(bits(got_pa), bits(a[perm]))
    assert np.array_equal(bits(got_ap), bits(a[:, torch.argsort(perm)]))


@pytest.mark.parametrize("seed", range(6))
def test_gemm_random_shapes(gpu, seed):
    rng = np.random.default_rng(3000 + seed)
    M = int(rng.integers(1, 700))
    N = 16 * int(rng.integers(1, 40))
    K = 16 * int(rng.integers(1, 60))
    trans_b = bool(rng.integers(0, 2))
    a, b = lt.make_inputs(800 + seed, (M, K), (K, N), std=K ** -0.25)
    bb = b.t().contiguous() if trans_b else b
    c = gpu.gemm_bf16(a.cuda(), bb.cuda(), trans_b=trans_b).cpu()
    assert rel_fro(c, a.float() @ b.float()) <= TOL_FRO, (M, N, K, trans_b)
    aq, sa = lt.quantize_e4m3(a.float() * 8)
    bq, sb = lt.quantize_e4m3(b.float() * 8)
    bqb = bq.t().contiguous() if trans_b else bq
    c8 = gpu.gemm_fp8(aq.cuda(), bqb.cuda(), sa, sb, trans_b=trans_b).cpu()
    assert rel_fro(c8, lt.fp8_mm(aq, bq, sa, sb)) <= TOL_FRO, (M, N, K, trans_b)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("M,N,K", [(256, 256, 64), (512, 256, 192), (300, 264, 72), (1, 16, 8), (257, 8, 520)])
def test_gemm_general_kernels_match_oracle(gpu, general_kernels, M, N, K, trans_b):
    # The general (register-staged) kernels serve shapes beyond the fast kernels' 32-bit offsets;
    # the library's switch sends ordinary shapes through them.
    a, b = lt.make_inputs(100 + M + N + K, (M, K), (K, N), std=K ** -0.25)
    bb = b.t().contiguous() if trans_b else b
    c = gpu.gemm_bf16(a.cuda(), bb.cuda(), trans_b=trans_b).cpu()
    assert rel_fro(c, a.float() @ b.float()) <= TOL_FRO
    want = from_bits(oracle.gemm_bf16(bits(a), bits(bb), trans_b=trans_b)).float()
    assert (c.float() - want).abs().max() <= 2.0 ** -7 * want.abs().max()
    K8 = (K + 15) // 16 * 16
    torch.manual_seed(M + N + K8)
    a8, b8 = torch.randn(M, K8), torch.randn(K8, N - N % 16 + 16)
    aq, sa = lt.quantize_e4m3(a8)
    bq, sb = lt.quantize_e4m3(b8)
    bqb = bq.t().contiguous() if trans_b else bq
    c8 = gpu.gemm_fp8(aq.cuda(), bqb.cuda(), sa, sb, trans_b=trans_b).cpu()
    assert rel_fro(c8, lt.fp8_mm(aq, bq, sa, sb)) <= TOL_FRO


@pytest.mark.parametrize("trans_b", [False, True])
def test_gemm_rows_longer_than_the_fast_kernels_offsets(gpu, trans_b):
    # 256 rows of K elements no longer fit a 31-bit byte offset: the launcher takes the general kernel.
    M, N, K = 8, 16, 1 << 22
    g = torch.Generator().manual_seed(5)
    a = (torch.randn(M, K, generator=g) * K ** -0.25).to(torch.bfloat16)
    b = (torch.randn(K, N, generator=g) * K ** -0.25).to(torch.bfloat16)
    bb = b.t().contiguous() if trans_b else b
    c = gpu.gemm_bf16(a.cuda(), bb.cuda(), trans_b=trans_b).cpu()
    assert rel_fro(c, a.double() @ b.double()) <= TOL_FRO


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("M,N,K", [(300, 264, 128), (257, 8, 64), (1, 272, 256), (511, 504, 72)])
def test_gemm_ragged_tiles_write_only_c(gpu, M, N, K, trans_b):
    # C sits inside a larger buffer of a canary value: tiles that overhang M or N must not
    # write outside the M*N elements of C.
    from tyr_amd import _lib
    lib = _lib.load()
    a, b = lt.make_inputs(4000 + M + N + K, (M, K), (K, N), std=K ** -0.25)
    bb = b.t().contiguous() if trans_b else b
    guard = 4096
    canary = torch.full((guard + M * N + guard,), -7.0, dtype=torch.bfloat16, device="cuda")
    ad, bd = a.cuda(), bb.cuda()
    rc = lib.tyr_hip_gemm_bf16(ad.data_ptr(), bd.data_ptr(), canary.data_ptr() + 2 * guard, M, N, K,
                               int(trans_b), 0)
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((canary[:guard] == -7.0).all()) and bool((canary[guard + M * N:] == -7.0).all())
    assert torch.equal(canary[guard:guard + M * N].view(M, N), gpu.gemm_bf16(ad, bd, trans_b=trans_b))
    if N % 16 == 0 and K % 16 == 0:
        aq, sa = lt.quantize_e4m3(a.float())
        bq, sb = lt.quantize_e4m3(b.float())
        bqb = (bq.t().contiguous() if trans_b else bq).cuda()
        aqd = aq.cuda()
        canary.fill_(-7.0)
        rc = lib.tyr_hip_gemm_fp8(aqd.data_ptr(), bqb.data_ptr(), canary.data_ptr() + 2 * guard, M, N, K,
                                  float(sa), float(sb), int(trans_b), 0)
        assert rc == 0
        torch.cuda.synchronize()
        assert bool((canary[:guard] == -7.0).all()) and bool((canary[guard + M * N:] == -7.0).all())
        assert torch.equal(canary[guard:guard + M * N].view(M, N),
                           gpu.gemm_fp8(aqd, bqb, sa, sb, trans_b=trans_b))


def test_gemm_bf16_full_size_config(gpu):
    # M = N = K = 4096, entries ~ N(0, 1/sqrt(K)) (std K^-1/4), row-major A and B.
    M = N = K = 4096
    a, b = lt.make_inputs(2, (M, K), (K, N), std=K ** -0.25)
    a, b = a.cuda(), b.cuda()
    c = gpu.gemm_bf16(a, b)
    ref = a.float() @ b.float()                      # fp32 reference of the bf16-rounded inputs
    assert rel_fro(c, ref) <= TOL_FRO
    # a 64-row slab against the scalar C restatement
    rows = slice(1000, 1064)
    want = from_bits(oracle.gemm_bf16(bits(a[rows]), bits(b))).float()
    assert float((c[rows].cpu().float() - want).abs().max()) <= float(want.abs().max()) * 2 ** -7
    # linearity in a power of two is exact
    c2 = gpu.gemm_bf16((a.float() * 2).to(torch.bfloat16), b)
    assert torch.equal(c2.float(), c.float() * 2)
    # NT on the transposed operand gives the same bits as NN (same k order per output)
    cnt = gpu.gemm_bf16(a, b.t().contiguous(), trans_b=True)
    assert rel_fro(cnt, ref) <= TOL_FRO
    # determinism
    assert torch.equal(gpu.gemm_bf16(a, b), c)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (512, 256, 384), (16, 16, 16), (300, 272, 80),
                                   (1, 16, 16), (257, 48, 1040), (768, 512, 640),
                                   (300, 272, 128), (1, 16, 128), (513, 528, 384), (700, 1008, 256),
                                   # K with a last slice shorter than 128
                                   (64, 64, 48), (129, 80, 1008), (512, 512, 4000)])
def test_gemm_fp8_matches_oracle(gpu, M, N, K, trans_b):
    torch.manual_seed(200 + M + N + K)
    a, b = torch.randn(M, K), torch.randn(K, N)
    aq, sa = lt.quantize_e4m3(a)
    bq, sb = lt.quantize_e4m3(b)
    bqb = bq.t().contiguous() if trans_b else bq
    c = gpu.gemm_fp8(aq.cuda(), bqb.cuda(), sa, sb, trans_b=trans_b).cpu()
    want_bits, want_f32 = oracle.gemm_fp8(u8(aq), u8(bqb), sa, sb, trans_b=trans_b)
    ref = lt.fp8_mm(aq, bq, sa, sb)                  # fp32 GEMM of the dequantised operands
    assert rel_fro(c, ref) <= TOL_FRO
    # products of e4m3 values are exact in f32; only the summation order differs
    assert float((c.float() - torch.from_numpy(want_f32)).abs().max()) <= float(ref.abs().max()) * 2 ** -7 + 1e-6


def test_gemm_fp8_every_code_decodes_like_ocp_e4m3(gpu):
    # B = identity (1.0 = 0x38): C = decode(Aq) * sa * sb exactly (every product is exact, one term per sum)
    tab = oracle.e4m3_table()
    codes = np.array([c for c in range(256) if not np.isnan(tab[c])], dtype=np.uint8)
    A = np.zeros((256, 256), np.uint8)
    A.flat[:codes.size] = codes
    eye = np.zeros((256, 256), np.uint8)
    np.fill_diagonal(eye, 0x38)
    aq = torch.from_numpy(A).view(torch.float8_e4m3fn).cuda()
    for trans_b in (False, True):
        c = gpu.gemm_fp8(aq, torch.from_numpy(eye).view(torch.float8_e4m3fn).cuda(), 0.5, 4.0, trans_b=trans_b).cpu()
        want = torch.from_numpy(tab[A] * 2.0)            # e4m3 values are exact in bf16
        assert torch.equal(c.float(), want)              # value equality (-0 accumulates to +0)


def test_gemm_fp8_full_size_config(gpu):
    # M = N = K = 8192, values ~ N(0,1) quantised with absmax scaling.
    M = N = K = 8192
    torch.manual_seed(5)
    a = torch.randn(M, K, device="cuda")
    b = torch.randn(K, N, device="cuda")
    from tyr_amd import quantize_e4m3
    aq, sa = quantize_e4m3(a)
    bq, sb = quantize_e4m3(b)
    c = gpu.gemm_fp8(aq, bq, sa, sb)
    ref = (aq.float() @ bq.float()) * (sa * sb)      # fp32 GEMM of the dequantised operands (GPU, checker only)
    assert rel_fro(c, ref) <= TOL_FRO
    rows = slice(4000, 4016)
    _, want = oracle.gemm_fp8(u8(aq[rows]), u8(bq), sa, sb)
    assert float((c[rows].cpu().float() - torch.from_numpy(want)).abs().max()) <= float(np.abs(want).max()) * 2 ** -7
    assert torch.equal(gpu.gemm_fp8(aq, bq, sa, sb), c)


def test_error_convention(gpu):
    from tyr_amd import TyrGpuError
    a = torch.zeros(16, 16, dtype=torch.bfloat16)
    with pytest.raises(TyrGpuError, match="a must be a CUDA tensor"):
        gpu.gemm_bf16(a, a.cuda())
    with pytest.raises(TyrGpuError, match="b must be contiguous"):
        gpu.gemm_bf16(a.cuda(), torch.zeros(32, 16, dtype=torch.bfloat16).cuda()[::2])
    with pytest.raises(TyrGpuError, match="not supported"):
        gpu.gemm_bf16(torch.zeros(16, 12, dtype=torch.bfloat16).cuda(), torch.zeros(12, 16, dtype=torch.bfloat16).cuda())


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("shape,broadcast_b", [((3, 300, 264, 72), False), ((2, 5, 64, 128, 256), False),
                                               ((4, 257, 512, 64), True), ((7, 1, 16, 8), False)])
def test_batched_matmul_matches_per_entry_gemm_and_libtorch(gpu, shape, broadcast_b, trans_b):
    # `lean_torch_matmul` on operands of rank > 2 (cc/src/tyr.cpp:1565-1570): one launch for all entries,
    # bit-identical to the 2-D entry point entry by entry, and within the GEMM bar of torch.matmul in f32.
    *lead, M, N, K = shape
    a, = lt.make_inputs(9000 + M + K, (*lead, M, K), std=K ** -0.25)
    b, = lt.make_inputs(9001 + N + K, ((K, N) if broadcast_b else (*lead, K, N)), std=K ** -0.25)
    bb = b.transpose(-1, -2).contiguous() if trans_b else b
    c = gpu.matmul_bf16(a.cuda(), bb.cuda(), trans_b=trans_b).cpu()
    assert tuple(c.shape) == (*lead, M, N)
    assert rel_fro(c, torch.matmul(a.float(), b.float())) <= TOL_FRO
    a2, c2 = a.reshape(-1, M, K), c.reshape(-1, M, N)
    b2 = None if broadcast_b else bb.reshape(-1, *bb.shape[-2:])
    for i in range(a2.shape[0]):
        one = gpu.gemm_bf16(a2[i].cuda(), (bb if broadcast_b else b2[i]).cuda(), trans_b=trans_b).cpu()
        assert np.array_equal(bits(one), bits(c2[i])), i


def test_batched_matmul_through_the_general_kernels(gpu, general_kernels):
    a, = lt.make_inputs(9100, (3, 130, 72), std=72 ** -0.25)
    b, = lt.make_inputs(9101, (3, 72, 40), std=72 ** -0.25)
    c = gpu.matmul_bf16(a.cuda(), b.cuda()).cpu()
    assert rel_fro(c, torch.matmul(a.float(), b.float())) <= TOL_FRO


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("M,N,K", [(300, 272, 256), (64, 512, 512), (513, 16, 144)])
def test_fp8_gemm_row_and_column_scales_f32_out(gpu, M, N, K, trans_b):
    # tkH100Fp8ScaledGemmFwd (PrecisionGemm.lean:97-115): unscaled E4M3 mainloop, per-row x per-column dequantisation
    # scales applied to the f32 accumulators, f32 output.  Products of E4M3 values are exact in f32, so only the
    # accumulation order differs from the f32 product of the dequantised operands.
    torch.manual_seed(M + N + K)
    aq, _ = lt.quantize_e4m3(torch.randn(M, K))
    bq, _ = lt.quantize_e4m3(torch.randn(K, N))
    g = torch.Generator().manual_seed(7)
    rs, cs = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5
    bqb = bq.t().contiguous() if trans_b else bq
    want = lt.fp8_mm(aq, bq, 1.0, 1.0).double() * rs[:, None].double() * cs[None, :].double() * 0.25
    for general in (False, True):
        prev = _force_general(general)
        try:
            c = gpu.gemm_fp8_scaled(aq.cuda(), bqb.cuda(), rs.cuda(), cs.cuda(), scale=0.25, trans_b=trans_b).cpu()
        finally:
            _force_general(prev)
        assert c.dtype == torch.float32
        # (the matrix pipe aligns a 64-term dot product to its largest product before summing: ~1e-5 relative)
        assert float((c.double() - want).norm() / want.norm()) <= 1e-4, (general,)
    # one vector only, bf16 out: same arithmetic, rounded once
    c2 = gpu.gemm_fp8_scaled(aq.cuda(), bqb.cuda(), None, cs.cuda(), out_dtype=torch.bfloat16, trans_b=trans_b).cpu()
    want2 = lt.fp8_mm(aq, bq, 1.0, 1.0) * cs[None, :]
    assert rel_fro(c2, want2) <= 3e-3


def _force_general(on):
    from tyr_amd import _lib
    return _lib.load().tyr_hip_gemm_force_general(int(bool(on)))


@pytest.mark.parametrize("trans_b", [False, True])
def test_fp8_gemm_e4m3_output(gpu, trans_b):
    # tkH100Fp8E4M3GemmFwd (PrecisionGemm.lean:78-89): E4M3 in, f32 accumulate, E4M3 out (round to nearest even,
    # saturating at +-448).  Expected bytes: LibTorch's float8_e4m3fn cast of the clamped f32 product.
    M, N, K = 200, 304, 256
    torch.manual_seed(77)
    aq, _ = lt.quantize_e4m3(torch.randn(M, K))
    bq, _ = lt.quantize_e4m3(torch.randn(K, N))
    bqb = bq.t().contiguous() if trans_b else bq
    prod = lt.fp8_mm(aq, bq, 1.0, 1.0)
    for scale in (2.0 ** -12, 2.0 ** -7):                     # values inside the E4M3 range, then mostly saturated
        c = gpu.gemm_fp8_scaled(aq.cuda(), bqb.cuda(), scale=scale, out_dtype=torch.float8_e4m3fn, trans_b=trans_b).cpu()
        want = (prod * scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
        same = (c.view(torch.uint8) == want.view(torch.uint8)).float().mean()
        assert float(same) >= 0.995, float(same)              # a sum that lands on a rounding boundary may go either way
        d = (c.float() - want.float()).abs()
        # never more than one E4M3 step apart, beyond the slack of the matrix pipe's own accumulation (a 64-term dot
        # product is aligned to its largest product before it is summed; products reach 448^2, so a sum that cancels
        # to a small value carries an absolute error of up to ~16 in accumulator units)
        assert bool((d <= want.float().abs() * 2.0 ** -3 + 2.0 ** -9 + 16.0 * scale).all())
        assert float(c.float().abs().max()) <= 448.0 and not bool(torch.isnan(c.float()).any())


@pytest.mark.parametrize("trans_b", [False, True])
def test_gemms_are_reproducible_over_many_launches(gpu, trans_b):
    # bit-identical results launch after launch at sizes with many slices and several tiles per CU
    torch.manual_seed(13)
    a = (torch.randn(4096, 4096, device="cuda") * 0.125).to(torch.bfloat16)
    b = (torch.randn(4096, 4096, device="cuda") * 0.125).to(torch.bfloat16)
    first = gpu.gemm_bf16(a, b, trans_b=trans_b)
    aq, sa = gpu.quantize_e4m3(torch.randn(8192, 4096, device="cuda"))
    bq, sb = gpu.quantize_e4m3(torch.randn(4096, 8192, device="cuda"))
    bqb = bq.t().contiguous() if trans_b else bq
    first8 = gpu.gemm_fp8(aq, bqb, sa, sb, trans_b=trans_b)
    for _ in range(8):
        assert torch.equal(gpu.gemm_bf16(a, b, trans_b=trans_b), first)
        assert torch.equal(gpu.gemm_fp8(aq, bqb, sa, sb, trans_b=trans_b), first8)
